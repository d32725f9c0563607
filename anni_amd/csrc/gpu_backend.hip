/*
** libanni_gpu_hip.so -- the optimizer-step subset of AnnI's backend C ABI
** (num/gpu.h) on MI355X.  See include/anni_gpu.h for the contract of each entry
** point and the reference line it stands in for.
*/
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>
#include <vector>
#include "adam_kernels.h"
#include "anni_gpu.h"
#include "backend_state.h"
#include "busy_flag.h"
#include "placement.h"
#include "pool_chunks.h"

namespace anni {

static std::once_flag g_init_once;
static bool g_ready;
static hipStream_t g_own_stream;
static hipStream_t g_stream;
static std::mutex g_mu;			/* guards everything below */
static char g_err[256];
static std::mutex g_pool_mu;		/* guards gpu_malloc's pools; never taken with g_mu held */

static void init_once(void)
{
	int n = 0;
	const char *off = getenv("ANNI_GPU_DISABLE");

	if (off && off[0] == '1')
		return;
	if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
		(void)hipGetLastError();
		return;
	}
	/* A blocking stream: synchronous hipMemcpy calls order themselves with it. */
	if (hipStreamCreate(&g_own_stream) != hipSuccess) {
		(void)hipGetLastError();
		return;
	}
	g_stream = g_own_stream;
	g_ready = true;
}

bool device_ready(void)
{
	std::call_once(g_init_once, init_once);
	return g_ready;
}

static void batch_flush(void);
static std::atomic<int> g_batch_dir;	/* written with g_mu held; read without it to see whether anything is pending */

hipStream_t compute_stream(void)
{
	if (g_batch_dir != 0)
		batch_flush();		/* pending small copies go first (see "small copies, batched") */
	return g_stream;
}

void set_compute_stream(hipStream_t st)
{
	g_stream = st ? st : g_own_stream;
}

/* The same with g_mu already held (the mutex is not recursive). */
static bool hip_ok_locked(hipError_t err, const char *what)
{
	if (err == hipSuccess)
		return true;
	if (!g_err[0])
		snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(err));
	return false;
}

bool hip_ok(hipError_t err, const char *what)
{
	if (err == hipSuccess)
		return true;
	std::lock_guard<std::mutex> lk(g_mu);
	return hip_ok_locked(err, what);
}

/* ---- small copies, batched ------------------------------------------------- */

/*
** lang/lm_adam.c moves every bias / LayerNorm vector with its own gpu_memcpy_h2d before the
** step and its own gpu_memcpy_d2h_async after it (lm_adam.c:372-377,407-413): 146 + 73 copies
** of a few KiB per step at the reference's 185M size (170 + 85 at 555M, the head bias of 400 KB
** among them), more time than the two kernels when each is a copy of its own.  Copies of
** kSmallCopy bytes or less are therefore batched: an H2D is copied into a page-locked staging
** ring at once (the caller may reuse its buffer on return, as with a pageable cudaMemcpyAsync)
** and described in a table, one entry per piece of kPieceBytes; a kernel with one workgroup per
** piece moves the batch.  That kernel is launched as soon as kFlushBytes are waiting -- it pulls
** them over the host link while the caller is still staging the next vectors -- and at the
** latest by the next operation on the stream.  A small async D2H is gathered the same way into
** the ring and handed to its host destination at the next synchronisation, which is when the
** contract makes it visible (num/gpu.h:44-47).  Order on the stream is kept because every entry
** point puts the pending batch on the stream before it enqueues anything.
** ANNI_SMALL_COPY_BATCH=0 switches the batching off.
*/
struct CopyDesc {
	void		*dev;
	unsigned long long	stage_off;
	unsigned long long	nbytes;
};

static const size_t kSmallCopy = (size_t)1 << 20;
static const size_t kPieceBytes = (size_t)16 << 10;	/* a multiple of 16: every piece keeps the copy's alignment */
static const size_t kFlushBytes = (size_t)256 << 10;
static const size_t kStageBytes = (size_t)16 << 20;
static const int kDescSlots = 8192;
static char *g_stage;			/* page-locked, device-visible */
static CopyDesc *g_desc;		/* page-locked, device-visible */
static size_t g_stage_used;		/* bump pointers; reset after every full synchronisation */
static int g_desc_used;
static int g_batch_first;		/* descriptors [g_batch_first, g_desc_used) are not launched yet */
static size_t g_batch_bytes;		/* what they move */
/* g_batch_dir (declared above): 0 none, 1 host-to-device, 2 device-to-host */
struct Delivery {
	void	*host;
	size_t	stage_off;
	size_t	nbytes;
};
static Delivery g_deliver[kDescSlots];	/* gathered D2H data waiting for a synchronisation */
static int g_deliver_n;

/*
** One workgroup per piece.  The staging side of every copy is placed at the same offset from
** a 16-byte boundary as its device side (batch_add_locked), so after at most 15 leading bytes
** both run in 16-byte steps, four of them in flight per lane: a bias / LayerNorm vector of a few
** KiB is one round, a long vector is spread over many workgroups.  (Byte by byte the same batch
** spent 0.3 ms of a 1.6 ms step waiting on the host link, one round trip after the other; one
** workgroup per 400 KB vector pulled it at a third of the link's rate.)
*/
__global__ __launch_bounds__(256) void small_copy_kernel(const CopyDesc *desc, char *stage,
	int to_device)
{
	const CopyDesc d = desc[blockIdx.x];
	char *dev = (char *)d.dev;
	char *stg = stage + d.stage_off;
	char *dst = to_device ? dev : stg;
	const char *src = to_device ? stg : dev;
	const size_t lead = (16 - ((uintptr_t)dev & 15)) & 15;
	const size_t head = lead < d.nbytes ? lead : d.nbytes;
	const size_t body = (d.nbytes - head) / 16;
	const size_t tail = head + body * 16;
	const uint4 *s16 = (const uint4 *)(src + head);
	uint4 *d16 = (uint4 *)(dst + head);

	static_assert(kPieceBytes == 4 * 256 * 16, "a piece is four 16-byte accesses per lane");
	if (threadIdx.x < head)
		dst[threadIdx.x] = src[threadIdx.x];
	if (body >= 1024) {
		uint4 w[4];

#pragma unroll
		for (int u = 0; u < 4; u++)
			w[u] = s16[threadIdx.x + u * 256];
#pragma unroll
		for (int u = 0; u < 4; u++)
			d16[threadIdx.x + u * 256] = w[u];
		for (size_t i = 1024 + threadIdx.x; i < body; i += 256)
			d16[i] = s16[i];
	} else {
		for (size_t i = threadIdx.x; i < body; i += 256)
			d16[i] = s16[i];
	}
	if (tail + threadIdx.x < d.nbytes)
		dst[tail + threadIdx.x] = src[tail + threadIdx.x];
}

static bool batch_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANNI_SMALL_COPY_BATCH");

		on = (e && e[0] == '0') ? 0 : 1;
		if (on) {
			void *a = nullptr, *b = nullptr;

			if (hipHostMalloc(&a, kStageBytes, hipHostMallocDefault) != hipSuccess
			    || hipHostMalloc(&b, sizeof(CopyDesc) * kDescSlots, hipHostMallocDefault)
			    != hipSuccess) {
				(void)hipGetLastError();
				on = 0;
			} else {
				g_stage = (char *)a;
				g_desc = (CopyDesc *)b;
			}
		}
	}
	return on == 1;
}

/* Launches the pending batch.  g_mu held. */
static void batch_flush_locked(void)
{
	const int count = g_desc_used - g_batch_first;

	if (count > 0) {
		hipLaunchKernelGGL(small_copy_kernel, dim3(count), dim3(256), 0, g_stream,
		    g_desc + g_batch_first, g_stage, g_batch_dir == 1 ? 1 : 0);
		(void)hip_ok_locked(hipGetLastError(), "small copy batch");
	}
	g_batch_first = g_desc_used;
	g_batch_bytes = 0;
	g_batch_dir = 0;
}

/* After the stream has drained: hand gathered data to its host destinations, recycle the rings.  g_mu held. */
static void batch_deliver_locked(void)
{
	for (int i = 0; i < g_deliver_n; i++)
		memcpy(g_deliver[i].host, g_stage + g_deliver[i].stage_off, g_deliver[i].nbytes);
	g_deliver_n = 0;
	g_stage_used = 0;
	g_desc_used = 0;
	g_batch_first = 0;
	g_batch_bytes = 0;
}

/* Queues one small copy; false = does not qualify (the caller copies the ordinary way).  g_mu held. */
static bool batch_add_locked(int dir, void *dev, void *host, size_t nbytes)
{
	const size_t skew = (uintptr_t)dev & 15;	/* staging keeps the device side's alignment */
	const size_t need = (skew + nbytes + 255) / 256 * 256;
	const int pieces = (int)((nbytes + kPieceBytes - 1) / kPieceBytes);
	size_t at;

	if (nbytes > kSmallCopy || !batch_on())
		return false;
	if (g_batch_dir != 0 && g_batch_dir != dir)
		batch_flush_locked();
	if (g_stage_used + need > kStageBytes || g_desc_used + pieces > kDescSlots
	    || g_deliver_n == kDescSlots) {
		/* rings full: drain everything, then start over */
		batch_flush_locked();
		if (hipStreamSynchronize(g_stream) != hipSuccess)
			return false;
		batch_deliver_locked();
	}
	at = g_stage_used + skew;
	for (size_t done = 0; done < nbytes; done += kPieceBytes) {
		g_desc[g_desc_used].dev = (char *)dev + done;
		g_desc[g_desc_used].stage_off = at + done;
		g_desc[g_desc_used].nbytes = nbytes - done < kPieceBytes ? nbytes - done : kPieceBytes;
		g_desc_used++;
	}
	if (dir == 1) {
		memcpy(g_stage + at, host, nbytes);
	} else {
		g_deliver[g_deliver_n].host = host;
		g_deliver[g_deliver_n].stage_off = at;
		g_deliver[g_deliver_n].nbytes = nbytes;
		g_deliver_n++;
	}
	g_stage_used += need;
	g_batch_bytes += nbytes;
	g_batch_dir = dir;
	/* enough for a launch of its own: the device pulls it while the caller stages the next vectors */
	if (dir == 1 && g_batch_bytes >= kFlushBytes)
		batch_flush_locked();
	return true;
}

static void batch_flush(void)
{
	std::lock_guard<std::mutex> lk(g_mu);

	batch_flush_locked();
}

/* The stream, after the pending small copies have been put on it. */
static hipStream_t stream_for_op(void)
{
	if (g_batch_dir != 0)
		batch_flush();
	return g_stream;
}

/* Waits for the stream and completes the batched D2H copies. */
hipError_t sync_stream_and_deliver(void)
{
	hipError_t err;

	batch_flush();
	err = hipStreamSynchronize(g_stream);
	if (err == hipSuccess) {
		std::lock_guard<std::mutex> lk(g_mu);

		batch_deliver_locked();
	}
	return err;
}

/* ---- state of the flat drop-in path ------------------------------------- */

static int g_prec = GPU_PREC_FP32;
static double g_wd;
static unsigned g_epoch;
static void *g_twin_bf16;		/* borrowed registration (gpu_adam_set_bf16_flat) */
static const float *g_twin_fp32;
static int g_twin_n;

#define PIN_SLOTS 256			/* as the reference's table, gpu_cuda.cu:2980 */
static const void *g_pinned[PIN_SLOTS];
static int g_pinned_n;

/* Scratch of the flat path: sum-of-squares partials + the step state, and a pinned result word. */
static double *g_partials;
static StepState *g_host_state;		/* page-locked, written by the device */

static bool scratch_ready(void)
{
	std::lock_guard<std::mutex> lk(g_mu);

	if (g_partials)
		return true;
	void *d = nullptr;
	void *h = nullptr;

	/* the partials and, behind them, the ticket counters of the second stage */
	if (hipMalloc(&d, sizeof(double) * kMaxPartials + kTicketBytes) != hipSuccess
	    || hipMemset(d, 0, sizeof(double) * kMaxPartials + kTicketBytes) != hipSuccess
	    || hipHostMalloc(&h, sizeof(StepState), hipHostMallocDefault) != hipSuccess) {
		(void)hipGetLastError();
		if (d)
			(void)hipFree(d);
		return false;
	}
	g_partials = (double *)d;
	g_host_state = (StepState *)h;
	memset(g_host_state, 0, sizeof(*g_host_state));
	return true;
}

/* ---- ANN_OP_PROF=1: event pairs around the step's launches ---------------- */

/*
** The reference times every backend operation with an event pair and prints the table from
** gpu_op_prof_dump, which lm_adam_step_scaled calls after each device step
** (num/gpu_cuda.cu:3205-3409, lang/lm_adam.c:541).  Here the operations are the optimizer's:
** the sum of squares, the update, and the passes that keep derived weight copies current.
** Pairs are resolved at gpu_device_sync and at the dump.  The table and its slots are guarded
** by g_mu; the events themselves are recorded on the compute stream outside it.
*/
struct ProfSlot {
	hipEvent_t	a;
	hipEvent_t	b;
	int		kind;
};
#define PROF_SLOTS 256
static ProfSlot g_prof[PROF_SLOTS];
static int g_prof_n;
static int g_prof_round;		/* counts resolutions: a slot number is only good within its round */
static double g_prof_ms[kProfKinds];
static int g_prof_calls[kProfKinds];

bool prof_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANN_OP_PROF");

		on = (e && e[0] == '1') ? 1 : 0;
	}
	return on == 1;
}

/* g_mu held.  Waits for the recorded pairs (the stream has to reach them) and adds them to the table. */
static void prof_resolve_locked(void)
{
	for (int i = 0; i < g_prof_n; i++) {
		float ms = 0.0f;

		if (g_prof[i].b && hipEventSynchronize(g_prof[i].b) == hipSuccess
		    && hipEventElapsedTime(&ms, g_prof[i].a, g_prof[i].b) == hipSuccess) {
			g_prof_ms[g_prof[i].kind] += ms;
			g_prof_calls[g_prof[i].kind]++;
		}
		(void)hipEventDestroy(g_prof[i].a);
		if (g_prof[i].b)
			(void)hipEventDestroy(g_prof[i].b);
	}
	(void)hipGetLastError();
	g_prof_n = 0;
	g_prof_round = (g_prof_round + 1) & 0xffff;
}

/* The first event of a pair, recorded on `st`; the pair's slot, or -1 (profiling off, no slot). */
int prof_begin(int kind, hipStream_t st)
{
	hipEvent_t a = nullptr;
	int slot;

	if (!prof_on() || kind < 0 || kind >= kProfKinds)
		return -1;
	if (hipEventCreate(&a) != hipSuccess) {
		(void)hipGetLastError();
		return -1;
	}
	{
		std::lock_guard<std::mutex> lk(g_mu);

		if (g_prof_n == PROF_SLOTS)
			prof_resolve_locked();
		slot = g_prof_n++;
		g_prof[slot].a = a;
		g_prof[slot].b = nullptr;
		g_prof[slot].kind = kind;
		slot += g_prof_round * PROF_SLOTS;
	}
	(void)hipEventRecord(a, st);
	return slot;
}

/* The second event of the pair `slot` (a result of prof_begin that the table has not resolved since). */
void prof_end(int slot, hipStream_t st)
{
	hipEvent_t b = nullptr;

	if (slot < 0)
		return;
	if (hipEventCreate(&b) != hipSuccess) {
		(void)hipGetLastError();
		return;
	}
	(void)hipEventRecord(b, st);
	std::lock_guard<std::mutex> lk(g_mu);

	/* a table that was resolved in between has dropped the pair: nothing to complete */
	if (slot / PROF_SLOTS == g_prof_round && slot % PROF_SLOTS < g_prof_n
	    && !g_prof[slot % PROF_SLOTS].b)
		g_prof[slot % PROF_SLOTS].b = b;
	else
		(void)hipEventDestroy(b);
}

} /* namespace anni */

using namespace anni;

extern "C" {

int gpu_available(void)
{
	return device_ready() ? 1 : 0;
}

const char *gpu_backend_name(void)
{
	return "hip-gfx950";
}

static size_t pools_idle_bytes_locked(void);

int gpu_mem_info(size_t *free_bytes, size_t *total_bytes)
{
	size_t f = 0;
	size_t t = 0;

	if (!device_ready() || !hip_ok(hipMemGetInfo(&f, &t), "hipMemGetInfo"))
		return -1;
	{
		std::lock_guard<std::mutex> lk(g_pool_mu);

		f += pools_idle_bytes_locked();	/* reserved, but there for the asking */
	}
	if (free_bytes)
		*free_bytes = f;
	if (total_bytes)
		*total_bytes = t;
	return 0;
}

void gpu_device_sync(void)
{
	hipError_t err;

	if (!device_ready())
		return;
	batch_flush();
	err = hipDeviceSynchronize();
	if (err == hipSuccess) {
		std::lock_guard<std::mutex> lk(g_mu);

		batch_deliver_locked();
	}
	if (err != hipSuccess) {
		fprintf(stderr, "gpu_device_sync: %s\n", hipGetErrorString(err));
		(void)hip_ok(err, "hipDeviceSynchronize");
	} else if (prof_on()) {
		std::lock_guard<std::mutex> lk(g_mu);
		prof_resolve_locked();
	}
}

int gpu_stream_sync(void)
{
	if (!device_ready())
		return -1;
	return hip_ok(sync_stream_and_deliver(), "hipStreamSynchronize") ? 0 : -1;
}

void gpu_set_compute_prec(int prec)
{
	g_prec = prec == GPU_PREC_BF16 ? GPU_PREC_BF16 : GPU_PREC_FP32;
}

const char *gpu_debug_last_error(void)
{
	static thread_local char out[256];
	std::lock_guard<std::mutex> lk(g_mu);

	if (!g_err[0] && device_ready()) {
		hipError_t err = hipGetLastError();

		if (err != hipSuccess)
			snprintf(g_err, sizeof(g_err), "%s", hipGetErrorString(err));
	}
	memcpy(out, g_err, sizeof(out));
	g_err[0] = '\0';
	return out;
}

void gpu_op_prof_dump(void)
{
	static const char *name[kProfKinds] = { "grad_sumsq", "adam_step", "derived" };

	if (!prof_on() || !device_ready())
		return;
	std::lock_guard<std::mutex> lk(g_mu);
	prof_resolve_locked();
	for (int k = 0; k < kProfKinds; k++) {
		if (!g_prof_calls[k])
			continue;
		fprintf(stderr, "[op-prof] %-12s %8.3f ms  %d calls\n", name[k], g_prof_ms[k],
		    g_prof_calls[k]);
		g_prof_ms[k] = 0.0;
		g_prof_calls[k] = 0;
	}
}

/* ---- memory --------------------------------------------------------------- */

/*
** Large blocks, placed.  lang/lm_adam.c asks for its five flats one gpu_malloc at a time
** (d_param, d_grad, d_param_bf16, later d_m, d_v: lm_adam.c:222-229,295-297).  On MI355X a kernel
** that streams all of them runs ~15 % slower when they all lie in one of the three 96 GiB
** sections of device memory than when they are split over two (placement.h).  So blocks of
** kPlaceMin bytes and more are dealt to TWO pools, each new block to the pool that holds fewer
** live bytes (p, twin, v | g, m for the caller above: 18 + 16 of the update's 34 bytes per
** parameter).  A pool grows by chunks of four times the request that opens them; a chunk that
** opens the second pool (or a later chunk of either) is looked for in another section than the
** other pool's memory by timing the update on free space of both (alloc_apart_from).  Inside a
** chunk blocks are handed out first-fit at 2 MiB boundaries and merged again when freed.  An
** emptied chunk stays reserved (a caller that frees all its flats and allocates them again --
** lm_adam_free and a new optimizer, the optional m/v offload -- would otherwise repeat the
** search every time) until memory is wanted elsewhere: an allocation that fails, or an arena
** being created, gives them back first; gpu_mem_info counts them as free.
** ANNI_MALLOC_PLACE=0 switches all of this off (every block a plain hipMalloc).
*/
static std::vector<PoolChunk> g_chunks;
static size_t g_pool_live[2];

static bool place_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANNI_MALLOC_PLACE");

		on = (e && e[0] == '0') ? 0 : 1;
	}
	return on == 1;
}

/* First fit inside one chunk.  g_pool_mu held. */
static void *chunk_take(PoolChunk &c, size_t need)
{
	const size_t off = c.take(need);

	if (off == (size_t)-1)
		return nullptr;
	g_pool_live[c.pool] += need;
	return c.base + off;
}

/* The largest free block of the chunks of `pool`: scratch for the placement probe.  g_pool_mu held. */
static char *pool_scratch(int pool, size_t *bytes)
{
	char *best = nullptr;

	*bytes = 0;
	for (PoolChunk &c : g_chunks) {
		size_t n = 0;
		const size_t off = c.largest_free(&n);

		if (c.pool == pool && n > *bytes) {
			*bytes = n;
			best = c.base + off;
		}
	}
	return best;
}

static bool g_pool_growing;		/* one thread at a time looks for a new chunk */

/*
** A block of a pool, or nullptr (the caller then allocates the plain way).  Takes g_pool_mu
** itself and lets go of it while it looks for a new chunk: the search requests and times tens of
** GiB and takes tens of milliseconds, and every other thread's gpu_malloc, gpu_free and
** gpu_mem_info would wait that long.  What the search needs from the pools -- the free space of
** the other pool that it uses as scratch -- is reserved as a block for the time, so nobody is
** handed it and its chunk does not count as idle; a second thread that needs a new chunk
** meanwhile gets a plain allocation.
*/
static void *pool_take(size_t nbytes)
{
	const size_t need = (nbytes + ((size_t)2 << 20) - 1) & ~(((size_t)2 << 20) - 1);
	size_t fr = 0, tt = 0, scratch_bytes = 0;
	size_t chunk_bytes = 4 * need;
	PoolChunk *scratch_chunk = nullptr;
	char *scratch = nullptr;
	void *mem = nullptr;
	void *got = nullptr;
	int pool;

	{
		std::lock_guard<std::mutex> lk(g_pool_mu);

		pool = g_pool_live[1] < g_pool_live[0] ? 1 : 0;
		for (PoolChunk &have : g_chunks)
			if (have.pool == pool) {
				void *p = chunk_take(have, need);

				if (p)
					return p;
			}
		if (g_pool_growing)
			return nullptr;
		if (hipMemGetInfo(&fr, &tt) != hipSuccess) {
			(void)hipGetLastError();
			return nullptr;
		}
		if (chunk_bytes > fr / 8)
			chunk_bytes = need;		/* memory is short: no more than what is asked for */
		if (chunk_bytes > fr / 2)
			return nullptr;
		scratch = pool_scratch(1 - pool, &scratch_bytes);
		if (scratch) {
			for (PoolChunk &c : g_chunks)
				if (scratch >= c.base && scratch < c.base + c.bytes)
					scratch_chunk = &c;
			if (!scratch_chunk || scratch_chunk->take_block((size_t)(scratch - scratch_chunk->base))
			    != scratch_bytes)
				return nullptr;
		}
		g_pool_growing = true;
	}
	/* the lock is free; g_chunks may grow or shrink meanwhile, so the reservation is found again by address */
	try {
		if (scratch) {
			mem = alloc_apart_from(scratch, scratch_bytes, chunk_bytes, nullptr);
		} else if (hipMalloc(&mem, chunk_bytes) != hipSuccess) {
			(void)hipGetLastError();
			mem = nullptr;
		}
	} catch (...) {
		mem = nullptr;		/* the reservation and the flag below are undone all the same */
	}
	{
		std::lock_guard<std::mutex> lk(g_pool_mu);

		g_pool_growing = false;
		if (scratch)
			for (PoolChunk &c : g_chunks)
				if (scratch >= c.base && scratch < c.base + c.bytes)
					(void)c.give((size_t)(scratch - c.base));
		if (mem) {
			try {
				g_chunks.push_back(PoolChunk((char *)mem, chunk_bytes, pool));
				got = chunk_take(g_chunks.back(), need);
			} catch (...) {
				(void)hipFree(mem);
				got = nullptr;
			}
		}
	}
	return got;
}

/*
** g_pool_mu held.  1 when p was a block of a pool (now free again), 0 when p lies in no chunk,
** -1 when it points into a chunk without being the start of a live block (a caller's mistake:
** nothing is freed).
*/
static int pool_give(void *p)
{
	for (PoolChunk &c : g_chunks) {
		if ((char *)p < c.base || (char *)p >= c.base + c.bytes)
			continue;
		const size_t n = c.give((size_t)((char *)p - c.base));

		if (n == 0)
			return -1;
		g_pool_live[c.pool] -= n;
		return 1;
	}
	return 0;
}

/*
** g_pool_mu held.  Bytes the pools hold without a block in them: whole chunks that are empty
** (given back to the driver on demand) and the free space inside chunks that are in use (handed
** out by the next large gpu_malloc).
*/
static size_t pools_idle_bytes_locked(void)
{
	size_t idle = 0;

	for (const PoolChunk &c : g_chunks)
		idle += c.bytes - c.live;
	return idle;
}

/* g_pool_mu held.  Gives the empty chunks back to the driver; true when there was one. */
static bool pools_release_idle_locked(void)
{
	bool any = false;

	for (size_t i = 0; i < g_chunks.size();) {
		if (g_chunks[i].live != 0) {
			i++;
			continue;
		}
		if (!any)
			(void)hipStreamSynchronize(g_stream);
		(void)hipFree(g_chunks[i].base);
		g_chunks.erase(g_chunks.begin() + (long)i);
		any = true;
	}
	return any;
}

void *gpu_malloc(size_t nbytes)
{
	void *p = nullptr;

	if (nbytes == 0 || !device_ready())
		return nullptr;
	if (nbytes >= kPlaceMin && place_on()) {
		batch_flush();			/* the placement probe runs on the compute stream */
		try {
			p = pool_take(nbytes);
		} catch (...) {
			p = nullptr;
		}
		if (p)
			return p;
	}
	if (hipMalloc(&p, nbytes) != hipSuccess) {
		bool released;

		(void)hipGetLastError();
		{
			std::lock_guard<std::mutex> lk(g_pool_mu);

			released = pools_release_idle_locked();
		}
		if (!released || !hip_ok(hipMalloc(&p, nbytes), "hipMalloc")) {
			if (!released)
				(void)hip_ok(hipErrorOutOfMemory, "hipMalloc");
			(void)hipGetLastError();
			return nullptr;
		}
	}
	return p;
}

void gpu_free(void *p)
{
	if (!p || !device_ready())
		return;
	batch_flush();		/* nothing pending may still point into the block */
	{
		std::lock_guard<std::mutex> lk(g_mu);

		/* A freed flat must not stay registered: the address may be reused. */
		if (p == g_twin_bf16 || p == (const void *)g_twin_fp32) {
			g_twin_bf16 = nullptr;
			g_twin_fp32 = nullptr;
			g_twin_n = 0;
		}
	}
	{
		int given;

		{
			std::lock_guard<std::mutex> lk(g_pool_mu);

			given = pool_give(p);
		}
		if (given > 0)
			return;
		if (given < 0) {
			(void)hip_ok(hipErrorInvalidDevicePointer, "gpu_free: not the start of a block");
			return;
		}
	}
	(void)hip_ok(hipFree(p), "hipFree");
}

int gpu_memcpy_h2d(void *dst, const void *src, size_t nbytes)
{
	if (!dst || !src || nbytes == 0 || !device_ready())
		return -1;
	if (nbytes <= kSmallCopy) {
		std::lock_guard<std::mutex> lk(g_mu);

		if (batch_add_locked(1, dst, const_cast<void *>(src), nbytes))
			return 0;
	}
	return hip_ok(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, stream_for_op()),
	    "h2d") ? 0 : -1;
}

int gpu_memcpy_d2h(void *dst, const void *src, size_t nbytes)
{
	if (!dst || !src || nbytes == 0 || !device_ready())
		return -1;
	if (!hip_ok(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, stream_for_op()), "d2h"))
		return -1;
	return hip_ok(sync_stream_and_deliver(), "d2h sync") ? 0 : -1;
}

/*
** The reference page-locks the caller's range here (gpu_cuda.cu:2982-3001).
** This backend only remembers it: an asynchronous copy into pageable memory is
** staged by the runtime and has landed by the next gpu_stream_sync, which is
** all lang/lm_adam.c:407-413,500 relies on.
*/
int gpu_host_pin(void *p, size_t nbytes)
{
	if (!p || nbytes == 0 || !device_ready())
		return -1;
	std::lock_guard<std::mutex> lk(g_mu);

	for (int i = 0; i < g_pinned_n; i++)
		if (g_pinned[i] == p)
			return 0;
	if (g_pinned_n >= PIN_SLOTS)
		return -1;
	g_pinned[g_pinned_n++] = p;
	return 0;
}

void gpu_host_forget(const void *host)
{
	std::lock_guard<std::mutex> lk(g_mu);

	for (int i = 0; i < g_pinned_n; i++)
		if (g_pinned[i] == host) {
			g_pinned[i] = g_pinned[--g_pinned_n];
			return;
		}
}

int gpu_memcpy_d2h_async(void *dst, const void *src, size_t nbytes)
{
	if (!dst || !src || nbytes == 0 || !device_ready())
		return -1;
	if (nbytes <= kSmallCopy) {
		std::lock_guard<std::mutex> lk(g_mu);

		if (batch_add_locked(2, const_cast<void *>(src), dst, nbytes))
			return 0;
	}
	return hip_ok(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, stream_for_op()),
	    "d2h async") ? 0 : -1;
}

int gpu_memcpy_d2d(void *dst, const void *src, size_t nbytes)
{
	if (!dst || !src || nbytes == 0 || !device_ready())
		return -1;
	return hip_ok(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, stream_for_op()),
	    "d2d") ? 0 : -1;
}

int gpu_memset(void *dst, int value, size_t nbytes)
{
	if (!dst || nbytes == 0 || !device_ready())
		return -1;
	return launch_fill_bytes(stream_for_op(), dst, value, nbytes);
}

void *gpu_host_alloc(size_t nbytes)
{
	void *p = nullptr;

	if (nbytes == 0 || !device_ready())
		return nullptr;
	if (!hip_ok(hipHostMalloc(&p, nbytes, hipHostMallocDefault), "hipHostMalloc")) {
		(void)hipGetLastError();
		return nullptr;
	}
	return p;
}

void gpu_host_free(void *p)
{
	if (p && device_ready())
		(void)hip_ok(hipHostFree(p), "hipHostFree");
}

/* ---- BF16 twins ------------------------------------------------------------- */

void gpu_adam_set_bf16_flat(void *bf16, const ann_real *fp32, int n)
{
	std::lock_guard<std::mutex> lk(g_mu);

	g_twin_bf16 = bf16;
	g_twin_fp32 = fp32;
	g_twin_n = (bf16 && fp32 && n > 0) ? n : 0;
}

int gpu_adam_seed_bf16_flat(void *bf16, const ann_real *fp32, int n)
{
	if (!bf16 || !fp32 || n <= 0 || !device_ready())
		return -1;
	return launch_f32_to_bf16(stream_for_op(), (uint16_t *)bf16, fp32, n);
}

void gpu_half_wt_invalidate(const ann_real *fp32_dev)
{
	(void)fp32_dev;		/* no per-matrix twin cache here: the flat twin is always current */
	std::lock_guard<std::mutex> lk(g_mu);
	g_epoch++;
}

unsigned gpu_param_epoch(void)
{
	std::lock_guard<std::mutex> lk(g_mu);
	return g_epoch;
}

/* ANN_TWIN_CHECK=1: served twin slices are checked against a fresh conversion (gpu_cuda.cu:1946-1995). */
static bool twin_check_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANN_TWIN_CHECK");

		on = (e && e[0] == '1') ? 1 : 0;
	}
	return on == 1;
}

static void twin_check(const void *twin, const ann_real *fp32, size_t n)
{
	const size_t bytes = n * 2;
	void *fresh = nullptr;
	unsigned char *a, *b;
	size_t bad = 0;

	if (device_alloc(&fresh, bytes) != hipSuccess)
		return;
	a = (unsigned char *)malloc(bytes);
	b = (unsigned char *)malloc(bytes);
	if (a && b && launch_f32_to_bf16(stream_for_op(), (uint16_t *)fresh, fp32, (int64_t)n) == 0
	    && hipMemcpyAsync(a, twin, bytes, hipMemcpyDeviceToHost, g_stream) == hipSuccess
	    && hipMemcpyAsync(b, fresh, bytes, hipMemcpyDeviceToHost, g_stream) == hipSuccess
	    && sync_stream_and_deliver() == hipSuccess) {
		for (size_t i = 0; i < bytes; i++)
			bad += a[i] != b[i];
		if (bad)
			fprintf(stderr, "[twin] STALE flat fp32=%p n=%zu bytes_diff=%zu\n",
			    (const void *)fp32, n, bad);
	}
	(void)hipGetLastError();
	free(a);
	free(b);
	(void)hipFree(fresh);
}

const void *anni_gpu_bf16_twin_of(const ann_real *fp32_dev, size_t n)
{
	const char *twin = nullptr;

	if (!fp32_dev || n == 0 || !device_ready())
		return nullptr;
	{
		std::lock_guard<std::mutex> lk(g_mu);

		if (g_twin_bf16 && g_twin_fp32 && g_twin_n > 0 && fp32_dev >= g_twin_fp32
		    && n <= (size_t)g_twin_n
		    && (size_t)(fp32_dev - g_twin_fp32) <= (size_t)g_twin_n - n)
			twin = (const char *)g_twin_bf16 + (size_t)(fp32_dev - g_twin_fp32) * 2u;
	}
	if (twin && twin_check_on())
		twin_check(twin, fp32_dev, n);
	return twin;
}

/* ---- the optimizer step -------------------------------------------------------- */

void gpu_adam_set_weight_decay(double wd)
{
	g_wd = wd > 0.0 ? wd : 0.0;
}

/*
** One result slot, one partials array and one set of ticket words serve every call (as the
** reference's static accumulator does, num/gpu_cuda.cu:8485-8486): a call that arrives while
** another is between its launch and its read-back would fold the other's partials or read the
** other's result, so it is turned away (-1: the caller takes its CPU path) instead.
*/
static BusyFlag g_sumsq_busy;

int gpu_grad_sumsq(const ann_real *d_x, int n, double *out)
{
	Flat f;
	int np = 0;

	if (!d_x || n <= 0 || !out || !device_ready() || !scratch_ready())
		return -1;
	BusyScope only(g_sumsq_busy);

	if (!only.entered)
		return -1;
	memset(&f, 0, sizeof(f));
	f.g = (void *)d_x;
	f.n = n;
	f.grad_type = kF32;
	(void)stream_for_op();
	{
		const int slot = prof_begin(kProfSumsq, g_stream);
		SumsqFinish fin;
		int rc;

		/* the second stage stores its result straight into page-locked host memory */
		fin.ticket = (unsigned int *)(g_partials + kMaxPartials);
		fin.clip = 0.0;
		fin.skip_nonfinite = 0;
		fin.state = g_host_state;
		rc = launch_sumsq(g_stream, f, 1.0, g_partials, &np, &fin);
		prof_end(slot, g_stream);
		if (rc != 0)
			return -1;
	}
	if (!hip_ok(sync_stream_and_deliver(), "sumsq sync"))
		return -1;
	*out = g_host_state->sumsq;
	return 0;
}

int gpu_adam_step_dev_bf16(ann_real *d_param, void *d_param_bf16, ann_real *d_grad,
	ann_real *d_m, ann_real *d_v, int n, double lr, double beta1, double beta2, double eps,
	int t, double grad_scale)
{
	Flat f;
	StepConsts c;
	NormIn norm;

	if (!d_param || !d_grad || !d_m || !d_v || n <= 0 || lr <= 0.0 || t < 1)
		return -1;
	if (!device_ready())
		return -1;
	c.bc1 = 1.0 - pow(beta1, (double)t);		/* lm_adam.c:571-572 */
	c.bc2 = 1.0 - pow(beta2, (double)t);
	if (c.bc1 <= 0.0 || c.bc2 <= 0.0)
		return -1;
	c.rbc1 = 1.0 / c.bc1;
	c.rbc2 = 1.0 / c.bc2;
	c.beta1 = beta1;
	c.omb1 = 1.0 - beta1;
	c.beta2 = beta2;
	c.omb2 = 1.0 - beta2;
	c.eps = eps;
	c.lr = lr;
	c.decay_on = g_wd > 0.0 ? 1 : 0;
	c.lr_wd = lr * g_wd;
	memset(&f, 0, sizeof(f));
	f.p = d_param;
	f.g = d_grad;
	f.m = d_m;
	f.v = d_v;
	f.twin = (d_param_bf16 && g_prec == GPU_PREC_BF16) ? (uint16_t *)d_param_bf16 : nullptr;
	f.n = n;
	f.grad_type = kF32;
	f.moment_type = kF32;
	f.uniform_flags = (g_wd > 0.0 ? kSegDecay : 0u) | (f.twin ? kSegTwin : 0u);
	memset(&norm, 0, sizeof(norm));
	(void)stream_for_op();
	{
		const int slot = prof_begin(kProfUpdate, g_stream);
		const int rc = launch_update(g_stream, f, c, grad_scale, norm);

		prof_end(slot, g_stream);
		return rc;
	}
}

} /* extern "C" */

namespace anni {

bool release_idle_pools(void)
{
	std::lock_guard<std::mutex> lk(g_pool_mu);

	return pools_release_idle_locked();
}

hipError_t device_alloc(void **p, size_t nbytes)
{
	hipError_t err = hipMalloc(p, nbytes);

	if (err != hipSuccess && release_idle_pools()) {
		(void)hipGetLastError();
		err = hipMalloc(p, nbytes);
	}
	if (err != hipSuccess) {
		(void)hipGetLastError();
		*p = nullptr;
	}
	return err;
}

} /* namespace anni */

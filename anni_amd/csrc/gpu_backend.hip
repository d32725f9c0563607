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
#include <algorithm>
#include <atomic>
#include <chrono>
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
static hipStream_t g_side_stream;	/* the sum begun early runs beside the small uploads, not in front of them */
static hipStream_t g_side_for;		/* the compute stream g_side_stream was tried against */
static int g_side_tries;		/* searches for such a stream so far */
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
/*
** Counts the times the stream was handed out for an operation other than a batch of small
** copies: whoever holds a value of it knows whether anything else has been put on the stream
** since (see "the sum begun early").
*/
static std::atomic<unsigned long long> g_op_seq;
/* a split update has left work on the side stream that the compute stream must not overtake (see "the vectors first") */
static std::atomic<int> g_vf_side_pending;
static void vf_side_wait(void);

hipStream_t compute_stream(void)
{
	g_op_seq.fetch_add(1, std::memory_order_relaxed);
	if (g_vf_side_pending.load(std::memory_order_acquire))
		vf_side_wait();
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
** The device ranges of the uploads that wait for the next launch, sorted, none overlapping another.
** The pieces of one launch are copied in no particular order, so an upload that overlaps one of them
** must not share their launch: the caller's order (the later copy wins) is kept by the launch boundary.
*/
struct UpRange {
	uintptr_t	lo, hi;
};
static std::vector<UpRange> g_up_pending;
static bool up_before(const UpRange &a, const UpRange &b)
{
	return a.lo < b.lo;
}
static const size_t kUpPendingMax = 512;	/* more than that waiting: launch, so that the list stays short */

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

static void early_sum_on_small_h2d_locked(const void *dev, size_t nbytes);
static void early_sum_on_sync_locked(void);
static void vf_side_wait_locked(void);
static void vf_on_sync_locked(void);
static bool vf_on_small_d2h_locked(const void *dev, void *host, size_t nbytes);
static void vf_on_small_h2d_locked(void);

/* Launches the pending batch.  g_mu held. */
static void batch_flush_locked(void)
{
	const int count = g_desc_used - g_batch_first;

	if (count > 0) {
		vf_side_wait_locked();
		hipLaunchKernelGGL(small_copy_kernel, dim3(count), dim3(256), 0, g_stream,
		    g_desc + g_batch_first, g_stage, g_batch_dir == 1 ? 1 : 0);
		(void)hip_ok_locked(hipGetLastError(), "small copy batch");
	}
	g_batch_first = g_desc_used;
	g_batch_bytes = 0;
	g_batch_dir = 0;
	g_up_pending.clear();
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
	vf_side_wait_locked();
	vf_on_sync_locked();
	early_sum_on_sync_locked();
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
	if (dir == 2 && vf_on_small_d2h_locked(dev, host, nbytes))
		return true;		/* a split update has copied it already */
	if (g_batch_dir != 0 && g_batch_dir != dir)
		batch_flush_locked();
	if (dir == 1) {
		const UpRange r = {(uintptr_t)dev, (uintptr_t)dev + nbytes};
		const auto nx = std::lower_bound(g_up_pending.begin(), g_up_pending.end(), r, up_before);

		if ((nx != g_up_pending.end() && nx->lo < r.hi)
		    || (nx != g_up_pending.begin() && (nx - 1)->hi > r.lo)
		    || g_up_pending.size() >= kUpPendingMax)
			batch_flush_locked();		/* what it overlaps goes first, in a launch of its own */
		vf_on_small_h2d_locked();
		early_sum_on_small_h2d_locked(dev, nbytes);	/* may put the sum of the gradient flat on the stream first */
	}
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
		const UpRange r = {(uintptr_t)dev, (uintptr_t)dev + nbytes};

		memcpy(g_stage + at, host, nbytes);
		g_up_pending.insert(std::lower_bound(g_up_pending.begin(), g_up_pending.end(), r, up_before), r);
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
	g_op_seq.fetch_add(1, std::memory_order_relaxed);
	if (g_vf_side_pending.load(std::memory_order_acquire))
		vf_side_wait();
	if (g_batch_dir != 0)
		batch_flush();
	return g_stream;
}

/* Waits for the stream and completes the batched D2H copies. */
hipError_t sync_stream_and_deliver(void)
{
	hipError_t err;

	batch_flush();
	if (g_vf_side_pending.load(std::memory_order_acquire))
		vf_side_wait();		/* the vectors are handed over while the rest of the update runs */
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

/*
** Scratch of the flat path's sum of squares: one partial sum per 16 KiB chunk of the flat
** (grown when a longer flat comes), the sums of their runs, and the result in page-locked host
** memory, which the last kernel writes directly.
*/
static double *g_chunk_part;
static int64_t g_chunk_cap;		/* chunks g_chunk_part has room for */
static double *g_chunk_runs;
static unsigned int *g_chunk_ticket;	/* of the sum's last stage; zero between launches */
static StepState *g_host_state;		/* page-locked, written by the device */
/*
** Two words the device writes for a host that is waiting: [0] by the last kernel of the sum, [1]
** by a one-lane kernel behind the sum begun early.  hipStreamSynchronize was seen to return 40 -
** 170 us after the last kernel had ended whenever a second stream had been busy shortly before,
** and asking hipStreamQuery in a loop slowed the kernels down; a load from page-locked memory
** does neither.  Every wait expects a number of its own.
*/
static unsigned long long *g_host_stamp;
static unsigned long long g_stamp_token;

/* g_mu held.  Room for the partials of a flat of n floats; false when memory cannot be had. */
static bool sum_scratch_locked(int64_t n)
{
	const int64_t chunks = chunk_sums_count(n);

	if (!g_host_state) {
		void *h = nullptr;
		void *r = nullptr;
		void *k = nullptr;

		static_assert(sizeof(StepState) <= 128, "the stamps lie 128 bytes behind the state");
		if (hipHostMalloc(&h, 256, hipHostMallocDefault) != hipSuccess
		    || hipMalloc(&r, sizeof(double) * kChunkRuns) != hipSuccess
		    || hipMalloc(&k, kTicketBytes) != hipSuccess
		    || hipMemset(k, 0, kTicketBytes) != hipSuccess) {
			(void)hipGetLastError();
			if (h)
				(void)hipHostFree(h);
			if (r)
				(void)hipFree(r);
			if (k)
				(void)hipFree(k);
			return false;
		}
		memset(h, 0, 256);
		g_host_state = (StepState *)h;
		g_host_stamp = (unsigned long long *)((char *)h + 128);
		g_chunk_runs = (double *)r;
		g_chunk_ticket = (unsigned int *)k;
		memset(g_host_state, 0, sizeof(*g_host_state));
	}
	if (chunks > g_chunk_cap) {
		void *d = nullptr;

		/* nothing on the stream may still write the old block */
		if (hipStreamSynchronize(g_stream) != hipSuccess
		    || hipMalloc(&d, sizeof(double) * (size_t)chunks) != hipSuccess) {
			(void)hipGetLastError();
			return false;
		}
		if (g_chunk_part)
			(void)hipFree(g_chunk_part);
		g_chunk_part = (double *)d;
		g_chunk_cap = chunks;
	}
	return true;
}

/* ---- the sum begun early ------------------------------------------------------------------ */

/*
** lang/lm_adam.c spends the first part of every step on the host: it uploads its bias and
** LayerNorm vectors and their gradients, one small gpu_memcpy_h2d each (lm_adam.c:372-377),
** and only then asks for the sum of squares of the gradient flat (:470) -- 0.12 ms at its 185M
** size, 0.19 ms at 555M, during which the device has nothing to do, followed by 0.11 - 0.32 ms in
** which the host has nothing to do.  All but a few hundred KiB of what the sum reads is in place
** when the first of those uploads arrives (the matrices' gradients were written by the backward
** pass; the caller synchronises before it begins, :539).  So once the caller has shown the pattern
** twice in a row -- since the last synchronisation nothing but small uploads, then gpu_grad_sumsq
** of the same flat -- the next first small upload into that flat or into the registered parameter
** flat (gpu_adam_set_bf16_flat) launches the chunk sums of the whole gradient flat on a second
** stream, where they run beside the uploads.  The chunks that small uploads write afterwards are
** noted; gpu_grad_sumsq then recomputes the partial sums of just those and folds.  The sum is a function of the flat's
** contents alone (adam_kernels.hip, chunk_sums_kernel), so the result has the bits of a sum begun
** when it was asked for.
**
** The early sum is used only if nothing but batches of small copies went onto the stream between
** its launch and the call (g_op_seq: every other entry point of this library draws a number
** there, and so does a caller who takes the stream handle or announces work of its own with
** anni_gpu_flush, which the header asks of it), and only if the call names the flat that was
** summed; otherwise it is dropped, the sum is taken from the start as if nothing had happened,
** and the pattern has to be shown twice again.  A guess that was wrong costs the stream one pass
** over the flat.  ANNI_EARLY_SUM=0 switches the guessing off.
*/
/*
** A stream whose kernels run BESIDE those of the compute stream.  The runtime deals its streams
** out over a few hardware queues (four by default), and two streams that share a queue take
** turns: which ones do depends on what else the process has created, so it is measured.  A
** kernel on the candidate notes the time, idles for 40 us (a bounded wait on the clock) and notes
** the time again; a kernel launched on the compute stream right behind it notes the time too.
** If that stamp lies before the candidate's second one, the two ran side by side.
*/
__global__ void probe_idle_kernel(unsigned long long *ts, unsigned long long ticks)
{
	if (threadIdx.x == 0) {
		const unsigned long long t0 = wall_clock64();

		ts[0] = t0;
		while (wall_clock64() - t0 < ticks)
			__builtin_amdgcn_s_sleep(8);
		ts[1] = wall_clock64();
	}
}

__global__ void probe_stamp_kernel(unsigned long long *ts)
{
	if (threadIdx.x == 0)
		ts[2] = wall_clock64();
}

/* g_mu held, the compute stream idle.  The side stream for g_stream, or NULL when none could be found. */
static hipStream_t side_stream_locked(void)
{
	const int kCandidates = 4;
	unsigned long long *ts = nullptr;
	hipStream_t found = nullptr;

	if (g_side_for == g_stream)
		return g_side_stream;
	if (g_side_tries >= 4)
		return nullptr;		/* a caller who keeps changing streams: not worth another search */
	g_side_tries++;
	if (g_side_stream) {
		(void)hipStreamSynchronize(g_side_stream);
		(void)hipStreamDestroy(g_side_stream);
		g_side_stream = nullptr;
	}
	g_side_for = g_stream;
	if (hipHostMalloc((void **)&ts, 3 * sizeof(*ts), hipHostMallocDefault) != hipSuccess) {
		(void)hipGetLastError();
		return nullptr;
	}
	for (int i = 0; i < kCandidates && !found; i++) {
		hipStream_t c = nullptr;

		if (hipStreamCreate(&c) != hipSuccess)
			break;
		ts[0] = ts[1] = ts[2] = 0;
		hipLaunchKernelGGL(probe_idle_kernel, dim3(1), dim3(64), 0, c, ts, 4000ull);	/* the clock runs at 100 MHz */
		hipLaunchKernelGGL(probe_stamp_kernel, dim3(1), dim3(64), 0, g_stream, ts);
		if (hipStreamSynchronize(c) == hipSuccess && hipStreamSynchronize(g_stream) == hipSuccess
		    && ts[1] != 0 && ts[2] != 0 && ts[2] < ts[1])
			found = c;
		else
			(void)hipStreamDestroy(c);
	}
	(void)hipGetLastError();
	(void)hipHostFree(ts);
	g_side_stream = found;
	return found;
}

__global__ void stamp_kernel(unsigned long long *stamp, unsigned long long token)
{
	if (threadIdx.x == 0)
		__hip_atomic_store(stamp, token, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

/*
** Watches *stamp until it holds `token` or a later one (the numbers written to one word only
** grow); false when it still does not after 50 ms (the caller then waits the ordinary way).
*/
static bool stamp_wait(const unsigned long long *stamp, unsigned long long token)
{
	const auto t0 = std::chrono::steady_clock::now();

	for (unsigned spins = 1; __atomic_load_n(stamp, __ATOMIC_ACQUIRE) < token; spins++) {
		__builtin_ia32_pause();
		if ((spins & 4095) == 0
		    && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(50))
			return false;
	}
	return true;
}

static const size_t kEarlyDirtyMax = 8192;

struct EarlySum {
	const float	*x;		/* the flat the last gpu_grad_sumsq summed */
	int		n;
	int		shown;		/* calls in a row that fitted the pattern */
	bool		launched;	/* chunk sums of (x, n) are on the side stream ... */
	unsigned long long	token;	/* ... and this number arrives in g_host_stamp[1] when they are done */
	unsigned long long	seq;	/* g_op_seq when they were launched */
	unsigned long long	seq_at_sync;	/* g_op_seq at the last synchronisation */
	bool		uploads;	/* small uploads into the watched flats have come since the last gpu_grad_sumsq */
	unsigned long long	seq_first;	/* g_op_seq at the first of them ... */
	bool		began_clean;	/* ... which was also its value at the synchronisation before it */
	std::vector<int32_t>	dirty;	/* chunks written by small uploads since the launch */
	bool		overflow;
	long		used, dropped;	/* for the record */
};
static EarlySum g_early;

static bool early_sum_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANNI_EARLY_SUM");

		on = (e && e[0] == '0') ? 0 : 1;
	}
	return on == 1;
}

/* Work put on the second stream would not become part of a graph being recorded on the compute stream. */
static bool compute_stream_is_recording(void)
{
	hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;

	if (hipStreamIsCapturing(g_stream, &cs) != hipSuccess) {
		(void)hipGetLastError();
		return true;
	}
	return cs != hipStreamCaptureStatusNone;
}

static bool inside(const void *p, size_t nbytes, const void *base, size_t span)
{
	return base && (const char *)p >= (const char *)base
	    && (const char *)p + nbytes <= (const char *)base + span;
}

/* g_mu held: a small upload of nbytes to dev is about to be queued. */
static void early_sum_on_small_h2d_locked(const void *dev, size_t nbytes)
{
	EarlySum &e = g_early;
	const size_t flat_bytes = (size_t)(e.n > 0 ? e.n : 0) * sizeof(float);
	const bool in_grad = e.x && inside(dev, nbytes, e.x, flat_bytes);
	const bool in_param = g_twin_fp32 && inside(dev, nbytes, g_twin_fp32, (size_t)g_twin_n * sizeof(float));

	if (!in_grad && !in_param)
		return;
	if (!e.uploads) {
		const unsigned long long now = g_op_seq.load(std::memory_order_relaxed);

		/* the first upload of what may be the caller's gather */
		e.uploads = true;
		e.seq_first = now;
		e.began_clean = now == e.seq_at_sync;
		if (!e.launched && e.shown >= 2 && e.began_clean && early_sum_on() && e.x
		    && g_chunk_part && chunk_sums_count(e.n) <= g_chunk_cap && !compute_stream_is_recording()
		    && side_stream_locked()) {
			/*
			** On a stream of its own, so that the uploads that follow run beside it instead of
			** queueing up behind it.  No event ties the two streams together (recording and
			** waiting for one costs the host 15 - 60 us here, more than the sum saves at this
			** size): the compute stream has just been synchronised and has been given nothing
			** since but small uploads elsewhere, which the sum does not read; and before the
			** partial sums are used the host waits for the side stream (sumsq_enqueue_locked).
			** An upload may write a chunk while the sum reads it; every such chunk is on the list
			** of those whose partial sums are computed again once both have finished, so what the
			** sum made of it is never used.
			*/
			if (launch_chunk_sums(g_side_stream, e.x, e.n, g_chunk_part, nullptr, 0, 1) == 0) {
				e.token = ++g_stamp_token;
				hipLaunchKernelGGL(stamp_kernel, dim3(1), dim3(64), 0, g_side_stream, g_host_stamp + 1,
				    e.token);
				(void)hipGetLastError();
				e.launched = true;
				e.seq = now;
				e.dirty.clear();
				e.overflow = false;
			}
		}
	}
	if (e.launched && in_grad) {
		const size_t off = (size_t)((const char *)dev - (const char *)e.x);
		const size_t chunk = kSumChunkBytes;

		for (size_t c = off / chunk; c <= (off + nbytes - 1) / chunk; c++) {
			if (e.dirty.size() >= kEarlyDirtyMax) {
				e.overflow = true;
				break;
			}
			if (e.dirty.empty() || e.dirty.back() != (int32_t)c)
				e.dirty.push_back((int32_t)c);
		}
	}
}

/* g_mu held: the stream has drained. */
static void early_sum_on_sync_locked(void)
{
	g_early.seq_at_sync = g_op_seq.load(std::memory_order_relaxed);
}

/* g_mu held: the flat p is being freed. */
static void early_sum_forget_locked(const void *p)
{
	if (g_early.x && p == (const void *)g_early.x) {
		if (g_early.launched && g_side_stream)
			(void)hipStreamSynchronize(g_side_stream);	/* it is still reading the flat */
		g_early.x = nullptr;
		g_early.n = 0;
		g_early.shown = 0;
		g_early.launched = false;
	}
}

/* ---- the vectors first ----------------------------------------------------------------------- */

/*
** After the update lang/lm_adam.c reads its bias and LayerNorm vectors back, one small
** gpu_memcpy_d2h_async each, and synchronises (lm_adam.c:407-413,500).  Queued behind the update
** those copies and their hand-over to the caller's memory are the tail of every step: 0.06 ms at
** 185M, 0.1 ms at 555M, with the device idle for most of it.  So once the caller has shown the same
** list of read-backs out of the parameter flat after two updates in a row, the update is split:
** the tiles that hold those vectors are updated by a launch of their own on the side stream,
** followed there by the copy of the listed ranges into page-locked memory and a stamp, while the
** compute stream updates all other tiles.  The caller's gpu_memcpy_d2h_async calls are then only
** matched against the list; gpu_stream_sync waits for the stamp, hands the vectors over while
** the large launch is still running, and then waits for that.
**
** The split is taken only when the compute stream is known to be idle at the update (it was
** synchronised and has been given nothing since), because the side stream is not ordered behind
** it.  A request that does not match the list, or anything else that reaches the stream after
** the update, ends the matching for this step: what was matched stays valid (it was asked for
** before), the rest is copied the ordinary way.  Whatever is put on the compute stream next waits
** for the side stream first.  ANNI_VECTORS_FIRST=0 switches the split off.
*/
struct Range {
	const char	*dev;
	size_t		nbytes;
	bool operator==(const Range &o) const { return dev == o.dev && nbytes == o.nbytes; }
};

struct VectorsFirst {
	/* what the caller did after the last update */
	bool		window;		/* an update was launched and no synchronisation has come since */
	bool		clean;		/* ... and nothing but small read-backs either */
	unsigned long long	seq;	/* g_op_seq right after that update */
	const float	*p;		/* its parameter flat */
	int		n;
	std::vector<Range>	cur;	/* the small read-backs out of that flat, in order */
	/* what it did the last times */
	std::vector<Range>	learned;
	const float	*learned_p;
	int		learned_n;
	int		shown;
	bool		refused;	/* the learned list does not lend itself to a split (too many tiles, too large) */
	/* built from the learned list */
	bool		built;
	int		built_backwards;
	int32_t		*order;		/* device: the vectors' tiles, then all others in the update's order */
	int64_t		k_first, n_tiles;
	CopyDesc	*desc;		/* page-locked: the copy of the learned ranges, in pieces */
	int		n_desc;
	char		*stage;		/* page-locked: where that copy lands */
	std::vector<size_t>	stage_off;	/* per learned range */
	/* this step */
	bool		active;		/* the update was split; requests are being matched */
	bool		side_pending;	/* the side stream holds work the compute stream must not overtake */
	unsigned long long	token;	/* arrives in g_host_stamp[1] when that work is done */
	std::vector<Delivery>	deliver;
	long		steps, served;	/* for the record */
};
static VectorsFirst g_vf;	/* g_vf_side_pending (above) mirrors side_pending for a look without g_mu */

static bool vectors_first_on(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANNI_VECTORS_FIRST");

		on = (e && e[0] == '0') ? 0 : 1;
	}
	return on == 1;
}

/* g_mu held.  Waits for the side stream's part of a split update and hands the matched vectors to the caller. */
static void vf_side_wait_locked(void)
{
	VectorsFirst &v = g_vf;

	if (!v.side_pending)
		return;
	if (!stamp_wait(g_host_stamp + 1, v.token))
		(void)hip_ok_locked(hipStreamSynchronize(g_side_stream), "side stream");
	v.side_pending = false;
	v.active = false;	/* whatever is asked for from here on is copied the ordinary way */
	g_vf_side_pending.store(0, std::memory_order_release);
	for (const Delivery &d : v.deliver)
		memcpy(d.host, v.stage + d.stage_off, d.nbytes);
	if (!v.deliver.empty()) {
		v.steps++;
		v.served += (long)v.deliver.size();
	}
	v.deliver.clear();
}

static void vf_side_wait(void)
{
	std::lock_guard<std::mutex> lk(g_mu);

	vf_side_wait_locked();
}

static void vf_free_built_locked(void)
{
	VectorsFirst &v = g_vf;

	if (v.order)
		(void)hipFree(v.order);
	if (v.desc)
		(void)hipHostFree(v.desc);
	if (v.stage)
		(void)hipHostFree(v.stage);
	(void)hipGetLastError();
	v.order = nullptr;
	v.desc = nullptr;
	v.stage = nullptr;
	v.stage_off.clear();
	v.built = false;
}

/* g_mu held, both streams idle.  Tile order, copy descriptors and landing place for the learned list. */
static void vf_build_locked(void)
{
	VectorsFirst &v = g_vf;
	const int64_t n_tiles = ((int64_t)v.learned_n + kTile - 1) / kTile;
	const int backwards = update_walks_backwards();
	std::vector<char> mark((size_t)n_tiles, 0);
	std::vector<int32_t> order;
	std::vector<CopyDesc> desc;
	size_t stage_bytes = 0;
	int64_t k = 0;
	void *o = nullptr, *d = nullptr, *s = nullptr;

	vf_free_built_locked();
	for (const Range &r : v.learned) {
		const size_t off = (size_t)(r.dev - (const char *)v.learned_p);
		const size_t skew = (uintptr_t)r.dev & 15;

		for (int64_t t = (int64_t)(off / 4 / kTile); t <= (int64_t)((off + r.nbytes - 1) / 4 / kTile); t++)
			if (!mark[(size_t)t]) {
				mark[(size_t)t] = 1;
				k++;
			}
		v.stage_off.push_back(stage_bytes + skew);
		for (size_t done = 0; done < r.nbytes; done += kPieceBytes) {
			CopyDesc c;

			c.dev = const_cast<char *>(r.dev) + done;
			c.stage_off = stage_bytes + skew + done;
			c.nbytes = r.nbytes - done < kPieceBytes ? r.nbytes - done : kPieceBytes;
			desc.push_back(c);
		}
		stage_bytes += (skew + r.nbytes + 255) / 256 * 256;
	}
	/* worth it only while the vectors are a small part of the flat */
	if (k < 1 || k * 8 > n_tiles || desc.size() > (size_t)kDescSlots || stage_bytes > kStageBytes) {
		v.refused = true;
		v.stage_off.clear();
		return;
	}
	order.reserve((size_t)n_tiles);
	for (int64_t t = 0; t < n_tiles; t++)
		if (mark[(size_t)t])
			order.push_back((int32_t)t);
	for (int64_t turn = 0; turn < n_tiles; turn++) {
		const int64_t t = backwards ? n_tiles - 1 - turn : turn;

		if (!mark[(size_t)t])
			order.push_back((int32_t)t);
	}
	if (device_alloc(&o, sizeof(int32_t) * (size_t)n_tiles) != hipSuccess
	    || hipHostMalloc(&d, sizeof(CopyDesc) * desc.size(), hipHostMallocDefault) != hipSuccess
	    || hipHostMalloc(&s, stage_bytes, hipHostMallocDefault) != hipSuccess
	    || hipMemcpy(o, order.data(), sizeof(int32_t) * (size_t)n_tiles, hipMemcpyHostToDevice) != hipSuccess) {
		(void)hipGetLastError();
		if (o)
			(void)hipFree(o);
		if (d)
			(void)hipHostFree(d);
		if (s)
			(void)hipHostFree(s);
		v.refused = true;
		v.stage_off.clear();
		return;
	}
	memcpy(d, desc.data(), sizeof(CopyDesc) * desc.size());
	v.order = (int32_t *)o;
	v.desc = (CopyDesc *)d;
	v.n_desc = (int)desc.size();
	v.stage = (char *)s;
	v.k_first = k;
	v.n_tiles = n_tiles;
	v.built_backwards = backwards;
	v.built = true;
}

/* g_mu held: the compute stream has drained (and the side stream, see batch_deliver_locked). */
static void vf_on_sync_locked(void)
{
	VectorsFirst &v = g_vf;

	if (!v.window)
		return;
	v.window = false;
	v.active = false;
	if (!v.clean) {
		v.shown = 0;
	} else if (!v.cur.empty()) {
		if (v.p == v.learned_p && v.n == v.learned_n && v.cur == v.learned) {
			if (v.shown < 1000)
				v.shown++;
		} else {
			v.learned = v.cur;
			v.learned_p = v.p;
			v.learned_n = v.n;
			v.shown = 1;
			v.refused = false;
			vf_free_built_locked();
		}
	}
	v.cur.clear();
	if (v.shown >= 2 && !v.refused && vectors_first_on()
	    && (!v.built || v.built_backwards != update_walks_backwards()))
		vf_build_locked();
}

/* g_mu held: a small read-back of nbytes at dev into host is asked for.  True when the split update's copy serves it. */
static bool vf_on_small_d2h_locked(const void *dev, void *host, size_t nbytes)
{
	VectorsFirst &v = g_vf;

	if (!v.window)
		return false;
	if (g_op_seq.load(std::memory_order_relaxed) != v.seq
	    || !inside(dev, nbytes, v.p, (size_t)v.n * sizeof(float))) {
		v.clean = false;
		v.active = false;
		return false;
	}
	if (!v.clean)
		return false;
	v.cur.push_back(Range{(const char *)dev, nbytes});
	if (v.active) {
		const size_t i = v.cur.size() - 1;

		if (i < v.learned.size() && v.learned[i] == v.cur[i]) {
			Delivery d;

			d.host = host;
			d.stage_off = v.stage_off[i];
			d.nbytes = nbytes;
			v.deliver.push_back(d);
			return true;
		}
		v.active = false;	/* this one and what follows are copied the ordinary way */
	}
	return false;
}

/* g_mu held: a small upload is asked for.  After an update it ends the caller's read-back pattern for this step. */
static void vf_on_small_h2d_locked(void)
{
	if (g_vf.window) {
		g_vf.clean = false;
		g_vf.active = false;
	}
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
		early_sum_forget_locked(p);
		vf_side_wait_locked();
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

/*
** g_mu held.  Puts the sum of squares of (d_x, n) on the stream, result into g_host_state.
** 0: g_host_stamp[0] will hold *token when the result is there; 1: no stamp will come; -1: failed.
*/
static int sumsq_enqueue_locked(const ann_real *d_x, int n, unsigned long long *token)
{
	EarlySum &e = g_early;
	const unsigned long long now = g_op_seq.load(std::memory_order_relaxed);
	/*
	** the pattern: small uploads into the watched flats, the first of them right after a
	** synchronisation, and nothing else on the stream since
	*/
	const bool fits = e.uploads && e.began_clean && now == e.seq_first;
	const bool same = e.x == d_x && e.n == n;
	bool early = e.launched && same && !e.overflow && now == e.seq;
	int rc = 0;

	vf_side_wait_locked();
	batch_flush_locked();			/* the last uploads go ahead of the sum */
	/*
	** Whatever becomes of the early sum, nothing below may overtake it: it writes the same
	** partials.  The host waits for it here and launches the rest afterwards.  (Queueing the
	** compute stream up behind it through an event instead was measured slower at both sizes:
	** 0.1 - 0.25 ms from the call to the result at 185M against 0.05 - 0.06 ms this way.)
	*/
	if (e.launched && !stamp_wait(g_host_stamp + 1, e.token)
	    && hipStreamSynchronize(g_side_stream) != hipSuccess) {
		(void)hipGetLastError();
		return -1;
	}
	if (!sum_scratch_locked(n))
		return -1;
	const int32_t *fix_dev = nullptr;

	if (early && !e.dirty.empty()) {
		/* the chunks written since the early sum, each once, rising; the list also travels in the staging ring */
		std::sort(e.dirty.begin(), e.dirty.end());
		e.dirty.erase(std::unique(e.dirty.begin(), e.dirty.end()), e.dirty.end());
		const size_t bytes = e.dirty.size() * sizeof(int32_t);
		const size_t need = (bytes + 255) / 256 * 256;

		if (!batch_on() || g_stage_used + need > kStageBytes) {
			early = false;
		} else {
			memcpy(g_stage + g_stage_used, e.dirty.data(), bytes);
			fix_dev = (const int32_t *)(g_stage + g_stage_used);
			g_stage_used += need;
		}
	}
	if (!early)
		rc = launch_chunk_sums(g_stream, d_x, n, g_chunk_part, nullptr, 0, 0);
	if (rc == 0)
		rc = launch_chunk_finish(g_stream, d_x, n, g_chunk_part, early ? e.dirty.data() : nullptr, fix_dev,
		    early ? (int)e.dirty.size() : 0, g_chunk_runs, g_chunk_ticket, g_host_state, g_host_stamp,
		    ++g_stamp_token);
	if (e.launched) {
		if (early)
			e.used++;
		else
			e.dropped++;
	}
	/* what this call teaches about the next step: a guess that was dropped starts the count again */
	if (!fits || (e.launched && !early))
		e.shown = 0;
	else
		e.shown = (same || !e.x) ? e.shown + 1 : 1;
	e.x = d_x;
	e.n = n;
	e.launched = false;
	e.uploads = false;
	*token = g_stamp_token;
	return rc;
}

int gpu_grad_sumsq(const ann_real *d_x, int n, double *out)
{
	unsigned long long token = 0;
	int rc;
	int slot;

	if (!d_x || n <= 0 || !out || !device_ready())
		return -1;
	BusyScope only(g_sumsq_busy);

	if (!only.entered)
		return -1;
	slot = prof_begin(kProfSumsq, g_stream);
	try {
		std::lock_guard<std::mutex> lk(g_mu);

		rc = sumsq_enqueue_locked(d_x, n, &token);
	} catch (...) {
		rc = -1;
	}
	prof_end(slot, g_stream);
	if (rc < 0)
		return -1;
	if (rc == 0 && stamp_wait(g_host_stamp, token)) {
		/*
		** The last kernel of the sum has stored its result, so everything that was put on the
		** stream before it has completed: as good as a synchronisation for the staging rings.
		*/
		std::lock_guard<std::mutex> lk(g_mu);

		batch_deliver_locked();
	} else if (!hip_ok(sync_stream_and_deliver(), "sumsq sync")) {
		return -1;
	}
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
	{
		const unsigned long long before = g_op_seq.load(std::memory_order_relaxed);
		const bool pending = g_batch_dir != 0 || g_vf_side_pending.load(std::memory_order_acquire) != 0;
		int rc = -1;
		int slot;

		(void)stream_for_op();
		slot = prof_begin(kProfUpdate, g_stream);
		{
			std::lock_guard<std::mutex> lk(g_mu);
			VectorsFirst &v = g_vf;
			bool split = false;

			v.active = false;	/* read-backs are matched only after an update that was split */
			v.deliver.clear();

			/*
			** "The vectors first": only with the list built for this very flat, and only when the
			** compute stream is known to be idle -- synchronised, and given nothing since.
			*/
			if (v.built && v.shown >= 2 && !pending && before == g_early.seq_at_sync
			    && d_param == v.learned_p && n == v.learned_n && vectors_first_on()
			    && v.built_backwards == update_walks_backwards()
			    && (g_host_stamp || sum_scratch_locked(1)) && !compute_stream_is_recording()
			    && side_stream_locked()) {
				rc = launch_update_tiles(g_stream, f, c, grad_scale, norm, v.order + v.k_first,
				    v.n_tiles - v.k_first);
				if (rc == 0) {
					split = true;
					rc = launch_update_tiles(g_side_stream, f, c, grad_scale, norm, v.order, v.k_first);
					if (rc != 0) {
						/* the vectors' tiles behind the others, then: nothing may stay without its update */
						rc = launch_update_tiles(g_stream, f, c, grad_scale, norm, v.order, v.k_first);
					} else {
						hipLaunchKernelGGL(small_copy_kernel, dim3(v.n_desc), dim3(256), 0, g_side_stream,
						    v.desc, v.stage, 0);
						v.token = ++g_stamp_token;
						hipLaunchKernelGGL(stamp_kernel, dim3(1), dim3(64), 0, g_side_stream,
						    g_host_stamp + 1, v.token);
						v.side_pending = true;
						g_vf_side_pending.store(1, std::memory_order_release);
						v.active = hip_ok_locked(hipGetLastError(), "vectors first");
						v.deliver.clear();
					}
				}
			}
			if (!split)
				rc = launch_update(g_stream, f, c, grad_scale, norm);
			/* what the caller reads back from here to its next synchronisation is the pattern to learn */
			v.window = true;
			v.clean = true;
			v.seq = g_op_seq.load(std::memory_order_relaxed);
			v.p = d_param;
			v.n = n;
			v.cur.clear();
		}
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

/* How often the sum begun early was used by the gpu_grad_sumsq that followed, and how often it was dropped. */
void early_sum_stats(long *used, long *dropped)
{
	std::lock_guard<std::mutex> lk(g_mu);

	if (used)
		*used = g_early.used;
	if (dropped)
		*dropped = g_early.dropped;
}

/* -1: no second stream has been looked for yet; 0: none runs beside the compute stream; 1: found. */
int second_stream_state(void)
{
	std::lock_guard<std::mutex> lk(g_mu);

	if (g_side_for != g_stream)
		return -1;
	return g_side_stream ? 1 : 0;
}

/* Steps whose read-backs were served by a split update, and how many read-backs that were. */
void vectors_first_stats(long *steps, long *served)
{
	std::lock_guard<std::mutex> lk(g_mu);

	if (steps)
		*steps = g_vf.steps;
	if (served)
		*served = g_vf.served;
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

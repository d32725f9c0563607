/*
** gfx950 kernels of the AnnI optimizer step: the global sum of squares (clip
** norm), the fused AdamW update with bf16 twin emission, and the small helpers
** around them.  Everything here is a memory-bound stream: 64-lane wavefronts,
** 16-byte accesses per lane where the element type allows, workgroups
** striding over tiles of 4096 elements, no matrix cores.
**
** Replaces (does not port) the reference's device step, num/gpu_cuda.cu:8417-8712:
** the arithmetic follows the reference's HOST loop (lang/lm_adam.c:571-598) in
** double, see adam_math.h.
*/
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>
#include "adam_kernels.h"

namespace anni {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

/*
** The launch table (tile -> tensor, the tensors' bounds, the per-tensor scales) is only read by
** the step's kernels.  Read through the constant address space it comes in by scalar loads, which
** have a counter of their own: a lookup does not wait for the vector loads in flight.
*/
#define ANNI_CONSTANT __attribute__((address_space(4)))
template <typename T>
__device__ __forceinline__ const ANNI_CONSTANT T *table(const T *p)
{
	return (const ANNI_CONSTANT T *)p;
}

/* ---- typed quad access ------------------------------------------------- */

template <bool NT, typename T>
__device__ __forceinline__ T ld(const T *p)
{
	if (NT)
		return __builtin_nontemporal_load(p);
	return *p;
}

template <bool NT, typename T>
__device__ __forceinline__ void st(T *p, T v)
{
	if (NT)
		__builtin_nontemporal_store(v, p);
	else
		*p = v;
}

/* Four consecutive values of a typed array as they lie in memory (16, 8 or 4 bytes). */
template <int T> struct RawQuad;
template <> struct RawQuad<kF32> { f32x4 v; };
template <> struct RawQuad<kBF16> { u32x2 v; };
template <> struct RawQuad<kFP8> { uint32_t v; };

template <int T, bool NT>
__device__ __forceinline__ RawQuad<T> load_raw(const void *base, int64_t i)
{
	RawQuad<T> r;

	if constexpr (T == kF32)
		r.v = ld<NT>((const f32x4 *)((const float *)base + i));
	else if constexpr (T == kBF16)
		r.v = ld<NT>((const u32x2 *)((const uint16_t *)base + i));
	else
		r.v = ld<NT>((const uint32_t *)((const uint8_t *)base + i));
	return r;
}

/* The four values as floats: bf16 widens exactly, E4M3 decodes exactly and is multiplied by scale. */
template <int T>
__device__ __forceinline__ f32x4 widen_raw(const RawQuad<T> &q, float scale)
{
	f32x4 r;

	if constexpr (T == kF32) {
		r = q.v;
	} else if constexpr (T == kBF16) {
		r.x = __uint_as_float(q.v.x << 16);
		r.y = __uint_as_float(q.v.x & 0xffff0000u);
		r.z = __uint_as_float(q.v.y << 16);
		r.w = __uint_as_float(q.v.y & 0xffff0000u);
	} else {
		const f32x2_t lo = fp8_e4m3_decode2(q.v, false);
		const f32x2_t hi = fp8_e4m3_decode2(q.v, true);

		r.x = lo.x * scale;
		r.y = lo.y * scale;
		r.z = hi.x * scale;
		r.w = hi.y * scale;
	}
	return r;
}

/* Four consecutive values of a typed array, starting at element i (i % 4 == 0), as floats. */
template <int T, bool NT>
__device__ __forceinline__ f32x4 load_quad(const void *base, int64_t i, float scale)
{
	return widen_raw<T>(load_raw<T, NT>(base, i), scale);
}

/* Stores four floats into an f32 or bf16 array (bf16: round to nearest even). */
template <int T, bool NT>
__device__ __forceinline__ void store_quad(void *base, int64_t i, f32x4 x)
{
	if (T == kF32) {
		st<NT>((f32x4 *)((float *)base + i), x);
	} else {
		u32x2 w;

		w.x = bf16_rne2(x.x, x.y);
		w.y = bf16_rne2(x.z, x.w);
		st<NT>((u32x2 *)((uint16_t *)base + i), w);
	}
}

template <int T, bool NT>
__device__ __forceinline__ void zero_quad(void *base, int64_t i)
{
	if (T == kF32) {
		const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};

		st<NT>((f32x4 *)((float *)base + i), z);
	} else if (T == kBF16) {
		const u32x2 z = {0u, 0u};

		st<NT>((u32x2 *)((uint16_t *)base + i), z);
	} else {
		st<NT>((uint32_t *)((uint8_t *)base + i), 0u);
	}
}

template <int T>
__device__ __forceinline__ float load_one(const void *base, int64_t i, float scale)
{
	if (T == kF32)
		return ((const float *)base)[i];
	if (T == kBF16)
		return bf16_widen(((const uint16_t *)base)[i]);
	return fp8_e4m3_decode(((const uint8_t *)base)[i]) * scale;
}

template <int T>
__device__ __forceinline__ void store_one(void *base, int64_t i, float x)
{
	if (T == kF32)
		((float *)base)[i] = x;
	else
		((uint16_t *)base)[i] = (uint16_t)bf16_rne(x);
}

template <int T>
__device__ __forceinline__ void zero_one(void *base, int64_t i)
{
	if (T == kF32)
		((float *)base)[i] = 0.0f;
	else if (T == kBF16)
		((uint16_t *)base)[i] = 0;
	else
		((uint8_t *)base)[i] = 0;
}

/* ---- reductions --------------------------------------------------------- */

/*
** Sum over the 256 lanes of a workgroup in a fixed tree: shuffles inside each
** 64-lane wavefront, then the four wavefront sums through LDS in index order.
** Every lane returns the same total.  lds must hold 4 doubles.
*/
__device__ __forceinline__ double block_sum(double x, double *lds)
{
	const int tid = threadIdx.x;

#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		x += __shfl_down(x, off, 64);
	if ((tid & 63) == 0)
		lds[tid >> 6] = x;
	__syncthreads();
	const double total = (lds[0] + lds[1]) + (lds[2] + lds[3]);
	__syncthreads();
	return total;
}

/* ---- derived outputs ------------------------------------------------------ */

/* Max over the 64 lanes of a wavefront; lane 0 holds it. */
__device__ __forceinline__ float wave_max(float x)
{
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		x = fmaxf(x, __shfl_down(x, off, 64));
	return x;
}

/* max |x| of four values; NaNs are ignored (fmaxf returns the other operand). */
__device__ __forceinline__ float amax4(float acc, f32x4 x)
{
	return fmaxf(acc, fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
}

/*
** Raises *word to the bits of m (m > 0, not NaN; such floats order like unsigned integers).
** The word only grows during a launch, so a stale read costs at most a redundant atomic.
*/
__device__ __forceinline__ void amax_raise(uint32_t *word, float m)
{
	const uint32_t bits = __float_as_uint(m);

	if (bits > __atomic_load_n(word, __ATOMIC_RELAXED))
		atomicMax(word, bits);
}

/* bf16 of element e of a packed tensor into its place in the packed matrix. */
__device__ __forceinline__ void pack_one(uint16_t *pack, const PackDesc &pd, uint32_t e, float x)
{
	const uint32_t r = e / pd.cols;
	const uint32_t c = e - r * pd.cols;

	pack[pd.dst_off + (int64_t)r * pd.dst_stride + c] = (uint16_t)bf16_rne(x);
}

/* The same for elements e..e+3: one 8-byte store when they share a row and the target is aligned. */
template <bool NT>
__device__ __forceinline__ void pack_quad(uint16_t *pack, const PackDesc &pd, uint32_t e, f32x4 x)
{
	const uint32_t r = e / pd.cols;
	const uint32_t c = e - r * pd.cols;
	const int64_t d = pd.dst_off + (int64_t)r * pd.dst_stride + c;

	if (c + kQuad <= pd.cols && (d & 3) == 0) {
		store_quad<kBF16, NT>(pack, d, x);
	} else {
		pack_one(pack, pd, e, x.x);
		pack_one(pack, pd, e + 1, x.y);
		pack_one(pack, pd, e + 2, x.z);
		pack_one(pack, pd, e + 3, x.w);
	}
}

struct NormOut {
	double	gs;
	bool	skip;
};

/*
** norm = sqrt(sum); a non-finite norm skips the step (lang/lm_adam.c:474-483);
** norm > clip scales the gradients by clip / (norm + 1e-12) (lm_adam.c:581-585).
*/
__device__ __forceinline__ NormOut norm_decide(double ss, double clip, int skip_nonfinite,
	double grad_scale, StepState *state, bool writer)
{
	NormOut o;
	const double norm = sqrt(ss);
	const bool bad = skip_nonfinite && !(fabs(norm) <= 1.7976931348623157e308);
	const bool clipped = !bad && clip > 0.0 && norm > clip;

	o.gs = grad_scale;
	o.skip = bad;
	if (clipped)
		o.gs = grad_scale * (clip / (norm + 1e-12));
	if (writer && state) {
		state->sumsq = ss;
		state->norm = norm;
		state->grad_scale = o.gs;
		state->skipped = bad ? 1 : 0;
		state->clipped = clipped ? 1 : 0;
	}
	return o;
}

/* ---- sum of squares ------------------------------------------------------ */

struct SumsqArgs {
	const void	*g;
	int64_t		n;
	const Seg	*segs;
	const int32_t	*tile_seg;
	const float	*gscale;
	double		grad_scale;
	double		*partials;
	int		vec_ok;
	int64_t		keep_from;	/* chunks from here on are read with ordinary (cacheable) loads */
	/* second stage (ticket == NULL: partials only) */
	unsigned int	*ticket;
	double		clip;
	int		skip_nonfinite;
	StepState	*state;
	int		fence;		/* 1: the conservative hand-over (fences) instead of atomic accesses */
};

/*
** Second stage of the norm, inside the same launch: every workgroup stores its partial and
** draws a ticket; the one that draws the last ticket knows that all partials are in memory, folds
** them in index order -- the same sum whichever workgroup it is -- decides clip and skip, stores
** the step state for the kernels that follow, and puts the ticket counters back to zero for the
** next launch.  Nobody waits for anybody.  `state` may lie in page-locked host memory.
**
** The compute dies have a level-two cache each, so a release / acquire pair at device scope
** writes back and invalidates whole caches -- 2048 of those at the end of the kernel were
** measured at 0.1 ms.  Instead the partials themselves travel as device-scope atomic accesses,
** which are performed where all dies see them: the partial is stored by an exchange whose result
** the ticket increment consumes (so the increment cannot be issued before the exchange has been
** performed), and the last workgroup reads the partials with atomic loads after its own increment
** has returned.  What this relies on, beyond the letter of the HIP memory model (which orders
** relaxed atomics on different addresses only through fences): on gfx950 a returning atomic is
** complete -- performed at the memory side that all dies share -- when its value arrives, an
** instruction that consumes that value cannot issue earlier, and agent-scope atomic accesses are
** performed there and not in a die's own level-two cache.  ANNI_FOLD=fence selects the hand-over
** that needs none of this: plain stores of the partials, a release fence at device scope before
** the tickets, an acquire fence in the last workgroup before it reads (+0.1 ms per launch at
** 555M); the test of the switches holds the two against each other bit for bit.
*/
constexpr int kFoldAhead = 8;	/* partials a lane of the last workgroup has in flight */

__device__ __forceinline__ void sumsq_finish(const SumsqArgs &a, double total, double *lds,
	int *last)
{
	unsigned long long *cells = (unsigned long long *)a.partials;

	if (threadIdx.x == 0) {
		*last = 0;
		if (a.ticket) {
			/*
			** Two levels of tickets: 2048 increments of one word, which the memory side takes
			** one after the other, were measured at 15 us.  Workgroup b draws from the counter
			** of group b mod 64; who draws a group's last ticket draws from the counter above.
			*/
			const unsigned int groups = gridDim.x < (unsigned int)kTicketGroups ? gridDim.x
			    : (unsigned int)kTicketGroups;
			const unsigned int g = blockIdx.x % (unsigned int)kTicketGroups;
			const unsigned int members = (gridDim.x - g + kTicketGroups - 1) / kTicketGroups;
			unsigned int one = 1u;

			if (a.fence) {
				a.partials[blockIdx.x] = total;
				__builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
			} else {
				const unsigned long long old = __hip_atomic_exchange(cells + blockIdx.x,
				    (unsigned long long)__double_as_longlong(total), __ATOMIC_RELAXED,
				    __HIP_MEMORY_SCOPE_AGENT);

				/* ties the increment to the exchange's result: it waits for the exchange to return */
				asm volatile("" : "+v"(one) : "v"(old));
			}
			if (__hip_atomic_fetch_add(a.ticket + (1 + g) * kTicketStride, one, __ATOMIC_RELAXED,
			    __HIP_MEMORY_SCOPE_AGENT) == members - 1u) {
				/* the value just returned decided this branch: the next increment follows it */
				*last = __hip_atomic_fetch_add(a.ticket, 1u, __ATOMIC_RELAXED,
				    __HIP_MEMORY_SCOPE_AGENT) == groups - 1u ? 1 : 0;
			}
		} else {
			a.partials[blockIdx.x] = total;
		}
	}
	__syncthreads();
	if (!*last)
		return;
	if (a.fence)
		__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
	/* lane l adds the partials l, l + 256, ... in that order, then the fixed tree over the lanes */
	double acc = 0.0;

	for (unsigned int i0 = threadIdx.x; i0 < gridDim.x; i0 += kFoldAhead * kThreads) {
		unsigned long long raw[kFoldAhead];

#pragma unroll
		for (int k = 0; k < kFoldAhead; k++) {
			const unsigned int i = i0 + (unsigned int)k * kThreads;

			raw[k] = i < gridDim.x ? __hip_atomic_load(cells + i, __ATOMIC_RELAXED,
			    __HIP_MEMORY_SCOPE_AGENT) : 0ull;
		}
#pragma unroll
		for (int k = 0; k < kFoldAhead; k++)
			if (i0 + (unsigned int)k * kThreads < gridDim.x)
				acc += __longlong_as_double((long long)raw[k]);
	}
	const double ss = block_sum(acc, lds);

	(void)norm_decide(ss, a.clip, a.skip_nonfinite, a.grad_scale, a.state, threadIdx.x == 0);
	if (threadIdx.x <= (unsigned int)kTicketGroups)
		__hip_atomic_store(a.ticket + threadIdx.x * kTicketStride, 0u, __ATOMIC_RELAXED,
		    __HIP_MEMORY_SCOPE_AGENT);
}

/*
** The sum walks the gradient flat in chunks of 16 KiB whatever the element type -- 4096 floats,
** 8192 bf16 values or 16384 E4M3 codes: one chunk is four 16-byte loads per lane, 4 KiB apart,
** all in flight together.  (Loads of several places a grid width apart in flight at once were
** measured slower, up to 35 % with bf16; narrower loads of one place reach 6.0 instead of 6.7 TB/s.)
** Whole chunks of f32 and bf16 gradients need nothing from the launch table.  E4M3 codes carry a
** scale per tensor: sum = SUM over tensors of (scale_t * gs)^2 * SUM_i decode(q_i)^2 -- the square
** of an E4M3 value is exact in float and a lane's sum of sixteen of them exact in double, so only
** the products round; each 4 KiB quarter of a chunk is one tile of the launch table, and a quarter
** shared by several tensors goes element by element.
*/
template <int GT>
struct SumsqChunk {
	static constexpr int64_t kBytes = 16384;
	static constexpr int64_t kElems = kBytes / (GT == kF32 ? 4 : GT == kBF16 ? 2 : 1);
};

/* Elements [from, to) one by one; s = the tensor of `from` (fp8 only). */
template <int GT>
__device__ __forceinline__ void sumsq_slow(const SumsqArgs &a, int64_t from, int64_t to, int s, int tid,
	double (&acc)[4])
{
	for (int64_t i = from + tid; i < to; i += kThreads) {
		if (GT == kFP8) {
			if (a.segs)
				while (i >= table(a.segs)[s].end)
					s++;
			const double sc = (double)table(a.gscale)[s] * a.grad_scale;
			const float d = fp8_e4m3_decode(((const uint8_t *)a.g)[i]);

			acc[0] += (sc * sc) * (double)(d * d);
		} else {
			const double x = (double)load_one<GT>(a.g, i, 1.0f) * a.grad_scale;

			acc[0] += x * x;
		}
	}
}

/* The chunks first, first + step, ... below `stop`, added to the lane's running sums in that order. */
template <int GT, bool NT>
__device__ __forceinline__ int64_t sumsq_chunks(const SumsqArgs &a, int64_t first, int64_t step,
	int64_t stop, int tid, double (&acc)[4])
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	constexpr int64_t kElems = SumsqChunk<GT>::kElems;
	int64_t c = first;

	for (; c < stop; c += step) {
		const int64_t base = c * kElems;

		if (a.vec_ok && base + kElems <= a.n) {
			const u32x4 *src = (const u32x4 *)((const uint8_t *)a.g + c * SumsqChunk<GT>::kBytes) + tid;
			u32x4 W[4];

#pragma unroll
			for (int u = 0; u < 4; u++)
				W[u] = ld<NT>(src + u * kThreads);
#pragma unroll
			for (int u = 0; u < 4; u++) {
				if constexpr (GT == kF32) {
#pragma unroll
					for (int k = 0; k < 4; k++) {
						const double x = (double)__uint_as_float(W[u][k]) * a.grad_scale;

						acc[k] += x * x;
					}
				} else if constexpr (GT == kBF16) {
#pragma unroll
					for (int k = 0; k < 4; k++) {
						const double lo = (double)__uint_as_float(W[u][k] << 16) * a.grad_scale;
						const double hi = (double)__uint_as_float(W[u][k] & 0xffff0000u) * a.grad_scale;

						acc[(2 * k) & 3] += lo * lo;
						acc[(2 * k + 1) & 3] += hi * hi;
					}
				} else {
					/* quarter u of the chunk is tile 4 c + u of the launch table */
					const int64_t tile = c * 4 + u;
					const int s = a.tile_seg ? table(a.tile_seg)[tile] : 0;
					const int64_t seg_end = a.segs ? table(a.segs)[s].end : a.n;

					if (seg_end >= (tile + 1) * kTile) {
						const double sc = (double)table(a.gscale)[s] * a.grad_scale;
						double t = 0.0;

#pragma unroll
						for (int k = 0; k < 4; k++) {
							const f32x2_t lo = fp8_e4m3_decode2(W[u][k], false);
							const f32x2_t hi = fp8_e4m3_decode2(W[u][k], true);

							t += (double)(lo.x * lo.x);
							t += (double)(lo.y * lo.y);
							t += (double)(hi.x * hi.x);
							t += (double)(hi.y * hi.y);
						}
						acc[0] += (sc * sc) * t;
					} else {
						sumsq_slow<GT>(a, tile * kTile, (tile + 1) * kTile, s, tid, acc);
					}
				}
			}
		} else {
			const int64_t end = base + kElems < a.n ? base + kElems : a.n;
			int s = 0;

			if (GT == kFP8 && a.tile_seg)
				s = table(a.tile_seg)[base / kTile];
			sumsq_slow<GT>(a, base, end, s, tid, acc);
		}
	}
	return c;
}

/*
** A workgroup takes the chunks blockIdx.x, blockIdx.x + gridDim.x, ... in rising order.  The
** chunks from `keep_from` on are read with ordinary loads, so the memory-side cache keeps them for
** the update kernel that follows; the others stream past it.
*/
template <int GT, bool NT>
__global__ __launch_bounds__(kThreads) void sumsq_kernel(SumsqArgs a)
{
	__shared__ double lds[4];
	__shared__ int last;
	const int tid = threadIdx.x;
	const int64_t n_chunks = (a.n + SumsqChunk<GT>::kElems - 1) / SumsqChunk<GT>::kElems;
	const int64_t keep_from = NT ? (a.keep_from < n_chunks ? a.keep_from : n_chunks) : 0;
	double acc[4] = {0.0, 0.0, 0.0, 0.0};
	int64_t c;

	c = sumsq_chunks<GT, NT>(a, blockIdx.x, gridDim.x, keep_from, tid, acc);
	(void)sumsq_chunks<GT, false>(a, c, gridDim.x, n_chunks, tid, acc);
	const double total = block_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), lds);

	sumsq_finish(a, total, lds, &last);
}

/* ---- sum of squares of a float flat, one partial per chunk ------------------------------ */

/*
** The flat entry point (gpu_grad_sumsq) sums in two steps that can be taken apart: first every
** 16 KiB chunk of the flat gets a partial sum, computed by one wavefront alone (shuffles only, no
** barrier, nothing shared), then the partials are folded in index order -- chunk_fold_kernel
** over contiguous runs, chunk_final_kernel over the runs' sums.  The result is a pure function of
** the flat: it does not depend on the grid, and recomputing the partials of some chunks after
** their elements changed gives bit for bit what a pass over the whole flat gives.  That is what
** lets the backend begin the sum before the caller asks for it (gpu_backend.hip, "the sum begun
** early") and repair the few chunks the caller still writes afterwards.
*/
struct ChunkSumArgs {
	const float	*x;
	int64_t		n;
	double		*part;		/* one per chunk */
	const int32_t	*list;		/* NULL: every chunk; else the chunks to (re)compute, one per wavefront */
	int		n_list;
	int		vec_ok;
	int64_t		keep_from;	/* chunks from here on are read with ordinary (cacheable) loads */
};

/*
** The sum of the squares of chunk c, by ONE wavefront: lane l reads the 16 bytes at l, l + 64, ...,
** l + 960 (in units of 16 bytes: sixteen loads, 1 KiB of the chunk per load instruction, all in
** flight together), adds the squares of each of the four floats of a load to a chain of its own,
** and the wavefront folds by shuffles.  The result is in lane 0.  A chunk that runs past the flat,
** or a flat that is not 16-byte aligned, goes element by element.
*/
template <bool NT>
__device__ __forceinline__ double chunk_sum_wave(const ChunkSumArgs &a, int64_t c, int lane)
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	constexpr int64_t kElems = SumsqChunk<kF32>::kElems;
	constexpr int kLoads = (int)(SumsqChunk<kF32>::kBytes / (64 * 16));
	const int64_t base = c * kElems;
	double acc[4] = {0.0, 0.0, 0.0, 0.0};
	double x;

	if (a.vec_ok && base + kElems <= a.n) {
		const u32x4 *src = (const u32x4 *)(a.x + base) + lane;
		u32x4 W[kLoads];

#pragma unroll
		for (int u = 0; u < kLoads; u++)
			W[u] = ld<NT>(src + u * 64);
#pragma unroll
		for (int u = 0; u < kLoads; u++) {
#pragma unroll
			for (int k = 0; k < 4; k++) {
				const double v = (double)__uint_as_float(W[u][k]);

				acc[k] += v * v;
			}
		}
	} else {
		const int64_t end = base + kElems < a.n ? base + kElems : a.n;

		for (int64_t i = base + lane; i < end; i += 64) {
			const double v = (double)a.x[i];

			acc[0] += v * v;
		}
	}
	x = (acc[0] + acc[1]) + (acc[2] + acc[3]);
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		x += __shfl_down(x, off, 64);
	return x;
}

/*
** Wavefront w of workgroup b takes the chunks 4 b + w, 4 (b + gridDim.x) + w, ...: a workgroup
** walks the flat in pieces of 64 KiB, each wavefront a contiguous quarter, and no wavefront waits
** for another.  With a list, wavefront 4 b + w takes the chunk list[4 b + w].
*/
template <bool NT>
__global__ __launch_bounds__(kThreads) void chunk_sums_kernel(ChunkSumArgs a)
{
	constexpr int64_t kElems = SumsqChunk<kF32>::kElems;
	const int lane = threadIdx.x & 63;
	const int64_t wave = (int64_t)blockIdx.x * kWaves + (threadIdx.x >> 6);
	const int64_t n_chunks = (a.n + kElems - 1) / kElems;

	if (a.list) {
		if (wave < a.n_list) {
			const int64_t c = (int64_t)a.list[wave];

			if (c >= 0 && c < n_chunks) {
				const double x = (NT && c < a.keep_from) ? chunk_sum_wave<true>(a, c, lane)
				    : chunk_sum_wave<false>(a, c, lane);

				if (lane == 0)
					a.part[c] = x;
			}
		}
		return;
	}
	for (int64_t c = wave; c < n_chunks; c += (int64_t)gridDim.x * kWaves) {
		const double x = (NT && c < a.keep_from) ? chunk_sum_wave<true>(a, c, lane)
		    : chunk_sum_wave<false>(a, c, lane);

		if (lane == 0)
			a.part[c] = x;
	}
}

/* run[g] = sum of part[g * per .. min((g + 1) * per, count)) : lane l adds every 256th, then the fixed tree. */
__global__ __launch_bounds__(kThreads) void chunk_fold_kernel(const double *part, int64_t count, int64_t per,
	double *run)
{
	__shared__ double lds[4];
	const int64_t lo = (int64_t)blockIdx.x * per;
	const int64_t hi = lo + per < count ? lo + per : count;
	double acc = 0.0;

	for (int64_t i0 = lo + threadIdx.x; i0 < hi; i0 += (int64_t)kFoldAhead * kThreads) {
		double v[kFoldAhead];

#pragma unroll
		for (int k = 0; k < kFoldAhead; k++) {
			const int64_t i = i0 + (int64_t)k * kThreads;

			v[k] = i < hi ? part[i] : 0.0;
		}
#pragma unroll
		for (int k = 0; k < kFoldAhead; k++)
			if (i0 + (int64_t)k * kThreads < hi)
				acc += v[k];
	}
	const double total = block_sum(acc, lds);

	if (threadIdx.x == 0)
		run[blockIdx.x] = total;
}

/* The runs' sums in index order -> the state (state may lie in page-locked host memory). */
__global__ __launch_bounds__(kThreads) void chunk_final_kernel(const double *run, int n_runs, StepState *state)
{
	__shared__ double lds[4];
	double acc = 0.0;

	for (int i = threadIdx.x; i < n_runs; i += kThreads)
		acc += run[i];
	const double ss = block_sum(acc, lds);

	(void)norm_decide(ss, 0.0, 0, 1.0, state, threadIdx.x == 0);
}

/*
** The three kernels above in one launch, for a caller who waits for the result: every kernel
** boundary on one stream costs about 10 us here.  Workgroup r owns run r.  It first computes anew
** the partials of those chunks of its run that are named in `fix` (rising, at most kFixMax, in the
** kernel's arguments), then folds its run exactly as chunk_fold_kernel does, then hands the run's
** sum over as the sum of squares' second stage does (sumsq_finish): whoever draws the last ticket
** folds the runs' sums as chunk_final_kernel does.  Same additions in the same order: same bits.
** The partials a workgroup has just written are read back by its other wavefronts; both sides use
** device-scope atomic accesses with the barrier between them, so no cache of a compute unit can
** stand in between.
*/
constexpr int kFixMax = 768;

struct ChunkFinishArgs {
	ChunkSumArgs	sum;		/* list unused */
	int64_t		count;		/* partials in all */
	int64_t		per;		/* partials per run */
	SumsqArgs	fin;		/* partials = the runs' sums, ticket, state, fence */
	unsigned long long	*stamp;	/* may be NULL: receives `token` once the state is stored */
	unsigned long long	token;
	int		n_fix;
	int32_t		fix[kFixMax];
};

template <bool NT>
__global__ __launch_bounds__(kThreads) void chunk_finish_kernel(ChunkFinishArgs a)
{
	__shared__ double lds[4];
	__shared__ int last;
	__shared__ int32_t fix_s[kFixMax];
	unsigned long long *cells = (unsigned long long *)a.sum.part;
	const int tid = threadIdx.x;
	const int64_t lo = (int64_t)blockIdx.x * a.per;
	const int64_t hi = lo + a.per < a.count ? lo + a.per : a.count;
	const int32_t c_lo = (int32_t)lo;	/* one partial per chunk */
	const int32_t c_hi = (int32_t)hi;
	int at = 0;
	double acc = 0.0;

	if (a.n_fix > 0) {
		int len = a.n_fix;

		/*
		** The list into LDS first, all lanes at once: the kernel's arguments may lie in host
		** memory, where every step of a search would be a trip over the host link of its own.
		*/
		for (int i = tid; i < a.n_fix; i += kThreads)
			fix_s[i] = a.fix[i];
		__syncthreads();
		/* the first entry not below c_lo (the same for every lane) */
		while (len > 0) {
			const int half = len / 2;

			if (fix_s[at + half] < c_lo) {
				at += half + 1;
				len -= half + 1;
			} else {
				len = half;
			}
		}
		/* the run's chunks on the list, dealt to the four wavefronts in turn */
		for (int i = at + (tid >> 6); i < a.n_fix && fix_s[i] < c_hi; i += kWaves) {
			const int64_t c = fix_s[i];
			const double x = (NT && c < a.sum.keep_from) ? chunk_sum_wave<true>(a.sum, c, tid & 63)
			    : chunk_sum_wave<false>(a.sum, c, tid & 63);

			if ((tid & 63) == 0)
				__hip_atomic_store(cells + c, (unsigned long long)__double_as_longlong(x),
				    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		}
		__syncthreads();
	}
	for (int64_t i0 = lo + tid; i0 < hi; i0 += (int64_t)kFoldAhead * kThreads) {
		unsigned long long v[kFoldAhead];

#pragma unroll
		for (int k = 0; k < kFoldAhead; k++) {
			const int64_t i = i0 + (int64_t)k * kThreads;

			v[k] = i < hi ? __hip_atomic_load(cells + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
			    : 0ull;
		}
#pragma unroll
		for (int k = 0; k < kFoldAhead; k++)
			if (i0 + (int64_t)k * kThreads < hi)
				acc += __longlong_as_double((long long)v[k]);
	}
	const double total = block_sum(acc, lds);

	__syncthreads();		/* lds is used again below */
	sumsq_finish(a.fin, total, lds, &last);
	/* the lane that stored the state tells a host that is watching `stamp` (page-locked memory) */
	if (last && a.stamp && tid == 0) {
		__threadfence_system();
		__hip_atomic_store(a.stamp, a.token, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
	}
}

/* ---- the update ---------------------------------------------------------- */

struct UpdateArgs {
	float		*p;
	void		*g;
	void		*m;
	void		*v;
	uint16_t	*twin;
	int64_t		n;
	const Seg	*segs;
	const int32_t	*tile_seg;
	const float	*gscale;
	uint32_t	uniform_flags;
	int		vec_ok;
	int		reverse;	/* walk the tiles from the last to the first */
	const int32_t	*order;		/* not NULL: only the tiles order[0 .. turns), in that order (adam_update_kernel) */
	int64_t		turns;
	StepConsts	c;
	double		grad_scale;
	int		use_norm;	/* scale and skip come from *state, stored by the sum of squares */
	const StepState	*state;
	Derived		der;
};

/*
** What a workgroup needs to know about a tile before it can issue the tile's loads: a chain of
** dependent scalar loads (tile -> tensor -> end, flags, scale).  The kernels look it up one tile
** ahead, so the chain runs while the current tile is computed.
*/
struct TileInfo {
	int64_t		tile;	/* the tile's place in the flat */
	int64_t		base;
	int64_t		end;
	int		s;
	uint32_t	flags;
	float		sc;	/* fp8 gradients: the tensor's scale */
	bool		whole;
	bool		vec;	/* a whole tile inside one tensor, not skipped: the vector path */
};

template <int GT>
__device__ __forceinline__ TileInfo tile_info(const UpdateArgs &a, int64_t turn, bool skip)
{
	TileInfo t;
	const int64_t tile = a.order ? (int64_t)a.order[turn]
	    : a.reverse ? (a.n + kTile - 1) / kTile - 1 - turn : turn;

	t.tile = tile;
	t.base = tile * kTile;
	t.end = t.base + kTile < a.n ? t.base + kTile : a.n;
	t.s = a.tile_seg ? a.tile_seg[tile] : 0;
	t.flags = a.segs ? a.segs[t.s].flags : a.uniform_flags;
	t.sc = (GT == kFP8) ? a.gscale[t.s] : 1.0f;
	t.whole = a.vec_ok && t.end - t.base == kTile;
	t.vec = t.whole && !skip && (a.segs ? a.segs[t.s].end : a.n) >= t.end;
	return t;
}

/*
** U = quads a lane keeps in flight at once (kQuadsPerTile % U == 0); the whole tile in every mode
** (half the tile was measured 0.5 % slower in the all-f32 mode).  With narrow storage types the
** kernel moves fewer bytes per element for the same arithmetic, so those modes take the cheaper
** constant division (adam_math.h).
*/
template <int GT, int MT, int U, bool NT, bool DER>
__global__ __launch_bounds__(kThreads) void adam_update_kernel(UpdateArgs a)
{
	const int tid = threadIdx.x;
	const int64_t n_tiles = a.order ? a.turns : (a.n + kTile - 1) / kTile;
	double gs = a.grad_scale;
	bool skip = false;

	if (a.use_norm) {
		gs = a.state->grad_scale;
		skip = a.state->skipped != 0;
	}
	TileInfo cur = tile_info<GT>(a, blockIdx.x < n_tiles ? (int64_t)blockIdx.x : 0, skip);

	for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
		const int64_t ahead = tile + gridDim.x < n_tiles ? tile + gridDim.x : tile;
		const TileInfo nxt = tile_info<GT>(a, ahead, skip);	/* used after this tile */
		const int64_t base = cur.base;
		const int64_t end = cur.end;
		int s = cur.s;
		const bool whole = cur.whole;
		const bool vec = cur.vec;
		const uint32_t flags = cur.flags;
		const float sc = cur.sc;
		const int64_t place = cur.tile;

		cur = nxt;
		if (skip) {
			/* Non-finite norm: p, m, v and the twins stay as they are; gradients are cleared. */
			if (whole) {
#pragma unroll
				for (int u = 0; u < kQuadsPerTile; u++)
					zero_quad<GT, NT>(a.g, base + (int64_t)(u * kThreads + tid) * kQuad);
			} else {
				for (int64_t i = base + tid; i < end; i += kThreads)
					zero_one<GT>(a.g, i);
			}
			continue;
		}
		if (vec) {
			const bool decay = a.c.decay_on && (flags & kSegDecay) != 0;
			const bool twin = (flags & kSegTwin) != 0 && a.twin != nullptr;
			const bool fp8w = DER && (flags & kSegFp8Twin) != 0 && a.der.wamax != nullptr;
			const bool pk = DER && (flags & kSegPack) != 0 && a.der.pack != nullptr;
			PackDesc pd = {0, 1u, 0u};
			int64_t seg_begin = 0;
			float amax_l = 0.0f;

			if (pk) {
				pd = a.der.packs[s];
				seg_begin = a.segs[s].begin;
			}
#pragma unroll
			for (int sub = 0; sub < kQuadsPerTile / U; sub++) {
				f32x4 P[U], G[U], M[U], V[U];
				int64_t idx[U];

#pragma unroll
				for (int u = 0; u < U; u++) {
					idx[u] = base + (int64_t)((sub * U + u) * kThreads + tid) * kQuad;
					G[u] = load_quad<GT, NT>(a.g, idx[u], sc);
					M[u] = load_quad<MT, NT>(a.m, idx[u], 1.0f);
					V[u] = load_quad<MT, NT>(a.v, idx[u], 1.0f);
					P[u] = load_quad<kF32, NT>(a.p, idx[u], 1.0f);
				}
#pragma unroll
				for (int u = 0; u < U; u++) {
#pragma unroll
					for (int k = 0; k < kQuad; k++) {
						const Elem e = adam_elem<(GT != kF32 || MT != kF32)>(P[u][k],
						    G[u][k], M[u][k], V[u][k], gs, a.c, decay);

						P[u][k] = e.p;
						M[u][k] = e.m;
						V[u][k] = e.v;
					}
				}
#pragma unroll
				for (int u = 0; u < U; u++) {
					store_quad<kF32, NT>(a.p, idx[u], P[u]);
					store_quad<MT, NT>(a.m, idx[u], M[u]);
					store_quad<MT, NT>(a.v, idx[u], V[u]);
					zero_quad<GT, NT>(a.g, idx[u]);
					if (twin)
						store_quad<kBF16, NT>(a.twin, idx[u], P[u]);
					if (fp8w)
						amax_l = amax4(amax_l, P[u]);
					if (pk)
						pack_quad<NT>(a.der.pack, pd, (uint32_t)(idx[u] - seg_begin), P[u]);
				}
			}
			if (fp8w) {
				amax_l = wave_max(amax_l);
				if ((tid & 63) == 0)
					a.der.tile_amax[place * kWaves + (tid >> 6)] = amax_l;
			}
		} else {
			for (int64_t i = base + tid; i < end; i += kThreads) {
				uint32_t flags = a.uniform_flags;
				float sc = 1.0f;

				if (a.segs) {
					while (i >= a.segs[s].end)
						s++;
					flags = a.segs[s].flags;
				}
				if (GT == kFP8)
					sc = a.gscale[s];
				const Elem e = adam_elem<(GT != kF32 || MT != kF32)>(a.p[i], load_one<GT>(a.g, i, sc),
				    load_one<MT>(a.m, i, 1.0f), load_one<MT>(a.v, i, 1.0f), gs, a.c,
				    a.c.decay_on && (flags & kSegDecay) != 0);

				a.p[i] = e.p;
				store_one<MT>(a.m, i, e.m);
				store_one<MT>(a.v, i, e.v);
				zero_one<GT>(a.g, i);
				if ((flags & kSegTwin) != 0 && a.twin != nullptr)
					a.twin[i] = (uint16_t)bf16_rne(e.p);
				if (DER && (flags & kSegFp8Twin) != 0 && a.der.wamax != nullptr) {
					const float ab = fmaxf(0.0f, fabsf(e.p));

					if (ab > 0.0f)
						amax_raise(a.der.wamax + s, ab);
				}
				if (DER && (flags & kSegPack) != 0 && a.der.pack != nullptr)
					pack_one(a.der.pack, a.der.packs[s], (uint32_t)(i - a.segs[s].begin), e.p);
			}
		}
	}
}

/* ---- the same update, software-pipelined (narrow storage modes) ----------------------- */

/*
** With bf16 moments or narrow gradients the update moves 22 - 28 bytes per element for the same
** arithmetic (~90 vector instructions per element, 55 of them double precision), and it shows: a
** wavefront that computes issues no memory instruction for thousands of cycles, and the memory
** pipeline runs dry whenever all wavefronts of a SIMD compute (a kernel with the same nine
** streams and no arithmetic is 9 % faster).  So here every wavefront has the loads of its NEXT tile in flight
** while it computes the current one: two register stages of half a tile each, used in turn
** (never copied -- a copy would wait for the loads it copies): while the first half of a tile is
** computed its second half is on the way, while the second half is computed the first half of
** the wavefront's next tile.  A stage holds the data as they lie in memory (16 + 8 + 8 + 8 bytes
** per quad with bf16 storage) and is widened quad by quad when it is consumed.  Half-tile stages
** need ~110 registers (whole-tile stages ~150) and were measured 0.6 % faster with fp8 gradients.
** Arithmetic, rounding points and stores are those of adam_update_kernel; results are
** bit-identical.
*/
/* A tile that is skipped, ragged or shared by several tensors: as in adam_update_kernel. */
template <int GT, int MT, bool NT, bool DER>
__device__ __forceinline__ void tile_slow(const UpdateArgs &a, const TileInfo &t, double gs,
	bool skip, int tid)
{
	int s = t.s;

	if (skip) {
		if (t.whole) {
#pragma unroll
			for (int u = 0; u < kQuadsPerTile; u++)
				zero_quad<GT, NT>(a.g, t.base + (int64_t)(u * kThreads + tid) * kQuad);
		} else {
			for (int64_t i = t.base + tid; i < t.end; i += kThreads)
				zero_one<GT>(a.g, i);
		}
		return;
	}
	for (int64_t i = t.base + tid; i < t.end; i += kThreads) {
		uint32_t flags = a.uniform_flags;
		float sc = 1.0f;

		if (a.segs) {
			while (i >= a.segs[s].end)
				s++;
			flags = a.segs[s].flags;
		}
		if (GT == kFP8)
			sc = a.gscale[s];
		const Elem e = adam_elem<(GT != kF32 || MT != kF32)>(a.p[i], load_one<GT>(a.g, i, sc),
		    load_one<MT>(a.m, i, 1.0f), load_one<MT>(a.v, i, 1.0f), gs, a.c,
		    a.c.decay_on && (flags & kSegDecay) != 0);

		a.p[i] = e.p;
		store_one<MT>(a.m, i, e.m);
		store_one<MT>(a.v, i, e.v);
		zero_one<GT>(a.g, i);
		if ((flags & kSegTwin) != 0 && a.twin != nullptr)
			a.twin[i] = (uint16_t)bf16_rne(e.p);
		if (DER && (flags & kSegFp8Twin) != 0 && a.der.wamax != nullptr) {
			const float ab = fmaxf(0.0f, fabsf(e.p));

			if (ab > 0.0f)
				amax_raise(a.der.wamax + s, ab);
		}
		if (DER && (flags & kSegPack) != 0 && a.der.pack != nullptr)
			pack_one(a.der.pack, a.der.packs[s], (uint32_t)(i - a.segs[s].begin), e.p);
	}
}

template <int GT, int MT>
struct HalfStage {
	f32x4		P[kQuadsPerTile / 2];
	RawQuad<GT>	G[kQuadsPerTile / 2];
	RawQuad<MT>	M[kQuadsPerTile / 2];
	RawQuad<MT>	V[kQuadsPerTile / 2];
};

template <int GT, int MT, bool NT, int Q0>
__device__ __forceinline__ void half_load(HalfStage<GT, MT> &st, const UpdateArgs &a, int64_t base,
	int tid)
{
#pragma unroll
	for (int u = 0; u < kQuadsPerTile / 2; u++) {
		const int64_t idx = base + (int64_t)((Q0 + u) * kThreads + tid) * kQuad;

		st.G[u] = load_raw<GT, NT>(a.g, idx);
		st.M[u] = load_raw<MT, NT>(a.m, idx);
		st.V[u] = load_raw<MT, NT>(a.v, idx);
		st.P[u] = ld<NT>((const f32x4 *)(a.p + idx));
	}
}

template <int GT, int MT, bool NT, bool DER, int Q0>
__device__ __forceinline__ void half_consume(const HalfStage<GT, MT> &st, const UpdateArgs &a,
	const TileInfo &t, double gs, int tid, float &amax_l)
{
	const int s = t.s;
	const uint32_t flags = t.flags;
	const bool decay = a.c.decay_on && (flags & kSegDecay) != 0;
	const bool twin = (flags & kSegTwin) != 0 && a.twin != nullptr;
	const float sc = t.sc;
	const bool fp8w = DER && (flags & kSegFp8Twin) != 0 && a.der.wamax != nullptr;
	const bool pk = DER && (flags & kSegPack) != 0 && a.der.pack != nullptr;
	PackDesc pd = {0, 1u, 0u};
	int64_t seg_begin = 0;

	if (pk) {
		pd = a.der.packs[s];
		seg_begin = a.segs[s].begin;
	}
#pragma unroll
	for (int u = 0; u < kQuadsPerTile / 2; u++) {
		const int64_t idx = t.base + (int64_t)((Q0 + u) * kThreads + tid) * kQuad;
		const f32x4 G = widen_raw<GT>(st.G[u], sc);
		f32x4 M = widen_raw<MT>(st.M[u], 1.0f);
		f32x4 V = widen_raw<MT>(st.V[u], 1.0f);
		f32x4 P = st.P[u];

#pragma unroll
		for (int k = 0; k < kQuad; k++) {
			const Elem e = adam_elem<(GT != kF32 || MT != kF32)>(P[k], G[k], M[k], V[k], gs, a.c,
			    decay);

			P[k] = e.p;
			M[k] = e.m;
			V[k] = e.v;
		}
		store_quad<kF32, NT>(a.p, idx, P);
		store_quad<MT, NT>(a.m, idx, M);
		store_quad<MT, NT>(a.v, idx, V);
		zero_quad<GT, NT>(a.g, idx);
		if (twin)
			store_quad<kBF16, NT>(a.twin, idx, P);
		if (fp8w)
			amax_l = amax4(amax_l, P);
		if (pk)
			pack_quad<NT>(a.der.pack, pd, (uint32_t)(idx - seg_begin), P);
	}
}

template <int GT, int MT, bool NT, bool DER>
__global__ __launch_bounds__(kThreads) void adam_update_pipe_kernel(UpdateArgs a)
{
	const int tid = threadIdx.x;
	const int64_t n_tiles = (a.n + kTile - 1) / kTile;
	const int64_t step = gridDim.x;
	double gs = a.grad_scale;
	bool skip = false;
	HalfStage<GT, MT> A, B;
	TileInfo ta, tn;
	int64_t tile = blockIdx.x;

	if (a.use_norm) {
		gs = a.state->grad_scale;
		skip = a.state->skipped != 0;
	}
	if (tile >= n_tiles)
		return;
	ta = tile_info<GT>(a, tile, skip);
	if (ta.vec)
		half_load<GT, MT, NT, 0>(A, a, ta.base, tid);
	for (;;) {
		const int64_t next = tile + step;
		const bool has = next < n_tiles;
		float amax_l = 0.0f;

		if (ta.vec) {
			half_load<GT, MT, NT, kQuadsPerTile / 2>(B, a, ta.base, tid);
			half_consume<GT, MT, NT, DER, 0>(A, a, ta, gs, tid, amax_l);
		}
		if (has) {
			tn = tile_info<GT>(a, next, skip);
			if (tn.vec)
				half_load<GT, MT, NT, 0>(A, a, tn.base, tid);
		}
		if (ta.vec) {
			half_consume<GT, MT, NT, DER, kQuadsPerTile / 2>(B, a, ta, gs, tid, amax_l);
			if (DER && a.der.wamax != nullptr && (ta.flags & kSegFp8Twin) != 0) {
				amax_l = wave_max(amax_l);
				if ((tid & 63) == 0)
					a.der.tile_amax[ta.tile * kWaves + (tid >> 6)] = amax_l;
			}
		} else {
			tile_slow<GT, MT, NT, DER>(a, ta, gs, skip, tid);
		}
		if (!has)
			break;
		tile = next;
		ta = tn;
	}
}

/* ---- derived outputs without an update, and the E4M3 twins ----------------------- */

struct DeriveArgs {
	const float	*p;
	int64_t		n;
	const Seg	*segs;
	const int32_t	*tile_seg;
	Derived		der;
	int		vec_ok;
	uint32_t	need;	/* tensors whose max |x| is wanted: those with this flag; 0 = every tensor */
};

/* Does a tensor with these flags take part, given the flag a pass asks for (0 = every tensor)? */
__device__ __forceinline__ bool wanted(uint32_t flags, uint32_t need)
{
	return need == 0u || (flags & need) != 0u;
}

template <bool NT>
__global__ __launch_bounds__(kThreads) void derive_kernel(DeriveArgs a)
{
	const int tid = threadIdx.x;
	const int64_t n_tiles = (a.n + kTile - 1) / kTile;

	for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
		const int64_t base = tile * kTile;
		const int64_t end = base + kTile < a.n ? base + kTile : a.n;
		const bool whole = a.vec_ok && end - base == kTile;
		f32x4 P[kQuadsPerTile] = {};

		/* a whole tile's loads go out before the launch table is asked whose tile it is */
		if (whole) {
#pragma unroll
			for (int u = 0; u < kQuadsPerTile; u++)
				P[u] = load_quad<kF32, NT>(a.p, base + (int64_t)(u * kThreads + tid) * kQuad, 1.0f);
		}
		int s = table(a.tile_seg)[tile];

		if (whole && table(a.segs)[s].end >= end) {
			const uint32_t flags = table(a.segs)[s].flags;
			const bool fp8w = wanted(flags, a.need) && a.der.wamax != nullptr;
			const bool pk = (flags & kSegPack) != 0 && a.der.pack != nullptr;
			float amax_l = 0.0f;

			if (!fp8w && !pk)
				continue;
			const PackDesc pd = pk ? a.der.packs[s] : PackDesc{0, 1u, 0u};
			const int64_t seg_begin = table(a.segs)[s].begin;

#pragma unroll
			for (int u = 0; u < kQuadsPerTile; u++) {
				const int64_t idx = base + (int64_t)(u * kThreads + tid) * kQuad;

				if (fp8w)
					amax_l = amax4(amax_l, P[u]);
				if (pk)
					pack_quad<NT>(a.der.pack, pd, (uint32_t)(idx - seg_begin), P[u]);
			}
			if (fp8w) {
				amax_l = wave_max(amax_l);
				if ((tid & 63) == 0)
					a.der.tile_amax[tile * kWaves + (tid >> 6)] = amax_l;
			}
		} else {
			for (int64_t i = base + tid; i < end; i += kThreads) {
				while (i >= a.segs[s].end)
					s++;
				const uint32_t flags = a.segs[s].flags;
				const float x = a.p[i];

				if (wanted(flags, a.need) && a.der.wamax != nullptr) {
					const float ab = fmaxf(0.0f, fabsf(x));

					if (ab > 0.0f)
						amax_raise(a.der.wamax + s, ab);
				}
				if ((flags & kSegPack) != 0 && a.der.pack != nullptr)
					pack_one(a.der.pack, a.der.packs[s], (uint32_t)(i - a.segs[s].begin), x);
			}
		}
	}
}

struct FoldArgs {
	int64_t		n;
	const Seg	*segs;
	const int32_t	*tile_seg;
	const float	*tile_amax;
	uint32_t	*wamax;
	const StepState	*state;
	uint32_t	need;
};

/*
** One lane per tile: the four wavefront maxima of a whole tile of a flagged tensor (the tiles
** the vector paths above wrote) go into the tensor's word.  Neighbouring tiles mostly belong
** to one tensor, so a wavefront whose 64 tiles all do raises the word once.
*/
__global__ __launch_bounds__(kThreads) void amax_fold_kernel(FoldArgs a)
{
	const int64_t n_tiles = (a.n + kTile - 1) / kTile;
	const int64_t tile = (int64_t)blockIdx.x * kThreads + threadIdx.x;
	int s = -1;
	float mx = 0.0f;

	if (a.state != nullptr && a.state->skipped != 0)
		return;
	if (tile < n_tiles) {
		const int t = a.tile_seg[tile];
		const int64_t base = tile * kTile;

		if (base + kTile <= a.n && a.segs[t].end >= base + kTile
		    && wanted(a.segs[t].flags, a.need)) {
			const f32x4 w = *(const f32x4 *)(a.tile_amax + tile * kWaves);

			s = t;
			mx = fmaxf(fmaxf(w.x, w.y), fmaxf(w.z, w.w));
		}
	}
	const int s0 = __shfl(s, 0, 64);

	if (__all(s == s0)) {
		if (s0 < 0)
			return;
		mx = wave_max(mx);
		if ((threadIdx.x & 63) == 0 && mx > 0.0f)
			amax_raise(a.wamax + s0, mx);
	} else if (s >= 0 && mx > 0.0f) {
		amax_raise(a.wamax + s, mx);
	}
}

struct Fp8TwinArgs {
	const float	*p;
	uint8_t		*q;
	int64_t		n;
	const Seg	*segs;
	const int32_t	*tile_seg;
	const uint32_t	*wamax;
	float		*wscale;
	int		n_tensors;
	const StepState	*state;
	int		vec_ok;
	uint32_t	need;
};

/*
** The quantisation pass of the E4M3 twins.  The scale of a tensor needs the max over ALL of
** its new values, which the update has just reduced into wamax, so this pass reads p once
** more (4 bytes) and writes 1 byte per element, where amax + quantise as separate passes
** over p would read it twice.
*/
template <bool NT>
__global__ __launch_bounds__(kThreads) void fp8_twin_kernel(Fp8TwinArgs a)
{
	const int tid = threadIdx.x;
	const int64_t n_tiles = (a.n + kTile - 1) / kTile;
	const bool skipped = a.state != nullptr && a.state->skipped != 0;

	if (blockIdx.x == 0) {
		for (int s = tid; s < a.n_tensors; s += kThreads) {
			if (!skipped && wanted(a.segs[s].flags, a.need))
				a.wscale[s] = scale_from_amax(__uint_as_float(a.wamax[s]));
		}
	}
	if (skipped)
		return;		/* p did not change: the twins and their scales stay */
	for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
		const int64_t base = tile * kTile;
		const int64_t end = base + kTile < a.n ? base + kTile : a.n;
		int s = a.tile_seg[tile];

		if (a.vec_ok && end - base == kTile && a.segs[s].end >= end) {
			if (!wanted(a.segs[s].flags, a.need))
				continue;
			const float inv = 1.0f / scale_from_amax(__uint_as_float(a.wamax[s]));
			f32x4 P[kQuadsPerTile];

#pragma unroll
			for (int u = 0; u < kQuadsPerTile; u++)
				P[u] = load_quad<kF32, NT>(a.p, base + (int64_t)(u * kThreads + tid) * kQuad, 1.0f);
#pragma unroll
			for (int u = 0; u < kQuadsPerTile; u++) {
				const uint32_t w = fp8_e4m3_encode4(P[u].x * inv, P[u].y * inv, P[u].z * inv,
				    P[u].w * inv);

				st<NT>((uint32_t *)(a.q + base + (int64_t)(u * kThreads + tid) * kQuad), w);
			}
		} else {
			for (int64_t i = base + tid; i < end; i += kThreads) {
				while (i >= a.segs[s].end)
					s++;
				if (wanted(a.segs[s].flags, a.need)) {
					const float inv = 1.0f / scale_from_amax(__uint_as_float(a.wamax[s]));

					a.q[i] = (uint8_t)fp8_e4m3_encode(a.p[i] * inv);
				}
			}
		}
	}
}

/* ---- helpers -------------------------------------------------------------- */

/* dst[i] = bf16(src[i]), round to nearest even (seed of the twins, gpu_cuda.cu:1497-1513). */
__global__ __launch_bounds__(kThreads) void f32_to_bf16_kernel(uint16_t *dst,
	const float *src, int64_t n, int vec_ok)
{
	const int64_t n4 = vec_ok ? n / kQuad : 0;
	const int64_t stride = (int64_t)gridDim.x * kThreads;

	for (int64_t q = (int64_t)blockIdx.x * kThreads + threadIdx.x; q < n4; q += stride) {
		const f32x4 x = *(const f32x4 *)(src + q * kQuad);

		store_quad<kBF16, false>(dst, q * kQuad, x);
	}
	for (int64_t i = n4 * kQuad + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
	    i += stride)
		dst[i] = (uint16_t)bf16_rne(src[i]);
}

/*
** Checkpoint layout of the moments: per slot one (m, v) float pair (lang/lm_serialize.c:263-296).
** A lane handles one slot: two scalar loads, one 8-byte store (or the reverse).
*/
template <int MT>
__global__ __launch_bounds__(kThreads) void mv_interleave_kernel(float *pairs, const void *m,
	const void *v, int64_t first, int64_t count)
{
	typedef float f32x2 __attribute__((ext_vector_type(2)));
	const int64_t stride = (int64_t)gridDim.x * kThreads;

	for (int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x; k < count; k += stride) {
		f32x2 mv;

		mv.x = load_one<MT>(m, first + k, 1.0f);
		mv.y = load_one<MT>(v, first + k, 1.0f);
		*(f32x2 *)(pairs + 2 * k) = mv;
	}
}

template <int MT>
__global__ __launch_bounds__(kThreads) void mv_deinterleave_kernel(void *m, void *v,
	const float *pairs, int64_t first, int64_t count)
{
	typedef float f32x2 __attribute__((ext_vector_type(2)));
	const int64_t stride = (int64_t)gridDim.x * kThreads;

	for (int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x; k < count; k += stride) {
		const f32x2 mv = *(const f32x2 *)(pairs + 2 * k);

		store_one<MT>(m, first + k, mv.x);
		store_one<MT>(v, first + k, mv.y);
	}
}

/* Byte fill on the stream (a kernel, so it can sit in a captured graph). */
__global__ __launch_bounds__(kThreads) void fill_bytes_kernel(uint8_t *dst, uint32_t pattern,
	size_t nbytes, size_t head, size_t n16)
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	const size_t stride = (size_t)gridDim.x * kThreads;
	const size_t gid = (size_t)blockIdx.x * kThreads + threadIdx.x;
	const u32x4 w = {pattern, pattern, pattern, pattern};

	/* [0, head) bytes up to 16-byte alignment, n16 aligned 16-byte words, then the rest. */
	for (size_t i = gid; i < head; i += stride)
		dst[i] = (uint8_t)pattern;
	/*
	** Word i goes to lane i mod (all lanes of the grid): with ONE workgroup per compute unit the
	** chip then writes one contiguous MiB at a time, every workgroup always the same 4 KiB of it --
	** measured 6.4 - 6.5 TB/s, what the runtime's own fill reaches, against 5.8 - 6.0 for any grid
	** of more workgroups (512: 5.3, 2048: 4.9) and for one contiguous slice or tile per workgroup.
	*/
	for (size_t i = gid; i < n16; i += stride)
		*(u32x4 *)(dst + head + i * 16) = w;
	for (size_t i = head + n16 * 16 + gid; i < nbytes; i += stride)
		dst[i] = (uint8_t)pattern;
}

/* ---- host side ------------------------------------------------------------ */

static int env_int(const char *name, int dflt, int lo, int hi)
{
	const char *e = getenv(name);
	int v;

	if (!e || !*e)
		return dflt;
	v = atoi(e);
	if (v < lo)
		v = lo;
	if (v > hi)
		v = hi;
	return v;
}

/*
** The tuning switches, read from the environment on first use and again whenever
** reload_switches() is called (a sweep that compares settings on one arena in one process: two
** processes differ by what memory they were given, by more than most settings do).
*/
struct Switches {
	int	loaded;
	int	blocks_per_cu;	/* ANNI_BLOCKS_PER_CU: workgroups per compute unit of a grid that is resident as a whole */
	int	nt;		/* ANNI_NT=0: no streaming (non-temporal) cache hints */
	int	reverse;	/* ANNI_REVERSE=0: the update walks the tiles from the first to the last */
	int	keep_mb;	/* ANNI_KEEP_MB: how much of the gradients' tail the sum of squares leaves in the memory-side cache */
	int	pipe;		/* ANNI_PIPE=0: narrow storage modes on the plain kernel; 2: the all-f32 mode pipelined too */
	int	tiles_per_wg;	/* ANNI_TILES_PER_WG: tiles per workgroup of the update; 0 = the resident grid; -1 = the default */
	int	sumsq_per_cu;	/* ANNI_SUMSQ_PER_CU: workgroups per compute unit of the sum of squares; 0 = the default */
	int	fold_fence;	/* ANNI_FOLD=fence: the norm's second stage takes the partials over with fences (see sumsq_finish) */
};
static Switches g_sw;
static void fold_guard_reset(void);

void reload_switches(void)
{
	g_sw.blocks_per_cu = env_int("ANNI_BLOCKS_PER_CU", 8, 1, 32);
	g_sw.nt = env_int("ANNI_NT", 1, 0, 1);
	g_sw.reverse = env_int("ANNI_REVERSE", 1, 0, 1);
	g_sw.keep_mb = env_int("ANNI_KEEP_MB", 256, 0, 1 << 20);
	g_sw.pipe = env_int("ANNI_PIPE", 1, 0, 2);
	g_sw.tiles_per_wg = env_int("ANNI_TILES_PER_WG", -1, -1, 1 << 20);
	g_sw.sumsq_per_cu = env_int("ANNI_SUMSQ_PER_CU", 0, 0, 32);
	{
		const char *e = getenv("ANNI_FOLD");

		g_sw.fold_fence = (e && strcmp(e, "fence") == 0) ? 1 : 0;
	}
	g_sw.loaded = 1;
	fold_guard_reset();
}

static const Switches &sw(void)
{
	if (!g_sw.loaded)
		reload_switches();
	return g_sw;
}

static int cu_count(void)
{
	static int cus;

	if (!cus) {
		int dev = 0;
		int n = 0;

		if (hipGetDevice(&dev) != hipSuccess
		    || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev)
		    != hipSuccess || n <= 0)
			n = 256;
		cus = n;
	}
	return cus;
}

/* A grid that is resident as a whole: ANNI_BLOCKS_PER_CU workgroups per compute unit (default 8). */
int grid_for(int64_t n)
{
	int64_t tiles = (n + kTile - 1) / kTile;
	int64_t g;

	g = (int64_t)cu_count() * sw().blocks_per_cu;
	if (g > kMaxPartials)
		g = kMaxPartials;
	if (g > tiles)
		g = tiles;
	if (g < 1)
		g = 1;
	return (int)g;
}

static bool nt_on(void)
{
	return sw().nt != 0;
}

static bool reverse_on(void)
{
	return sw().reverse != 0;
}

static int keep_mb(void)
{
	return sw().keep_mb;
}

static bool aligned(const void *p, uintptr_t a)
{
	return ((uintptr_t)p & (a - 1)) == 0;
}

static uintptr_t quad_bytes(int type)
{
	return type == kF32 ? 16 : type == kBF16 ? 8 : 4;
}

static int check_flat(const Flat &f, bool need_state)
{
	if (!f.g || f.n <= 0)
		return -1;
	if (f.grad_type < kF32 || f.grad_type > kFP8)
		return -1;
	if (f.grad_type == kFP8 && !f.gscale)
		return -1;
	if ((f.segs == nullptr) != (f.tile_seg == nullptr))
		return -1;
	if (need_state) {
		if (!f.p || !f.m || !f.v)
			return -1;
		if (f.moment_type != kF32 && f.moment_type != kBF16)
			return -1;
	}
	return 0;
}

/* fence: 1 = the second stage takes the partials over with fences, 0 = with atomic accesses. */
static int sumsq_launch(hipStream_t st, const Flat &f, double grad_scale, double *partials,
	int *n_partials, const SumsqFinish *fin, int fence)
{
	SumsqArgs a;
	int grid;

	if (check_flat(f, false) != 0 || !partials || !n_partials)
		return -1;
	const int64_t chunk_elems = f.grad_type == kF32 ? SumsqChunk<kF32>::kElems
	    : f.grad_type == kBF16 ? SumsqChunk<kBF16>::kElems : SumsqChunk<kFP8>::kElems;
	const int64_t n_chunks = (f.n + chunk_elems - 1) / chunk_elems;

	{
		/*
		** Workgroups of the sum, resident as a whole.  Float gradients: two per compute unit
		** (0.327 against 0.337 ms for eight at 555M, measured inside one process; one is too few,
		** 0.444).  bf16 and E4M3 gradients do more arithmetic per byte and want the usual eight
		** (two: +25 - 35 %).
		*/
		const int per_cu = sw().sumsq_per_cu ? sw().sumsq_per_cu
		    : f.grad_type == kF32 ? 2 : sw().blocks_per_cu;
		int64_t g = (int64_t)cu_count() * per_cu;

		if (g > kMaxPartials)
			g = kMaxPartials;
		if (g > n_chunks)
			g = n_chunks;
		grid = g < 1 ? 1 : (int)g;
	}
	a.g = f.g;
	a.n = f.n;
	a.segs = f.segs;
	a.tile_seg = f.tile_seg;
	a.gscale = f.gscale;
	a.grad_scale = grad_scale;
	a.partials = partials;
	a.ticket = nullptr;
	a.clip = 0.0;
	a.skip_nonfinite = 0;
	a.state = nullptr;
	a.fence = fence;
	if (fin) {
		if (!fin->ticket || !fin->state || !aligned(fin->ticket, 128))
			return -1;
		a.ticket = fin->ticket;
		a.clip = fin->clip;
		a.skip_nonfinite = fin->skip_nonfinite;
		a.state = fin->state;
	}
	a.vec_ok = aligned(f.g, 16) ? 1 : 0;
	{
		/*
		** The update that follows reads the gradients again.  What the sum reads last with
		** ordinary loads stays in the memory-side cache (256 MiB on this part; streaming
		** accesses pass it by), and the update, walking the flat from its end, finds it there.
		*/
		const int64_t keep = (int64_t)keep_mb() * (1 << 20) / SumsqChunk<kF32>::kBytes;

		a.keep_from = n_chunks > keep ? n_chunks - keep : 0;
	}
#define SUMSQ_LAUNCH(GT) \
	do { \
		if (nt_on()) \
			hipLaunchKernelGGL((sumsq_kernel<GT, true>), dim3(grid), dim3(kThreads), 0, st, a); \
		else \
			hipLaunchKernelGGL((sumsq_kernel<GT, false>), dim3(grid), dim3(kThreads), 0, st, a); \
	} while (0)
	if (f.grad_type == kF32)
		SUMSQ_LAUNCH(kF32);
	else if (f.grad_type == kBF16)
		SUMSQ_LAUNCH(kBF16);
	else
		SUMSQ_LAUNCH(kFP8);
#undef SUMSQ_LAUNCH
	*n_partials = grid;
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

/*
** Self-check of the second stage.  The default hand-over of the partials (atomic accesses, see
** sumsq_finish) leans on how gfx950 performs device-scope atomics, which the HIP memory model
** does not promise; the fenced form leans on nothing.  So the first sum of squares with a second
** stage on each device -- and the first after the switches were read again -- runs both forms on
** the caller's own gradient flat and grid before anything consumes a result, waits, and compares
** the two step states bit for bit.  If they differ the process goes over to the fenced form for
** good and says so once on stderr.  Cost: two extra launches and one stream synchronisation per
** process and device.  A stream under capture cannot be waited for: there the check is put off
** until the first launch outside a capture.
*/
static const int kGuardDevices = 64;
static std::atomic<int> g_fold_checked[kGuardDevices];
static std::atomic<int> g_finish_checked[kGuardDevices];	/* chunk_finish_kernel: 0 not checked yet, 1 good, 2 use the separate kernels */
static std::mutex g_fold_mu;
static StepState *g_fold_host;		/* page-locked, two states */
static int g_fold_runs;
static int g_fold_mismatches;

static void fold_guard_reset(void)
{
	for (int i = 0; i < kGuardDevices; i++) {
		g_fold_checked[i].store(0, std::memory_order_relaxed);
		g_finish_checked[i].store(0, std::memory_order_relaxed);
	}
}

void fold_guard_stats(int *runs, int *mismatches)
{
	std::lock_guard<std::mutex> lk(g_fold_mu);

	if (runs)
		*runs = g_fold_runs;
	if (mismatches)
		*mismatches = g_fold_mismatches;
}

static void fold_guard(hipStream_t st, const Flat &f, double grad_scale, double *partials,
	const SumsqFinish *fin)
{
	hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
	SumsqFinish mine;
	int dev = -1;
	int np = 0;

	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kGuardDevices) {
		(void)hipGetLastError();
		return;
	}
	if (g_fold_checked[dev].load(std::memory_order_acquire))
		return;
	if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
		(void)hipGetLastError();
		return;
	}
	std::lock_guard<std::mutex> lk(g_fold_mu);

	if (g_fold_checked[dev].load(std::memory_order_relaxed))
		return;
	if (!g_fold_host && hipHostMalloc((void **)&g_fold_host, 2 * sizeof(StepState),
	    hipHostMallocPortable) != hipSuccess) {
		(void)hipGetLastError();
		g_fold_host = nullptr;
		return;
	}
	memset(g_fold_host, 0xff, 2 * sizeof(StepState));
	mine = *fin;
	for (int fence = 0; fence < 2; fence++) {
		mine.state = g_fold_host + fence;
		if (sumsq_launch(st, f, grad_scale, partials, &np, &mine, fence) != 0)
			return;
	}
	if (hipStreamSynchronize(st) != hipSuccess) {
		(void)hipGetLastError();
		return;
	}
	g_fold_runs++;
	if (memcmp(&g_fold_host[0], &g_fold_host[1], sizeof(StepState)) != 0) {
		g_fold_mismatches++;
		g_sw.fold_fence = 1;
		fprintf(stderr, "[anni] sum of squares: the atomic and the fenced hand-over of the partials "
		    "disagree on this device (sum %.17g against %.17g over %d workgroups); "
		    "using the fenced one from now on\n", g_fold_host[0].sumsq, g_fold_host[1].sumsq, np);
	}
	g_fold_checked[dev].store(1, std::memory_order_release);
}

int launch_sumsq(hipStream_t st, const Flat &f, double grad_scale, double *partials,
	int *n_partials, const SumsqFinish *fin)
{
	if (fin && fin->ticket && fin->state && !sw().fold_fence && check_flat(f, false) == 0
	    && partials)
		fold_guard(st, f, grad_scale, partials, fin);
	return sumsq_launch(st, f, grad_scale, partials, n_partials, fin, sw().fold_fence);
}

static_assert(SumsqChunk<kF32>::kBytes == (int64_t)kSumChunkBytes, "callers note rewritten chunks in these units");

int chunk_sums_count(int64_t n)
{
	const int64_t c = (n + SumsqChunk<kF32>::kElems - 1) / SumsqChunk<kF32>::kElems;

	return (int)c;
}

int launch_chunk_sums(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *list,
	int n_list, int beside)
{
	ChunkSumArgs a;
	const int64_t n_chunks = chunk_sums_count(n);
	int64_t grid;

	if (!x || n <= 0 || !part || (list && n_list <= 0))
		return -1;
	a.x = x;
	a.n = n;
	a.part = part;
	a.list = list;
	a.n_list = list ? n_list : 0;
	a.vec_ok = aligned(x, 16) ? 1 : 0;
	{
		const int64_t keep = (int64_t)keep_mb() * (1 << 20) / SumsqChunk<kF32>::kBytes;

		a.keep_from = n_chunks > keep ? n_chunks - keep : 0;
	}
	if (list) {
		grid = ((int64_t)n_list + kWaves - 1) / kWaves;		/* one wavefront per listed chunk */
	} else {
		/*
		** Workgroups per compute unit, resident as a whole.  Alone on the device eight are best
		** (0.332 ms per call at 555M against 0.351 for two, 0.335 - 0.337 for 12 and 16); a sum that
		** runs beside the caller's copy pieces leaves them room: with eight the unchanged caller's
		** 555M step was 0.04 ms slower than with two.
		*/
		grid = (int64_t)cu_count() * (sw().sumsq_per_cu ? sw().sumsq_per_cu : beside ? 2 : 8);
		if (grid > (n_chunks + kWaves - 1) / kWaves)
			grid = (n_chunks + kWaves - 1) / kWaves;
	}
	if (grid < 1)
		grid = 1;
	if (nt_on())
		hipLaunchKernelGGL((chunk_sums_kernel<true>), dim3((unsigned)grid), dim3(kThreads), 0, st, a);
	else
		hipLaunchKernelGGL((chunk_sums_kernel<false>), dim3((unsigned)grid), dim3(kThreads), 0, st, a);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_chunk_fold(hipStream_t st, const double *part, int64_t n, double *runs, StepState *state)
{
	const int64_t count = (int64_t)chunk_sums_count(n);
	int64_t per = kChunkPer;
	int64_t n_runs;

	if (!part || !runs || !state || n <= 0)
		return -1;
	while ((count + per - 1) / per > kChunkRuns)
		per *= 2;
	n_runs = (count + per - 1) / per;
	hipLaunchKernelGGL(chunk_fold_kernel, dim3((unsigned)n_runs), dim3(kThreads), 0, st, part, count, per, runs);
	hipLaunchKernelGGL(chunk_final_kernel, dim3(1), dim3(kThreads), 0, st, (const double *)runs, (int)n_runs,
	    state);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

/*
** Self-check of chunk_finish_kernel, as for the sum of squares' second stage (fold_guard): the
** first call on each device, and the first after the switches were read again, runs the merged
** kernel and the three separate ones (which hand nothing over inside a launch) on the caller's
** own flat, waits, and compares the two states bit for bit.  If they differ the process stays
** with the separate kernels and says so once on stderr.
*/

static int chunk_finish_launch(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *fix,
	int n_fix, double *runs, unsigned int *ticket, StepState *state, unsigned long long *stamp,
	unsigned long long token)
{
	ChunkFinishArgs a;
	const int64_t n_chunks = chunk_sums_count(n);
	const int64_t keep = (int64_t)keep_mb() * (1 << 20) / SumsqChunk<kF32>::kBytes;
	int64_t per = kChunkPer;

	a.count = n_chunks;
	while ((a.count + per - 1) / per > kChunkRuns)
		per *= 2;
	a.per = per;
	a.sum.x = x;
	a.sum.n = n;
	a.sum.part = part;
	a.sum.list = nullptr;
	a.sum.n_list = 0;
	a.sum.vec_ok = aligned(x, 16) ? 1 : 0;
	a.sum.keep_from = n_chunks > keep ? n_chunks - keep : 0;
	memset(&a.fin, 0, sizeof(a.fin));
	a.fin.partials = runs;
	a.fin.ticket = ticket;
	a.fin.grad_scale = 1.0;
	a.fin.state = state;
	a.fin.fence = sw().fold_fence;
	a.stamp = stamp;
	a.token = token;
	a.n_fix = n_fix;
	if (n_fix > 0)
		memcpy(a.fix, fix, (size_t)n_fix * sizeof(int32_t));
	const unsigned grid = (unsigned)((a.count + per - 1) / per);

	if (nt_on())
		hipLaunchKernelGGL((chunk_finish_kernel<true>), dim3(grid), dim3(kThreads), 0, st, a);
	else
		hipLaunchKernelGGL((chunk_finish_kernel<false>), dim3(grid), dim3(kThreads), 0, st, a);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

static int chunk_finish_apart(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *fix_dev,
	int n_fix, double *runs, StepState *state)
{
	if (n_fix > 0 && launch_chunk_sums(st, x, n, part, fix_dev, n_fix, 0) != 0)
		return -1;
	return launch_chunk_fold(st, part, n, runs, state);
}

int launch_chunk_finish(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *fix,
	const int32_t *fix_dev, int n_fix, double *runs, unsigned int *ticket, StepState *state,
	unsigned long long *stamp, unsigned long long token)
{
	int dev = -1;
	int how;

	if (!x || n <= 0 || !part || !runs || !state || n_fix < 0 || (n_fix > 0 && (!fix || !fix_dev)))
		return -1;
	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kGuardDevices) {
		(void)hipGetLastError();
		dev = -1;
	}
	how = (dev < 0 || !ticket || !aligned(ticket, 128) || n_fix > kFixMax) ? 2
	    : g_finish_checked[dev].load(std::memory_order_acquire);
	if (how == 0) {
		hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
		std::lock_guard<std::mutex> lk(g_fold_mu);

		if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone
		    || (!g_fold_host && hipHostMalloc((void **)&g_fold_host, 2 * sizeof(StepState),
		    hipHostMallocPortable) != hipSuccess)) {
			(void)hipGetLastError();
			how = 2;	/* this call only: the check is put off */
		} else {
			memset(g_fold_host, 0xff, 2 * sizeof(StepState));
			if (chunk_finish_launch(st, x, n, part, fix, n_fix, runs, ticket, g_fold_host, nullptr, 0) != 0
			    || chunk_finish_apart(st, x, n, part, fix_dev, n_fix, runs, g_fold_host + 1) != 0
			    || hipStreamSynchronize(st) != hipSuccess) {
				(void)hipGetLastError();
				return -1;
			}
			g_fold_runs++;
			how = 1;
			if (memcmp(&g_fold_host[0], &g_fold_host[1], sizeof(StepState)) != 0) {
				g_fold_mismatches++;
				how = 2;
				fprintf(stderr, "[anni] sum of squares of a flat: the merged last stage and the separate "
				    "kernels disagree on this device (sum %.17g against %.17g); using the separate "
				    "kernels from now on\n", g_fold_host[0].sumsq, g_fold_host[1].sumsq);
			}
			g_finish_checked[dev].store(how, std::memory_order_release);
		}
	}
	if (how == 1)
		return chunk_finish_launch(st, x, n, part, fix, n_fix, runs, ticket, state, stamp, token);
	return chunk_finish_apart(st, x, n, part, fix_dev, n_fix, runs, state) == 0 ? 1 : -1;
}

#ifndef ANNI_UPDATE_UNROLL
#define ANNI_UPDATE_UNROLL 4		/* all-f32 mode: the whole tile in flight */
#endif
#ifndef ANNI_UPDATE_UNROLL_NARROW
#define ANNI_UPDATE_UNROLL_NARROW 4	/* bf16 moments / bf16 or fp8 gradients */
#endif

static int pipe_level(void)
{
	return sw().pipe;
}

template <int GT, int MT>
static void update_launch(hipStream_t st, int grid, const UpdateArgs &a)
{
	constexpr int U = (GT == kF32 && MT == kF32) ? ANNI_UPDATE_UNROLL : ANNI_UPDATE_UNROLL_NARROW;
	constexpr bool narrow = GT != kF32 || MT != kF32;
	const bool der = a.der.wamax != nullptr || a.der.pack != nullptr;

	if (pipe_level() >= (narrow ? 1 : 2)) {
		if (der) {
			if (nt_on())
				hipLaunchKernelGGL((adam_update_pipe_kernel<GT, MT, true, true>), dim3(grid),
				    dim3(kThreads), 0, st, a);
			else
				hipLaunchKernelGGL((adam_update_pipe_kernel<GT, MT, false, true>), dim3(grid),
				    dim3(kThreads), 0, st, a);
		} else if (nt_on()) {
			hipLaunchKernelGGL((adam_update_pipe_kernel<GT, MT, true, false>), dim3(grid),
			    dim3(kThreads), 0, st, a);
		} else {
			hipLaunchKernelGGL((adam_update_pipe_kernel<GT, MT, false, false>), dim3(grid),
			    dim3(kThreads), 0, st, a);
		}
		return;
	}
	if (der) {
		if (nt_on())
			hipLaunchKernelGGL((adam_update_kernel<GT, MT, U, true, true>), dim3(grid),
			    dim3(kThreads), 0, st, a);
		else
			hipLaunchKernelGGL((adam_update_kernel<GT, MT, U, false, true>), dim3(grid),
			    dim3(kThreads), 0, st, a);
	} else if (nt_on()) {
		hipLaunchKernelGGL((adam_update_kernel<GT, MT, U, true, false>), dim3(grid),
		    dim3(kThreads), 0, st, a);
	} else {
		hipLaunchKernelGGL((adam_update_kernel<GT, MT, U, false, false>), dim3(grid),
		    dim3(kThreads), 0, st, a);
	}
}

/*
** Workgroups of the update.  Compute units do not stream at one speed (where their data lie,
** what shares their part of the chip), so a grid in which every workgroup owns an equal share of
** the flat ends as fast as its slowest member.  With many more workgroups than fit the chip at
** once the dispatcher hands the next one to whichever compute unit falls free: -4 to -6 % against
** eight resident workgroups per compute unit.  Measured best in every storage mode, for the kernels
** with derived outputs and for the E4M3 pass: one tile per workgroup.  ANNI_TILES_PER_WG sets
** another number for all of them; 0 = the resident grid.
*/
static int balanced_grid(int64_t n, int tiles_per_wg)
{
	const int64_t tiles = (n + kTile - 1) / kTile;
	const int per = sw().tiles_per_wg;
	int grid = grid_for(n);
	int k;

	k = per >= 0 ? per : tiles_per_wg;
	if (k > 0 && tiles / k > grid) {
		const int64_t cap = (int64_t)1 << 22;	/* 2^30 lanes: within every launch limit; more tiles than that take turns */

		grid = (int)(tiles / k < cap ? tiles / k : cap);
	}
	return grid;
}

/* Derived outputs need the launch table, an 8-byte aligned pack flat and descriptors for it. */
static int check_derived(const Flat &f)
{
	if (!f.der.wamax && !f.der.pack)
		return 0;
	if (!f.segs || !f.tile_seg)
		return -1;
	if (f.der.wamax && !aligned(f.der.tile_amax, 16))
		return -1;
	if (f.der.pack && (!f.der.packs || !aligned(f.der.pack, 8)))
		return -1;
	return 0;
}

static int update_go(hipStream_t st, const Flat &f, const StepConsts &c, double grad_scale,
	const NormIn &norm, const int32_t *order, int64_t turns)
{
	UpdateArgs a;
	int grid;

	if (check_flat(f, true) != 0 || check_derived(f) != 0)
		return -1;
	if (norm.use_norm && !norm.state)
		return -1;
	grid = balanced_grid(f.n, 1);
	if (order) {
		const bool narrow = f.grad_type != kF32 || f.moment_type != kF32;

		/* the software-pipelined kernels walk the flat their own way */
		if (turns < 1 || turns > (f.n + kTile - 1) / kTile || pipe_level() >= (narrow ? 1 : 2))
			return -1;
		grid = balanced_grid(turns * kTile, 1);
	}
	a.order = order;
	a.turns = order ? turns : 0;
	a.p = f.p;
	a.g = f.g;
	a.m = f.m;
	a.v = f.v;
	a.twin = f.twin;
	a.n = f.n;
	a.segs = f.segs;
	a.tile_seg = f.tile_seg;
	a.gscale = f.gscale;
	a.uniform_flags = f.uniform_flags;
	a.vec_ok = aligned(f.p, 16) && aligned(f.g, quad_bytes(f.grad_type))
	    && aligned(f.m, quad_bytes(f.moment_type)) && aligned(f.v, quad_bytes(f.moment_type))
	    && (!f.twin || aligned(f.twin, 8)) ? 1 : 0;
	if (f.der.wamax && !a.vec_ok)
		return -1;	/* the tile maxima come from the vector path: the flats must be aligned */
	a.c = c;
	a.grad_scale = grad_scale;
	a.use_norm = norm.use_norm;
	a.state = norm.state;
	a.der = f.der;
	a.reverse = reverse_on() ? 1 : 0;
	if (f.moment_type == kF32) {
		if (f.grad_type == kF32)
			update_launch<kF32, kF32>(st, grid, a);
		else if (f.grad_type == kBF16)
			update_launch<kBF16, kF32>(st, grid, a);
		else
			update_launch<kFP8, kF32>(st, grid, a);
	} else {
		if (f.grad_type == kF32)
			update_launch<kF32, kBF16>(st, grid, a);
		else if (f.grad_type == kBF16)
			update_launch<kBF16, kBF16>(st, grid, a);
		else
			update_launch<kFP8, kBF16>(st, grid, a);
	}
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_update(hipStream_t st, const Flat &f, const StepConsts &c, double grad_scale,
	const NormIn &norm)
{
	return update_go(st, f, c, grad_scale, norm, nullptr, 0);
}

int update_walks_backwards(void)
{
	return reverse_on() ? 1 : 0;
}

int launch_update_tiles(hipStream_t st, const Flat &f, const StepConsts &c, double grad_scale,
	const NormIn &norm, const int32_t *order, int64_t turns)
{
	if (!order)
		return -1;
	return update_go(st, f, c, grad_scale, norm, order, turns);
}

static int helper_grid(int64_t work_items)
{
	int64_t g = (work_items + kThreads - 1) / kThreads;
	int64_t cap = (int64_t)cu_count() * 8;

	if (g > cap)
		g = cap;
	if (g < 1)
		g = 1;
	return (int)g;
}

int launch_f32_to_bf16(hipStream_t st, uint16_t *dst, const float *src, int64_t n)
{
	if (!dst || !src || n <= 0)
		return -1;
	hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(helper_grid(n / kQuad + 1)), dim3(kThreads),
	    0, st, dst, src, n, aligned(src, 16) && aligned(dst, 8) ? 1 : 0);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_derive(hipStream_t st, const Flat &f, uint32_t need)
{
	DeriveArgs a;

	if (!f.p || f.n <= 0 || check_derived(f) != 0 || (!f.der.wamax && !f.der.pack))
		return -1;
	a.p = f.p;
	a.n = f.n;
	a.segs = f.segs;
	a.tile_seg = f.tile_seg;
	a.der = f.der;
	a.need = need;
	a.vec_ok = aligned(f.p, 16) ? 1 : 0;
	if (f.der.wamax && !a.vec_ok)
		return -1;
	if (nt_on())
		hipLaunchKernelGGL((derive_kernel<true>), dim3(grid_for(f.n)), dim3(kThreads), 0, st, a);
	else
		hipLaunchKernelGGL((derive_kernel<false>), dim3(grid_for(f.n)), dim3(kThreads), 0, st, a);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_amax_fold(hipStream_t st, const Flat &f, const StepState *state, uint32_t need)
{
	FoldArgs a;
	const int64_t n_tiles = (f.n + kTile - 1) / kTile;

	static_assert(kWaves == 4, "one 16-byte load per tile");
	if (f.n <= 0 || !f.der.wamax || check_derived(f) != 0)
		return -1;
	a.n = f.n;
	a.segs = f.segs;
	a.tile_seg = f.tile_seg;
	a.tile_amax = f.der.tile_amax;
	a.wamax = f.der.wamax;
	a.state = state;
	a.need = need;
	hipLaunchKernelGGL(amax_fold_kernel, dim3((unsigned)((n_tiles + kThreads - 1) / kThreads)),
	    dim3(kThreads), 0, st, a);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_fp8_twins(hipStream_t st, const Flat &f, uint8_t *q, float *wscale,
	const uint32_t *wamax, int n_tensors, const StepState *state, uint32_t need)
{
	Fp8TwinArgs a;

	if (!f.p || f.n <= 0 || !f.segs || !f.tile_seg || !q || !wscale || !wamax
	    || n_tensors <= 0)
		return -1;
	a.p = f.p;
	a.q = q;
	a.n = f.n;
	a.segs = f.segs;
	a.tile_seg = f.tile_seg;
	a.wamax = wamax;
	a.wscale = wscale;
	a.n_tensors = n_tensors;
	a.state = state;
	a.need = need;
	a.vec_ok = aligned(f.p, 16) && aligned(q, 4) ? 1 : 0;
	if (nt_on())
		hipLaunchKernelGGL((fp8_twin_kernel<true>), dim3(balanced_grid(f.n, 1)), dim3(kThreads), 0, st, a);
	else
		hipLaunchKernelGGL((fp8_twin_kernel<false>), dim3(balanced_grid(f.n, 1)), dim3(kThreads), 0, st, a);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_mv_interleave(hipStream_t st, float *pairs, const void *m, const void *v,
	int moment_type, int64_t first, int64_t count)
{
	if (!pairs || !m || !v || first < 0 || count <= 0 || !aligned(pairs, 8))
		return -1;
	if (moment_type == kF32)
		hipLaunchKernelGGL((mv_interleave_kernel<kF32>), dim3(helper_grid(count)), dim3(kThreads),
		    0, st, pairs, m, v, first, count);
	else if (moment_type == kBF16)
		hipLaunchKernelGGL((mv_interleave_kernel<kBF16>), dim3(helper_grid(count)),
		    dim3(kThreads), 0, st, pairs, m, v, first, count);
	else
		return -1;
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_mv_deinterleave(hipStream_t st, void *m, void *v, int moment_type, const float *pairs,
	int64_t first, int64_t count)
{
	if (!pairs || !m || !v || first < 0 || count <= 0 || !aligned(pairs, 8))
		return -1;
	if (moment_type == kF32)
		hipLaunchKernelGGL((mv_deinterleave_kernel<kF32>), dim3(helper_grid(count)),
		    dim3(kThreads), 0, st, m, v, pairs, first, count);
	else if (moment_type == kBF16)
		hipLaunchKernelGGL((mv_deinterleave_kernel<kBF16>), dim3(helper_grid(count)),
		    dim3(kThreads), 0, st, m, v, pairs, first, count);
	else
		return -1;
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_fill_bytes(hipStream_t st, void *dst, int value, size_t nbytes)
{
	const uint32_t b = (uint32_t)(value & 0xff);
	const uint32_t pattern = b | (b << 8) | (b << 16) | (b << 24);
	size_t head;
	size_t n16;

	if (!dst || nbytes == 0)
		return -1;
	head = (16 - ((uintptr_t)dst & 15)) & 15;
	if (head > nbytes)
		head = nbytes;
	n16 = (nbytes - head) / 16;
	{
		/* large fills: one workgroup per compute unit (see the kernel) */
		int grid = helper_grid((int64_t)n16 + 16);

		if (grid > cu_count())
			grid = cu_count();
		hipLaunchKernelGGL(fill_bytes_kernel, dim3(grid), dim3(kThreads), 0, st, (uint8_t *)dst,
		    pattern, nbytes, head, n16);
	}
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

} /* namespace anni */

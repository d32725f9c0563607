/*
** libanni_bench.so -- what measures and tests libanni_gpu_hip.so (include/anni_bench.h): step
** loops timed with HIP events, synthetic input generators, a calibration copy kernel, re-reading
** of the tuning switches.  Linked against the product library and kept out of it, so that the
** product carries nothing a training program does not call.  None of this has a counterpart in
** the reference.
*/
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <vector>
#include "anni_adam.h"
#include "anni_bench.h"
#include "anni_gpu.h"
#include "anni_hooks.h"

namespace anni_bench {

constexpr int kLanes = 256;

/* splitmix64 finaliser: a bijective 64-bit mix, used as a counter-based generator. */
__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
	z += 0x9e3779b97f4a7c15ull;
	z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
	z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
	return z ^ (z >> 31);
}

/* Element pair k of (seed, stream) -> two standard normals (Box-Muller). */
__global__ __launch_bounds__(kLanes) void fill_normal_kernel(float *x, int64_t n, uint64_t seed,
	uint64_t stream, float mean, float std)
{
	const int64_t pairs = (n + 1) / 2;
	const int64_t stride = (int64_t)gridDim.x * kLanes;
	const uint64_t key = mix64(seed ^ mix64(stream));

	for (int64_t k = (int64_t)blockIdx.x * kLanes + threadIdx.x; k < pairs; k += stride) {
		const uint64_t r = mix64(key + (uint64_t)k * 0xd1342543de82ef95ull);
		/* u1 in (0,1], u2 in [0,1): 24 bits each */
		const float u1 = ((float)(uint32_t)(r >> 40) + 1.0f) * (1.0f / 16777216.0f);
		const float u2 = (float)(uint32_t)((r >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
		const float rad = sqrtf(-2.0f * logf(u1));
		float sn, cs;

		sincospif(2.0f * u2, &sn, &cs);
		x[2 * k] = mean + std * (rad * cs);
		if (2 * k + 1 < n)
			x[2 * k + 1] = mean + std * (rad * sn);
	}
}

/* dst[i] = src[i] over n16 16-byte words: a plain copy of known size (counter calibration). */
__global__ __launch_bounds__(kLanes) void copy16_kernel(void *dst, const void *src, size_t n16)
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	const size_t stride = (size_t)gridDim.x * kLanes;

	for (size_t i = (size_t)blockIdx.x * kLanes + threadIdx.x; i < n16; i += stride)
		((u32x4 *)dst)[i] = ((const u32x4 *)src)[i];
}

/*
** The same copy in the update kernel's shape: one workgroup per 16 KiB, four 16-byte words per
** lane in flight, the dispatcher handing the next piece to whichever compute unit falls free;
** NT selects non-temporal loads and stores.  n16 is a multiple of 1024 here; the tail goes to
** copy16_kernel.
*/
template <bool NT>
__global__ __launch_bounds__(kLanes) void copy_tiled_kernel(void *dst, const void *src)
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	const u32x4 *s = (const u32x4 *)src + (size_t)blockIdx.x * 1024 + threadIdx.x;
	u32x4 *d = (u32x4 *)dst + (size_t)blockIdx.x * 1024 + threadIdx.x;
	u32x4 w[4];

	static_assert(kLanes == 256, "a piece is four words per lane");
#pragma unroll
	for (int u = 0; u < 4; u++)
		w[u] = NT ? __builtin_nontemporal_load(s + u * 256) : s[u * 256];
#pragma unroll
	for (int u = 0; u < 4; u++) {
		if (NT)
			__builtin_nontemporal_store(w[u], d + u * 256);
		else
			d[u * 256] = w[u];
	}
}

static int util_grid(int64_t items)
{
	int64_t g = (items + kLanes - 1) / kLanes;

	if (g > 2048)
		g = 2048;
	if (g < 1)
		g = 1;
	return (int)g;
}

static float g_last_derived_ms;	/* E4M3 pass time of the last per-kernel run of anni_adam_time_steps */

static int time_steps_body(anni_adam *opt, int count, void *const *grads, int n_grads, const double *lr,
	const double *grad_scale, float *ms_total, float *ms_sumsq, float *ms_update)
{
	std::vector<hipEvent_t> ev;
	hipStream_t st;
	int rc = 0;
	const bool per_kernel = ms_sumsq || ms_update;

	if (!opt || count <= 0 || !lr || !grad_scale || !ms_total || !gpu_available())
		return -1;
	if (grads && n_grads <= 0)
		return -1;
	st = (hipStream_t)anni_gpu_stream();
	/*
	** Per kernel: ev[0] before the first step, then per step the events after the sum of squares,
	** after the update and (only with derived outputs) after those; a step begins where the one
	** before ended.  Every record costs the stream a few microseconds between two kernels, so
	** there is none that is not read.
	*/
	const bool derived = opt->d_param_fp8 != nullptr;
	const size_t per_step = derived ? 3 : 2;

	ev.resize(per_kernel ? (size_t)count * per_step + 1 : 2);
	for (size_t i = 0; i < ev.size(); i++)
		if (hipEventCreate(&ev[i]) != hipSuccess) {
			for (size_t k = 0; k < i; k++)
				(void)hipEventDestroy(ev[k]);
			(void)hipGetLastError();
			return -1;
		}
	if (!per_kernel)
		(void)hipEventRecord(ev[0], st);
	for (int i = 0; i < count && rc == 0; i++) {
		void *four[4] = { nullptr, nullptr, nullptr, nullptr };

		if (per_kernel) {
			const size_t at = 1 + (size_t)i * per_step;

			four[0] = i == 0 ? ev[0] : nullptr;
			four[1] = ev[at];
			four[2] = ev[at + 1];
			four[3] = derived ? ev[at + 2] : nullptr;
		}
		if (grads)
			(void)anni_adam_bind_grad(opt, grads[i % n_grads]);
		rc = anni_hook_step_events(opt, lr[i], grad_scale[i], four);
		if (rc == 1)
			rc = -1;		/* a timed run must not contain no-op steps */
	}
	if (!per_kernel)
		(void)hipEventRecord(ev[1], st);
	if (gpu_stream_sync() != 0)
		rc = -1;
	if (rc == 0) {
		float ms = 0.0f;

		if (per_kernel) {
			float a = 0.0f, b = 0.0f, d = 0.0f;

			for (int i = 0; i < count; i++) {
				const size_t at = 1 + (size_t)i * per_step;
				float x = 0.0f, y = 0.0f, w = 0.0f;

				(void)hipEventElapsedTime(&x, ev[at - 1], ev[at]);
				(void)hipEventElapsedTime(&y, ev[at], ev[at + 1]);
				if (derived)
					(void)hipEventElapsedTime(&w, ev[at + 1], ev[at + 2]);
				a += x;
				b += y;
				d += w;
			}
			g_last_derived_ms = d;
			(void)hipEventElapsedTime(&ms, ev[0], ev[ev.size() - 1]);
			if (ms_sumsq)
				*ms_sumsq = a;
			if (ms_update)
				*ms_update = b;
		} else {
			(void)hipEventElapsedTime(&ms, ev[0], ev[1]);
		}
		*ms_total = ms;
	}
	for (size_t i = 0; i < ev.size(); i++)
		(void)hipEventDestroy(ev[i]);
	(void)hipGetLastError();
	return rc;
}

} /* namespace anni_bench */

using namespace anni_bench;

extern "C" {

int anni_adam_time_steps(anni_adam *opt, int count, void *const *grads, int n_grads,
	const double *lr, const double *grad_scale, float *ms_total, float *ms_sumsq,
	float *ms_update)
{
	try {
		return time_steps_body(opt, count, grads, n_grads, lr, grad_scale, ms_total, ms_sumsq,
		    ms_update);
	} catch (...) {
		return -1;
	}
}

float anni_adam_timed_derived_ms(const anni_adam *opt)
{
	return opt ? g_last_derived_ms : 0.0f;
}

int anni_fill_normal_f32(float *d_x, int64_t n, uint64_t seed, uint64_t stream, float mean,
	float std)
{
	if (!d_x || n <= 0 || !gpu_available())
		return -1;
	hipLaunchKernelGGL(fill_normal_kernel, dim3(util_grid((n + 1) / 2)), dim3(kLanes), 0,
	    (hipStream_t)anni_gpu_stream(), d_x, n, seed, stream, mean, std);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int anni_copy_bytes(void *d_dst, const void *d_src, size_t nbytes)
{
	if (!d_dst || !d_src || nbytes == 0 || (nbytes & 15) || ((uintptr_t)d_dst & 15)
	    || ((uintptr_t)d_src & 15) || !gpu_available())
		return -1;
	hipLaunchKernelGGL(copy16_kernel, dim3(util_grid((int64_t)(nbytes / 16))), dim3(kLanes), 0,
	    (hipStream_t)anni_gpu_stream(), d_dst, d_src, nbytes / 16);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

int anni_copy_bytes_tiled(void *d_dst, const void *d_src, size_t nbytes, int nontemporal)
{
	const size_t pieces = nbytes / 16384;
	const size_t done = pieces * 16384;
	hipStream_t st;

	if (!d_dst || !d_src || nbytes == 0 || (nbytes & 15) || ((uintptr_t)d_dst & 15)
	    || ((uintptr_t)d_src & 15) || pieces > 0x7fffffffu || !gpu_available())
		return -1;
	st = (hipStream_t)anni_gpu_stream();
	if (pieces > 0) {
		if (nontemporal)
			hipLaunchKernelGGL((copy_tiled_kernel<true>), dim3((unsigned)pieces), dim3(kLanes), 0, st,
			    d_dst, d_src);
		else
			hipLaunchKernelGGL((copy_tiled_kernel<false>), dim3((unsigned)pieces), dim3(kLanes), 0, st,
			    d_dst, d_src);
	}
	if (done < nbytes)
		hipLaunchKernelGGL(copy16_kernel, dim3(util_grid((int64_t)((nbytes - done) / 16))), dim3(kLanes), 0,
		    st, (char *)d_dst + done, (const char *)d_src + done, (nbytes - done) / 16);
	return hipGetLastError() == hipSuccess ? 0 : -1;
}

void anni_gpu_reload_switches(void)
{
	anni_hook_reload_switches();
}

int anni_fold_guard_stats(int *runs, int *mismatches)
{
	if (runs)
		*runs = (int)anni_hook_counter("fold_guard_runs");
	if (mismatches)
		*mismatches = (int)anni_hook_counter("fold_guard_mismatches");
	return 0;
}

int anni_early_sum_stats(long *used, long *dropped)
{
	if (used)
		*used = anni_hook_counter("early_sum_used");
	if (dropped)
		*dropped = anni_hook_counter("early_sum_dropped");
	return 0;
}

int anni_second_stream_state(void)
{
	return (int)anni_hook_counter("second_stream");
}

int anni_vectors_first_stats(long *steps, long *served)
{
	if (steps)
		*steps = anni_hook_counter("vectors_first_steps");
	if (served)
		*served = anni_hook_counter("vectors_first_served");
	return 0;
}

} /* extern "C" */

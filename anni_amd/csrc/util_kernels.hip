/*
** Producers either side of the optimizer step, as device utilities: a seeded
** normal generator for synthetic parameters / gradients, the float -> bf16
** conversion, and per-tensor FP8 (E4M3) quantisation by the reference's scale
** convention (num/gpu_cuda.cu:796-851,927-938).  None of them is on the timed
** path of the step.
*/
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "adam_kernels.h"
#include "anni_adam.h"
#include "backend_state.h"

namespace anni {

/* splitmix64 finaliser: a bijective 64-bit mix, used as a counter-based generator. */
__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
	z += 0x9e3779b97f4a7c15ull;
	z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
	z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
	return z ^ (z >> 31);
}

/* Element pair k of (seed, stream) -> two standard normals (Box-Muller). */
__global__ __launch_bounds__(kThreads) void fill_normal_kernel(float *x, int64_t n,
	uint64_t seed, uint64_t stream, float mean, float std)
{
	const int64_t pairs = (n + 1) / 2;
	const int64_t stride = (int64_t)gridDim.x * kThreads;
	const uint64_t key = mix64(seed ^ mix64(stream));

	for (int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x; k < pairs; k += stride) {
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

/* amax[0] = max |x| as unsigned bits (non-negative floats order like integers); NaNs are ignored. */
__global__ __launch_bounds__(kThreads) void amax_kernel(uint32_t *amax, const float *x, int64_t n)
{
	__shared__ float lds[4];
	const int64_t stride = (int64_t)gridDim.x * kThreads;
	float m = 0.0f;

	for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
		m = fmaxf(m, fabsf(x[i]));
#pragma unroll
	for (int off = 32; off > 0; off >>= 1)
		m = fmaxf(m, __shfl_down(m, off, 64));
	if ((threadIdx.x & 63) == 0)
		lds[threadIdx.x >> 6] = m;
	__syncthreads();
	if (threadIdx.x == 0) {
		m = fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
		if (m > 0.0f)
			atomicMax(amax, __float_as_uint(m));
	}
}

/* In place: the amax word becomes the tensor's scale. */
__global__ void amax_to_scale_kernel(float *word)
{
	if (blockIdx.x == 0 && threadIdx.x == 0)
		word[0] = scale_from_amax(word[0]);
}

__global__ __launch_bounds__(kThreads) void fp8_quantize_kernel(uint8_t *q, const float *scale,
	const float *x, int64_t n)
{
	const int64_t stride = (int64_t)gridDim.x * kThreads;
	const float inv = 1.0f / scale[0];

	for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
		q[i] = (uint8_t)fp8_e4m3_encode(x[i] * inv);
}

/* dst[i] = src[i] over n16 16-byte words: a plain copy of known size (counter calibration). */
__global__ __launch_bounds__(kThreads) void copy16_kernel(void *dst, const void *src, size_t n16)
{
	typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
	const size_t stride = (size_t)gridDim.x * kThreads;

	for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n16; i += stride)
		((u32x4 *)dst)[i] = ((const u32x4 *)src)[i];
}

static int util_grid(int64_t items)
{
	int64_t g = (items + kThreads - 1) / kThreads;

	if (g > 2048)
		g = 2048;
	if (g < 1)
		g = 1;
	return (int)g;
}

} /* namespace anni */

using namespace anni;

extern "C" {

int anni_fill_normal_f32(float *d_x, int64_t n, uint64_t seed, uint64_t stream, float mean,
	float std)
{
	if (!d_x || n <= 0 || !device_ready())
		return -1;
	hipLaunchKernelGGL(fill_normal_kernel, dim3(util_grid((n + 1) / 2)), dim3(kThreads), 0,
	    compute_stream(), d_x, n, seed, stream, mean, std);
	return hip_ok(hipGetLastError(), "fill_normal") ? 0 : -1;
}

int anni_f32_to_bf16(void *d_dst, const float *d_src, int64_t n)
{
	if (!d_dst || !d_src || n <= 0 || !device_ready())
		return -1;
	return launch_f32_to_bf16(compute_stream(), (uint16_t *)d_dst, d_src, n);
}

int anni_copy_bytes(void *d_dst, const void *d_src, size_t nbytes)
{
	if (!d_dst || !d_src || nbytes == 0 || (nbytes & 15) || ((uintptr_t)d_dst & 15)
	    || ((uintptr_t)d_src & 15) || !device_ready())
		return -1;
	hipLaunchKernelGGL(copy16_kernel, dim3(util_grid((int64_t)(nbytes / 16))), dim3(kThreads), 0,
	    compute_stream(), d_dst, d_src, nbytes / 16);
	return hip_ok(hipGetLastError(), "copy_bytes") ? 0 : -1;
}

int anni_fp8_quantize(void *d_q, float *d_scale, const float *d_src, int64_t n)
{
	hipStream_t st;

	if (!d_q || !d_scale || !d_src || n <= 0 || !device_ready())
		return -1;
	st = compute_stream();
	/* d_scale doubles as the amax word: cleared, raised to max|x|, turned into the scale, then read. */
	if (launch_fill_bytes(st, d_scale, 0, sizeof(float)) != 0)
		return -1;
	hipLaunchKernelGGL(amax_kernel, dim3(util_grid(n)), dim3(kThreads), 0, st,
	    (uint32_t *)d_scale, d_src, n);
	hipLaunchKernelGGL(amax_to_scale_kernel, dim3(1), dim3(64), 0, st, d_scale);
	hipLaunchKernelGGL(fp8_quantize_kernel, dim3(util_grid(n)), dim3(kThreads), 0, st,
	    (uint8_t *)d_q, (const float *)d_scale, d_src, n);
	return hip_ok(hipGetLastError(), "fp8_quantize") ? 0 : -1;
}

} /* extern "C" */

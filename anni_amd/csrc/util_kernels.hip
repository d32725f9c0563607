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

/* ---- column sums in the host loop's order ----------------------------------------- */

constexpr int kCsCols = 64;		/* columns per workgroup: one per lane of the summing wavefront */
constexpr int kCsWaves = 8;
constexpr int kCsRows = 16;		/* rows a wavefront fetches per round */
constexpr int kCsRound = kCsWaves * kCsRows;

/*
** acc[c] = (...((acc[c] + t_0) + t_1) ... + t_{rows-1}) in float, t_r = x[r][c] (PROD: the float
** product x[r][c] * y[r][c]), rows strictly in order: bit for bit what the reference's host
** loops leave in a bias or LayerNorm gradient (lang/ffn.c:301-305,358-362,
** lang/layernorm.c:368-372).  Float addition does not associate, so the chain of one column
** cannot be split; what is spread out is everything else: a workgroup owns 64 columns, its
** eight wavefronts keep 128 rows of loads in flight and park them in LDS, and while wavefront 0
** walks one parked round in order the loads of the next round are already under way (two LDS
** buffers, one barrier per round).  The chain costs a few cycles per row; the matrix streams
** from HBM once, in 256-byte row segments.
*/
template <bool PROD>
__global__ __launch_bounds__(kCsWaves * 64) void colsum_add_kernel(float *acc, const float *x,
	const float *y, int64_t rows, int cols)
{
	__shared__ float park[2][kCsRound][kCsCols];
	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int64_t c = (int64_t)blockIdx.x * kCsCols + lane;
	const bool live = c < cols;
	const int64_t n_rounds = (rows + kCsRound - 1) / kCsRound;
	float rx[kCsRows], ry[kCsRows];
	float a = (wave == 0 && live) ? acc[c] : 0.0f;

#pragma unroll
	for (int i = 0; i < kCsRows; i++) {
		const int64_t r = (int64_t)wave * kCsRows + i;
		const bool in = live && r < rows;

		rx[i] = in ? x[r * cols + c] : 0.0f;
		ry[i] = (PROD && in) ? y[r * cols + c] : 1.0f;
	}
	for (int64_t round = 0; round < n_rounds; round++) {
		float (*b)[kCsCols] = park[round & 1];

#pragma unroll
		for (int i = 0; i < kCsRows; i++)
			b[wave * kCsRows + i][lane] = PROD ? rx[i] * ry[i] : rx[i];
		__syncthreads();
		if (round + 1 < n_rounds) {
#pragma unroll
			for (int i = 0; i < kCsRows; i++) {
				const int64_t r = (round + 1) * kCsRound + (int64_t)wave * kCsRows + i;
				const bool in = live && r < rows;

				rx[i] = in ? x[r * cols + c] : 0.0f;
				ry[i] = (PROD && in) ? y[r * cols + c] : 1.0f;
			}
		}
		if (wave == 0) {
			const int64_t left = rows - round * kCsRound;

			if (left >= kCsRound) {
#pragma unroll 16
				for (int i = 0; i < kCsRound; i++)
					a += b[i][lane];
			} else {
				/* rows past the end are never added: x + 0 is not x for x = -0 */
				for (int i = 0; i < (int)left; i++)
					a += b[i][lane];
			}
		}
	}
	if (wave == 0 && live)
		acc[c] = a;
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

int anni_colsum_add(float *d_acc, const float *d_x, const float *d_y, int64_t rows, int cols)
{
	const int64_t groups = ((int64_t)cols + kCsCols - 1) / kCsCols;

	if (!d_acc || !d_x || rows < 0 || cols <= 0 || !device_ready())
		return -1;
	if (rows == 0)
		return 0;
	if (d_y)
		hipLaunchKernelGGL((colsum_add_kernel<true>), dim3((unsigned)groups), dim3(kCsWaves * 64),
		    0, compute_stream(), d_acc, d_x, d_y, rows, cols);
	else
		hipLaunchKernelGGL((colsum_add_kernel<false>), dim3((unsigned)groups),
		    dim3(kCsWaves * 64), 0, compute_stream(), d_acc, d_x, d_y, rows, cols);
	return hip_ok(hipGetLastError(), "colsum_add") ? 0 : -1;
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

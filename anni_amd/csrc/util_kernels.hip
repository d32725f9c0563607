/*
** Producers either side of the optimizer step, as device utilities: the float -> bf16
** conversion, per-tensor FP8 (E4M3) quantisation by the reference's scale convention
** (num/gpu_cuda.cu:796-851,927-938) and the bias / LayerNorm gradient column sums.  None of
** them is on the timed path of the step.
*/
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <mutex>
#include "adam_kernels.h"
#include "anni_adam.h"
#include "anni_gpu.h"
#include "backend_state.h"

namespace anni {

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

/* ---- column sums in the host loop's order ----------------------------------------- */

constexpr int kCsCols = 64;		/* columns per workgroup: one per lane */
/*
** Wavefronts per workgroup: eight turns cover the latency of the loads; 12 and 16 were measured
** no faster (a narrow matrix is bound by the chain and the hand-over, ~5 ns a row, not by loads).
*/
template <bool PROD> struct CsWaves { static constexpr int n = 8; };
/*
** Rows per chunk = what one wavefront holds in registers.  (With two matrices a chunk is 128
** loads, more than the 63 a wavefront can have outstanding, so that variant waits inside its
** fetches and runs at about half the rate; 32-row chunks were measured slower still, the
** hand-over between wavefronts then costs more than the waits.)
*/
template <bool PROD> struct CsRows { static constexpr int n = 64; };

/*
** Rows FIRST .. FIRST + COUNT - 1 of a chunk of the lane's column into registers, as raw buffer loads: the
** descriptor (scalar registers) starts at the chunk's first row, the row offset is a scalar, the
** lane supplies only its constant column offset -- no vector arithmetic per load.  The one chunk
** of a column that runs past the matrix reads its last valid row again for the rows beyond it
** (those registers are never added): there the scalar row index is clamped, so every address
** lies inside the matrix by construction.  (The descriptor's range check is not relied on for
** this: it compares the vector offset only, the scalar offset takes no part in it.)  A select on
** a loaded value instead would make the wavefront wait for the load on the spot.
*/
template <bool PROD, int FIRST, int COUNT>
__device__ __forceinline__ void colsum_fetch(float (&rx)[CsRows<PROD>::n], float (&ry)[CsRows<PROD>::n],
	const float *x, const float *y, int64_t chunk, int64_t rows, int cols, uint32_t col_bytes)
{
	constexpr int kCsRows = CsRows<PROD>::n;
	const int64_t r0 = chunk * kCsRows;

	if (r0 >= rows)
		return;
	const int64_t rows_left = rows - r0;
	const uint32_t last = (uint32_t)(rows_left < kCsRows ? rows_left - 1 : kCsRows - 1);
	const uint64_t left = (uint64_t)rows_left * (uint64_t)cols * sizeof(float);
	const uint32_t span = left < 0xffffffffull ? (uint32_t)left : 0xffffffffu;
	const __amdgpu_buffer_rsrc_t bx = __builtin_amdgcn_make_buffer_rsrc(
	    (void *)(x + r0 * cols), 0, (int)span, 0x00020000);
	const __amdgpu_buffer_rsrc_t by = __builtin_amdgcn_make_buffer_rsrc(
	    (void *)((PROD ? y : x) + r0 * cols), 0, (int)span, 0x00020000);
	const uint32_t pitch = (uint32_t)cols * (uint32_t)sizeof(float);

	if (rows_left >= kCsRows) {
		/* a whole chunk (all but the last one of a column): the row offsets are multiples of the pitch */
#pragma unroll
		for (int i = FIRST; i < FIRST + COUNT; i++) {
			rx[i] = __builtin_bit_cast(float,
			    __builtin_amdgcn_raw_buffer_load_b32(bx, (int)col_bytes, (int)(i * pitch), 0));
			if (PROD)
				ry[i] = __builtin_bit_cast(float,
				    __builtin_amdgcn_raw_buffer_load_b32(by, (int)col_bytes, (int)(i * pitch), 0));
		}
		return;
	}
#pragma unroll
	for (int i = FIRST; i < FIRST + COUNT; i++) {
		const uint32_t row = (uint32_t)i < last ? (uint32_t)i : last;

		rx[i] = __builtin_bit_cast(float,
		    __builtin_amdgcn_raw_buffer_load_b32(bx, (int)col_bytes, (int)(row * pitch), 0));
		if (PROD)
			ry[i] = __builtin_bit_cast(float,
			    __builtin_amdgcn_raw_buffer_load_b32(by, (int)col_bytes, (int)(row * pitch), 0));
	}
}

/*
** acc[c] = (...((acc[c] + t_0) + t_1) ... + t_{rows-1}) in float, t_r = x[r][c] (PROD: the float
** product x[r][c] * y[r][c]), rows strictly in order: bit for bit what the reference's host
** loops leave in a bias or LayerNorm gradient (lang/ffn.c:301-305,358-362,
** lang/layernorm.c:368-372).  Float addition does not associate, so the chain of one column
** cannot be split; what is spread out is the memory traffic.  A workgroup owns 64 columns, one
** per lane.  Its eight wavefronts take chunks of 64 rows in turn: a wavefront holds its chunk
** in registers (loaded several turns earlier), picks the running sums up from LDS, adds its
** rows in order and hands the sums on; during the four following turns it fetches the chunk of
** its next turn.  So ~100 KiB per workgroup are in flight while the chain runs at register speed,
** or at the HBM rate where the matrix is wide.  One barrier per chunk; no wavefront ever waits
** for a later one.
*/
constexpr int kCsMaxJobs = 16;

/* One column sum of a launch; the jobs of a launch travel by value in the kernel arguments. */
struct CsJob {
	float		*acc;
	const float	*x;
	const float	*y;
	int64_t		rows;
	int		cols;
	int		first_group;	/* workgroups [first_group, next job's first_group) work on this job */
};

struct CsJobs {
	int	n;
	CsJob	job[kCsMaxJobs];
};

template <bool PROD>
__global__ __launch_bounds__(CsWaves<PROD>::n * 64) void colsum_add_kernel(CsJobs jobs)
{
	constexpr int kCsRows = CsRows<PROD>::n;
	constexpr int kCsWaves = CsWaves<PROD>::n;
	__shared__ float carry[kCsCols];
	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	int k = 0;

	while (k + 1 < jobs.n && (int)blockIdx.x >= jobs.job[k + 1].first_group)
		k++;
	float *const acc = jobs.job[k].acc;
	const float *const x = jobs.job[k].x;
	const float *const y = jobs.job[k].y;
	const int64_t rows = jobs.job[k].rows;
	const int cols = jobs.job[k].cols;
	const int64_t c_own = (int64_t)((int)blockIdx.x - jobs.job[k].first_group) * kCsCols + lane;
	const bool live = c_own < cols;
	const uint32_t c = (uint32_t)(live ? c_own : cols - 1);
	const uint32_t col_bytes = c * (uint32_t)sizeof(float);
	const int64_t n_chunks = (rows + kCsRows - 1) / kCsRows;
	int64_t done = 0;		/* chunks added so far = barriers passed, the same in every wavefront */
	float rx[kCsRows], ry[kCsRows];

	if (wave == 0)
		carry[lane] = acc[c];
	colsum_fetch<PROD, 0, kCsRows>(rx, ry, x, y, wave, rows, cols, col_bytes);
	if (PROD) {
		/* products are rounded to float before they are added: no fused multiply-add */
#pragma unroll
		for (int i = 0; i < kCsRows; i++)
			rx[i] = rx[i] * ry[i];
	}
	__syncthreads();
	/*
	** Every wavefront runs the same cycle of eight chunks -- own turn, four chunks during each
	** of which it fetches a quarter of its next chunk, two idle chunks, multiply -- shifted by its
	** index, with one barrier per chunk.  (One loop with the phase as a run-time value made the
	** compiler copy the row registers at the loop end, which waits for every load in flight.)
	*/
	for (int k = 0; k < wave && done < n_chunks; k++) {
		__syncthreads();
		done++;
	}
	while (done < n_chunks) {
		{
			const int64_t left = rows - done * kCsRows;
			float a = carry[lane];

			if (left >= kCsRows) {
#pragma unroll
				for (int i = 0; i < kCsRows; i++)
					a += rx[i];
			} else {
				/* rows past the end are never added: x + 0 is not x for x = -0 */
#pragma unroll
				for (int i = 0; i < kCsRows; i++)
					if (i < left)
						a += rx[i];
			}
			carry[lane] = a;
		}
		__syncthreads();
		if (++done >= n_chunks)
			break;
		/*
		** Not inside the own turn, and a quarter at a time: issuing the loads of a whole chunk takes
		** as long as the chain of one, and would hold up the barrier the next chain waits on.
		*/
		colsum_fetch<PROD, 0, kCsRows / 4>(rx, ry, x, y, done - 1 + kCsWaves, rows, cols, col_bytes);
		__syncthreads();
		if (++done >= n_chunks)
			break;
		colsum_fetch<PROD, kCsRows / 4, kCsRows / 4>(rx, ry, x, y, done - 2 + kCsWaves, rows, cols,
		    col_bytes);
		__syncthreads();
		if (++done >= n_chunks)
			break;
		colsum_fetch<PROD, kCsRows / 2, kCsRows / 4>(rx, ry, x, y, done - 3 + kCsWaves, rows, cols,
		    col_bytes);
		__syncthreads();
		if (++done >= n_chunks)
			break;
		colsum_fetch<PROD, 3 * kCsRows / 4, kCsRows / 4>(rx, ry, x, y, done - 4 + kCsWaves, rows,
		    cols, col_bytes);
		__syncthreads();
		if (++done >= n_chunks)
			break;
#pragma unroll 1
		for (int k = 5; k < kCsWaves - 1 && done < n_chunks; k++) {
			__syncthreads();
			done++;
		}
		if (done >= n_chunks)
			break;
		if (PROD) {
#pragma unroll
			for (int i = 0; i < kCsRows; i++)
				rx[i] = rx[i] * ry[i];
		}
		__syncthreads();
		done++;
	}
	if (wave == 0 && live)
		acc[c] = carry[lane];
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

int anni_f32_to_bf16(void *d_dst, const float *d_src, int64_t n)
{
	if (!d_dst || !d_src || n <= 0 || !device_ready())
		return -1;
	return launch_f32_to_bf16(compute_stream(), (uint16_t *)d_dst, d_src, n);
}

int anni_colsum_add_batch(const anni_colsum *jobs, int n_jobs)
{
	CsJobs plain, prod;
	int groups[2] = { 0, 0 };

	if (!jobs || n_jobs <= 0 || n_jobs > kCsMaxJobs || !device_ready())
		return -1;
	plain.n = 0;
	prod.n = 0;
	for (int i = 0; i < n_jobs; i++) {
		const anni_colsum &j = jobs[i];

		/* 63 row pitches must fit the 32-bit scalar offset of a buffer load */
		if (!j.d_acc || !j.d_x || j.rows < 0 || j.cols <= 0 || j.cols > (1 << 24))
			return -1;
		if (j.rows == 0)
			continue;
		CsJobs &dst = j.d_y ? prod : plain;
		CsJob &c = dst.job[dst.n++];

		c.acc = j.d_acc;
		c.x = j.d_x;
		c.y = j.d_y;
		c.rows = j.rows;
		c.cols = j.cols;
		c.first_group = groups[j.d_y ? 1 : 0];
		groups[j.d_y ? 1 : 0] += (j.cols + kCsCols - 1) / kCsCols;
	}
	if (plain.n)
		hipLaunchKernelGGL((colsum_add_kernel<false>), dim3((unsigned)groups[0]),
		    dim3(CsWaves<false>::n * 64), 0, compute_stream(), plain);
	if (prod.n)
		hipLaunchKernelGGL((colsum_add_kernel<true>), dim3((unsigned)groups[1]),
		    dim3(CsWaves<true>::n * 64), 0, compute_stream(), prod);
	return hip_ok(hipGetLastError(), "colsum_add") ? 0 : -1;
}

int anni_colsum_add(float *d_acc, const float *d_x, const float *d_y, int64_t rows, int cols)
{
	anni_colsum job;

	job.d_acc = d_acc;
	job.d_x = d_x;
	job.d_y = d_y;
	job.rows = rows;
	job.cols = cols;
	return anni_colsum_add_batch(&job, 1);
}

int gpu_mat_col_sum_add(ann_real *db_host, const ann_real *x, int rows, int cols)
{
	static std::mutex mu;			/* one accumulator, grown on demand */
	static float *d_acc;
	static int d_acc_cols;
	hipPointerAttribute_t attr;
	hipStream_t st;
	int rc = -1;

	if (!db_host || !x || rows <= 0 || cols <= 0 || !device_ready())
		return -1;
	if (hipPointerGetAttributes(&attr, x) != hipSuccess || attr.type != hipMemoryTypeDevice) {
		(void)hipGetLastError();
		return -1;			/* a host matrix: the caller's own loop */
	}
	std::lock_guard<std::mutex> lk(mu);

	if (cols > d_acc_cols) {
		void *p = nullptr;

		if (!hip_ok(device_alloc(&p, (size_t)cols * sizeof(float)), "colsum hipMalloc")) {
			(void)hipGetLastError();
			return -1;
		}
		if (d_acc)
			(void)hipFree(d_acc);
		d_acc = (float *)p;
		d_acc_cols = cols;
	}
	st = compute_stream();
	if (hip_ok(hipMemcpyAsync(d_acc, db_host, (size_t)cols * sizeof(float), hipMemcpyHostToDevice, st),
	    "colsum h2d")
	    && anni_colsum_add(d_acc, x, nullptr, rows, cols) == 0
	    && hip_ok(hipMemcpyAsync(db_host, d_acc, (size_t)cols * sizeof(float), hipMemcpyDeviceToHost,
	    compute_stream()), "colsum d2h")
	    && hip_ok(sync_stream_and_deliver(), "colsum sync"))
		rc = 0;
	return rc;
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

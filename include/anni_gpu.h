/*
** anni_gpu.h -- the optimizer-step subset of AnnI's backend C ABI, served by the
** MI355X (gfx950, HIP) backend libanni_gpu_hip.so.
**
** The reference selects its backend at link time: one object exporting the
** functions of num/gpu.h (reference Makefile:27-29,198-204: gpu_stub.o or
** gpu_cuda.o).  libanni_gpu_hip.so is a third choice.  It exports every symbol of
** num/gpu.h; the ones below are the ones lang/lm_adam.c calls on the optimizer
** step and they do real work on the GPU.  The remaining symbols (GEMM,
** attention, LayerNorm, decode ...: anni_gpu_unserved.h) answer "not done here,
** use your CPU path" exactly as the reference's CPU stub does, because that
** work is outside this library's scope.
**
** Conventions, as in the reference (num/gpu.h:125-127,134-139): int results are
** 0 = done, -1 = the caller must use its CPU path; pointer results are NULL on
** failure; nothing throws, nothing sets errno.  Every asynchronous operation
** and kernel is issued on one in-order compute stream; gpu_memcpy_d2h blocks.
** Buffers are owned by the caller (gpu_malloc / gpu_free); the backend only
** borrows the registered twin flat.
**
** Threads: gpu_grad_sumsq and gpu_adam_step_dev_bf16 keep one result slot, one
** set of partial sums and one set of ticket words per process, as the reference's
** do (static s_acc, num/gpu_cuda.cu:8485-8486): they are for ONE thread on the
** library's one compute stream.  The memory functions may be called from any thread.
**
** Order of completion is the order of the calls, always.  Within that contract the
** library may begin work before it is asked for, on a second stream of its own, when
** a caller has shown the call order of lang/lm_adam.c:452-515 twice in a row (small
** uploads, the sum of squares, the update, small read-backs, a synchronisation); see
** gpu_grad_sumsq and gpu_adam_step_dev_bf16 below.  Results do not depend on it.
*/
#ifndef ANNI_GPU_H__
#define ANNI_GPU_H__

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* num/real.h:3 */
#ifndef ANN_REAL_H__
typedef float ann_real;
#endif

/* num/gpu.h:23-24 */
#ifndef GPU_PREC_FP32
#define GPU_PREC_FP32	0
#define GPU_PREC_BF16	1
#endif

/* ---- device, stream ---------------------------------------------------- */

/* num/gpu.h:11 -- 1 when a HIP device is usable (creates the compute stream on first call). */
int	gpu_available(void);
/* num/gpu.h:12 -- "hip-gfx950". */
const char	*gpu_backend_name(void);
/* num/gpu.h:14 -- free / total device memory in bytes; 0 ok, -1 no device. */
int	gpu_mem_info(size_t *free_bytes, size_t *total_bytes);
/* num/gpu.h:38 -- block until all queued device work has finished. */
void	gpu_device_sync(void);
/* num/gpu.h:47 -- block until the compute stream has drained; 0 ok. */
int	gpu_stream_sync(void);
/* num/gpu.h:25 -- BF16 twins are written by the step only in GPU_PREC_BF16 (gpu_cuda.cu:8687,8704). */
void	gpu_set_compute_prec(int prec);
/* num/gpu.h:64 -- pending HIP error text, cleared by the call; "" when none. */
const char	*gpu_debug_last_error(void);
/* num/gpu.h:66 -- ANN_OP_PROF=1: print and reset the optimizer-step timing table (stderr). */
void	gpu_op_prof_dump(void);

/* ---- memory ------------------------------------------------------------ */

/* num/gpu.h:40-41 -- device allocation; thread-safe; gpu_free forgets registrations keyed on p. */
void	*gpu_malloc(size_t nbytes);
void	gpu_free(void *p);
/* num/gpu.h:42 -- host to device, ordered on the compute stream. */
int	gpu_memcpy_h2d(void *dst, const void *src, size_t nbytes);
/* num/gpu.h:43 -- device to host, synchronous: dst is valid on return. */
int	gpu_memcpy_d2h(void *dst, const void *src, size_t nbytes);
/* num/gpu.h:45 -- mark a host range as a target of later asynchronous copies (idempotent). */
int	gpu_host_pin(void *p, size_t nbytes);
/* num/gpu.h:46 -- device to host on the compute stream; valid after gpu_stream_sync. */
int	gpu_memcpy_d2h_async(void *dst, const void *src, size_t nbytes);
/* num/gpu.h:48 -- device to device on the compute stream. */
int	gpu_memcpy_d2d(void *dst, const void *src, size_t nbytes);
/* num/gpu.h:49 -- byte fill on the compute stream. */
int	gpu_memset(void *dst, int value, size_t nbytes);
/* num/gpu.h:62 -- a host vector is being freed: drop what was remembered about it. */
void	gpu_host_forget(const void *host);
/* num/gpu.h:312-313 -- page-locked host allocation for staging. */
void	*gpu_host_alloc(size_t nbytes);
void	gpu_host_free(void *p);

/* ---- BF16 twins -------------------------------------------------------- */

/* num/gpu.h:71 -- register (borrow) the flat BF16 twin of Adam's d_param; NULL,NULL,0 clears. */
void	gpu_adam_set_bf16_flat(void *bf16, const ann_real *fp32, int n);
/* num/gpu.h:73 -- one-shot FP32 -> BF16 (round to nearest even) of the flat. */
int	gpu_adam_seed_bf16_flat(void *bf16, const ann_real *fp32, int n);
/* num/gpu.h:56 -- weights were rewritten: bump the weight epoch (NULL = everything). */
void	gpu_half_wt_invalidate(const ann_real *fp32_dev);
/* num/gpu.h:346 -- changes at every optimizer step. */
unsigned	gpu_param_epoch(void);
/*
** The consumer side of the twin flat: the reference's GEMM wrappers ask half_wt_get for the
** BF16 copy of a device FP32 operand (static in num/gpu_cuda.cu:2018-2034, so not part of
** num/gpu.h; exported here for a GEMM backend written against this library).  A slice
** [fp32_dev, fp32_dev + n) that lies inside the registered flat (gpu_adam_set_bf16_flat) is served
** from the twin flat, bf16 + (fp32_dev - fp32_base) * 2 -- current after every step, no
** conversion; any other pointer gets NULL once a flat is registered (it is an activation and
** must not get a persistent twin), and NULL when none is.  gpu_free of either flat and
** gpu_adam_set_bf16_flat(NULL, NULL, 0) end the service.  ANN_TWIN_CHECK=1 (gpu_cuda.cu:1946-1995):
** every served slice is converted afresh on the device, compared, and a difference reported on
** stderr as "[twin] STALE flat fp32=... n=... bytes_diff=..." (debug aid; synchronises).
*/
const void	*anni_gpu_bf16_twin_of(const ann_real *fp32_dev, size_t n);

/*
** num/gpu.h:195-199 -- db_host[cols] += column sums of the rows x cols matrix x (a bias gradient,
** lang/ffn.c:298,355).  Served when x is DEVICE memory: db_host goes up, the column sums are
** added to it row after row in float exactly as the caller's host loop would add them
** (lang/ffn.c:301-305), the result comes back -- the host loop's bits, where the reference's
** CUDA path keeps device accumulators that it flushes at the next sync (num/gpu_cuda.cu:
** 3131-3193,9972-10030).  Synchronous.  -1 (the caller's host loop runs) for a host x: with this
** backend's host GEMMs that is every call of the unchanged caller; a caller with a
** device-resident backward and an arena adds straight into the gradient flat with
** anni_colsum_add instead.
*/
int	gpu_mat_col_sum_add(ann_real *db_host, const ann_real *x, int rows, int cols);

/* ---- the optimizer step ------------------------------------------------ */

/* num/gpu.h:121 -- decoupled weight decay used by the next step (negative -> 0; sticky). */
void	gpu_adam_set_weight_decay(double wd);
/*
** num/gpu.h:123 -- *out = sum of d_x[i]^2 over n device floats, accumulated in
** double in a fixed order that depends on n alone (run-to-run deterministic).
** Everything put on the compute stream before the call has completed when it
** returns.  -1 also when another thread's call is between its launch and its
** read-back (one result slot per process; the caller takes its CPU path).
** Once the caller has twice in a row synchronised, made nothing but small uploads
** into this flat and the registered parameter flat, and then asked for this sum,
** the sum over the chunks those uploads do not touch is begun at the first such
** upload of the next step; the call then only adds the chunks written since.
** Same bits either way.  ANNI_EARLY_SUM=0 switches that off.
*/
int	gpu_grad_sumsq(const ann_real *d_x, int n, double *out);
/*
** num/gpu.h:129-132 -- flat AdamW step on device pointers of length n:
** g = grad_scale * d_grad, bias-corrected update, decoupled decay, d_grad
** zeroed; the BF16 twins are written when d_param_bf16 != NULL and the
** precision is GPU_PREC_BF16.  Validation as gpu_cuda.cu:8675-8682: -1 for a
** NULL pointer, n <= 0, lr <= 0, t < 1, 1-beta^t <= 0 or no device.
** The arithmetic follows the reference's host loop (lang/lm_adam.c:587-598) in
** double, so results equal the CPU path bit for bit for the same grad_scale.
** Once the caller has read the same list of small ranges of d_param back
** (gpu_memcpy_d2h_async) after two steps in a row, the tiles holding those ranges
** are updated by a launch of their own and copied out ahead of the rest, so that
** gpu_stream_sync can hand them over while the large launch is still running; only
** when the compute stream is idle at the call.  ANNI_VECTORS_FIRST=0 switches that off.
*/
int	gpu_adam_step_dev_bf16(ann_real *d_param, void *d_param_bf16, ann_real *d_grad,
		ann_real *d_m, ann_real *d_v, int n, double lr, double beta1,
		double beta2, double eps, int t, double grad_scale);

#ifdef __cplusplus
}
#endif
#endif

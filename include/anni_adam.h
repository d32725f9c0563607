/*
** anni_adam.h -- device-resident AdamW optimizer over a multi-tensor flat, the
** MI355X counterpart of the reference's lang/lm_adam.{h,c}.
**
** What the reference's flat ABI (num/gpu.h:121-132) cannot express is added
** here: weight decay on selected tensors only, bf16-stored moments, bf16 or
** fp8-E4M3 gradients with a per-tensor scale, the clip norm and the non-finite
** skip decided on the device without a host round trip, and a launch table that
** covers every tensor -- matrices, embeddings, biases, LayerNorm vectors -- in
** one sum-of-squares launch and one update launch per step.
**
** The struct mirrors the public fields of the reference's lm_adam
** (lang/lm_adam.h:30-54): callers set beta1/beta2/eps/weight_decay/grad_clip
** directly and read t / last_grad_norm, as lang/lm_train.c:1336-1351 does.
**
** Arithmetic: the reference's host loop (lang/lm_adam.c:571-598) -- double
** intermediates, float stores after m, v, the step and the decay -- so the FP32
** state equals the CPU path bit for bit under the same effective gradient
** scale; the twins are round-to-nearest-even bf16 of the final p
** (num/gpu_cuda.cu:8578).
**
** Results: 0 = done, -1 = failed (bad argument, no device, launch error); no
** CPU fallback exists in this library.
*/
#ifndef ANNI_ADAM_H__
#define ANNI_ADAM_H__

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element storage types. */
#define ANNI_F32	0
#define ANNI_BF16	1	/* upper 16 bits of an IEEE float */
#define ANNI_FP8_E4M3	2	/* OCP E4M3: bias 7, max 448, S.1111.111 = NaN, no infinities */

/*
** Arena layouts.  MI355X's device memory behaves as three sections of 96 GiB, and a kernel
** that streams several arrays at once is ~15 % faster when they are split over two sections
** than when one holds them all.  SPLIT makes two allocations of exactly the size of their
** contents -- p, m and the tables in one; v, the twins and the gradient slots in the other -- and
** looks for the second in another section by timing the update on the (still empty) flats:
** blocks of its size are requested one after the other and kept, every 8 GiB one is timed, until
** one is fast or the walk has covered one section and one block (96 GiB + the block), never more
** than half of what was free when it began; everything but the arena is returned before
** anni_adam_create returns (anni_adam_placement_cost says what was held and for how long;
** ANNI_PLACE_MAX_GIB sets another limit, 0 = no search).
** COMPACT is one allocation.  AUTO splits when the parameter flat has 256 MiB or more.
*/
#define ANNI_LAYOUT_AUTO	0
#define ANNI_LAYOUT_COMPACT	1
#define ANNI_LAYOUT_SPLIT	2

/* Tensor flags. */
#define ANNI_T_DECAY	1u	/* decoupled weight decay applies (the benchmark configurations: matrices only) */
#define ANNI_T_TWIN	2u	/* the bf16 twin of this tensor is written */
#define ANNI_T_FP8TWIN	4u	/* an E4M3 twin with its own scale is kept current (needs anni_adam_enable_derived) */

/* One registered tensor; tensors are packed in registration order with no padding (lm_adam.c:25-57). */
typedef struct anni_tensor {
	int64_t		n;
	uint32_t	flags;
} anni_tensor;

typedef struct anni_adam_config {
	int	grad_type;	/* ANNI_F32 / ANNI_BF16 / ANNI_FP8_E4M3 */
	int	moment_type;	/* ANNI_F32 / ANNI_BF16 (computed in double, rounded f32 then bf16 on store) */
	int	twins;		/* 1: allocate the bf16 twin flat */
	int	skip_nonfinite;	/* 1: a non-finite gradient norm skips the update (lm_adam.c:474-483) */
	int	grad_slots;	/* gradient flats the arena allocates (slot 0 starts bound); 0: bind one with anni_adam_bind_grad */
	int	layout;		/* ANNI_LAYOUT_AUTO / _COMPACT / _SPLIT */
} anni_adam_config;

/*
** A second home for the bf16 of a row-major matrix: element (r, c) of tensor `tensor`, which
** has `cols` columns, also goes to pack[dst_offset + r * dst_stride + c].  Three of these with
** dst_stride = 3 D and dst_offset = 0, D, 2 D build the [Wq | Wk | Wv] operand that the
** reference rebuilds from the three twins after each step (num/gpu_cuda.cu:6456-6470,6483-6517).
*/
typedef struct anni_pack {
	int	tensor;
	int32_t	cols;
	int64_t	dst_offset;
	int32_t	dst_stride;
} anni_pack;

struct anni_adam_priv;

typedef struct anni_adam {
	int64_t	n;		/* elements in the flat */
	int	n_tensors;
	int	t;		/* steps taken (advanced by every step with lr > 0, lm_adam.c:531-533) */
	double	beta1;		/* defaults 0.9, 0.999, 1e-8, 0, 0 (lm_adam.c:110-115) */
	double	beta2;
	double	eps;
	double	weight_decay;
	double	grad_clip;	/* global L2 clip; 0 = off */
	double	last_sumsq;	/* valid after anni_adam_sync_stats */
	double	last_grad_norm;
	double	last_grad_scale;
	int	last_skipped;
	int	last_clipped;
	anni_adam_config cfg;
	/* the device arena: one or two allocations, each flat 2 MiB aligned (see ANNI_LAYOUT_*) */
	float	*d_param;
	void	*d_param_bf16;
	void	*d_grad;
	void	*d_m;
	void	*d_v;
	float	*d_gscale;	/* per-tensor fp8 dequant scale (n_tensors floats) */
	/* derived outputs, NULL until anni_adam_enable_derived */
	void	*d_param_fp8;	/* E4M3 twins: n bytes, tensor i at byte anni_adam_tensor_offset(i) */
	float	*d_wscale;	/* their per-tensor scales (n_tensors floats; 1 for tensors without a twin) */
	void	*d_pack_bf16;	/* the packed bf16 matrices */
	struct anni_adam_priv *priv;
} anni_adam;

/*
** Counterpart of lm_adam_create + gpu_buffers_init (lm_adam.c:79-139,217-311):
** registers the tensors in order at packed offsets, allocates the arena (p, m,
** v zeroed; gradient slots zeroed), builds the launch table.
** NULL on failure.
*/
anni_adam	*anni_adam_create(const anni_tensor *tensors, int n_tensors,
			const anni_adam_config *cfg);
/* lm_adam_free (lm_adam.c:185-194). */
void	anni_adam_free(anni_adam **opt);
/* Element offset of tensor i in every flat. */
int64_t	anni_adam_tensor_offset(const anni_adam *opt, int i);
/* Gradient slot k of the arena (k < cfg.grad_slots), else NULL. */
void	*anni_adam_grad_slot(const anni_adam *opt, int k);
/* 1 when the layout came out SPLIT. */
int	anni_adam_is_split(const anni_adam *opt);
/*
** What creation measured: time of the update with all flats in one block / time on this arena's
** two blocks, on a probe of 64 M elements (>= 1.07: the halves lie in different sections; ~1.0:
** no such memory was found, or the blocks the driver handed out are pieced together from several
** sections already and there was nothing to gain; 1.0 exactly: compact or not measured), and the
** GB/s of algorithmic traffic the update then reached on the whole arena, whatever its layout
** (0: not measured; needs a gradient slot and a parameter flat of 256 MiB or more).
*/
double	anni_adam_apart_ratio(const anni_adam *opt);
double	anni_adam_probe_gbps(const anni_adam *opt);
/*
** What the search for the second block cost at creation: GiB of device memory requested and held
** while it ran (the block that was kept included) and its wall-clock time; returns the number of
** candidate blocks that were timed (0 for a compact arena or when nothing was searched), -1 for
** a bad handle.
*/
int	anni_adam_placement_cost(const anni_adam *opt, double *walked_gib, double *ms);
/* Device memory the arena holds, and what one step touches (p, m, v, twins, one gradient flat, tables). */
size_t	anni_adam_arena_bytes(const anni_adam *opt);
size_t	anni_adam_resident_bytes(const anni_adam *opt);
/* Use another gradient flat: a slot of the arena or an external one (n elements of grad_type); NULL = slot 0. */
int	anni_adam_bind_grad(anni_adam *opt, void *d_grad);
/*
** Producers of the step's neighbours, fused into the step (no counterpart as code in the
** reference, which rebuilds both after the step: the E4M3 weight copies by an amax pass and a
** quantise pass over p per matrix, num/gpu_cuda.cu:1090-1115,1187-1262, the packed QKV operand
** by a kernel per layer, :6456-6517; docs/low-precision-plan.md:31 asks for this fusion).
** After this call every step also
**   - writes bf16(p) of each packed tensor into its place in d_pack_bf16 (pack_elems bf16), and
**   - keeps q = satfinite_e4m3(p * (1 / scale)), scale = max(amax / 448, 1e-12), current for
**     the tensors flagged ANNI_T_FP8TWIN: the update reduces max |p| per tensor while it
**     holds the new values, one more launch reads p and writes q and d_wscale.  The bytes and
**     scales equal what the reference's fp8_quant_now gives on the new weights.
** A step skipped for a non-finite norm leaves both as they are.  Call once, before
** anni_adam_seed_twins; -1 when nothing is flagged and no pack is given, or on a bad descriptor.
*/
int	anni_adam_enable_derived(anni_adam *opt, const anni_pack *packs, int n_packs,
		int64_t pack_elems);
/* gpu_adam_seed_bf16_flat: twins = bf16(p) for the whole flat (after loading weights); also seeds the derived outputs. */
int	anni_adam_seed_twins(anni_adam *opt);
/* lm_adam_zero_grad: clears the gradient flat on the stream. */
int	anni_adam_zero_grad(anni_adam *opt);
/*
** The producer side of the fp8 gradient format (grad_type ANNI_FP8_E4M3): d_src, a device flat
** of n floats in the optimizer's tensor order (16-byte aligned), is quantised into the bound
** gradient flat and d_gscale, every tensor with its own scale = max(max|x| / 448, 1e-12) and
** q = E4M3(x * (1 / scale)), saturating -- the arithmetic of anni_fp8_quantize and of the
** reference's FP8 quantiser (num/gpu_cuda.cu:826-851,927-938) on each tensor, in four launches
** for the whole flat instead of four per tensor.  Asynchronous on the compute stream; allocates
** its scratch at the first call.  No counterpart in the reference (it has no fp8 gradients).
*/
int	anni_adam_quantize_grads(anni_adam *opt, const float *d_src);
/*
** anni_adam_quantize_grads for callers that cannot allocate device memory (a stream under HIP
** graph capture, a tight serving loop, a harness that forbids hipMalloc): same arguments, same
** codes and scales, but the work area (one word per tensor + 16 bytes per tile of 4096 elements)
** is a fixed array of ANNI_QUANT_STATIC_BYTES in device memory that every GPU the library runs on
** holds until the process ends, instead of a block allocated at the first call.  No counterpart
** in the reference.  Calls no hipMalloc / hipFree; -1 (gpu_debug_last_error says why) for an
** optimizer of more than ANNI_QUANT_STATIC_MAX_ELEMS elements or ANNI_QUANT_STATIC_MAX_TENSORS
** tensors.  All calls on one GPU share the array: calls that overlap in time (two optimizers on
** two streams) race; calls one after the other on the compute stream are fine, each clears what
** it needs cleared.
*/
#define ANNI_QUANT_STATIC_MAX_ELEMS	((int64_t)1 << 31)
#define ANNI_QUANT_STATIC_MAX_TENSORS	4096
#define ANNI_QUANT_STATIC_BYTES		(16384 + (1 << 23))	/* the words + 2^31 / 4096 tiles x 16 bytes */
int	anni_adam_quantize_grads_static(anni_adam *opt, const float *d_src);
/*
** lm_adam_step_scaled (lm_adam.c:522-607): lr <= 0 returns 1 without advancing t;
** otherwise t++, [sum of squares when grad_clip > 0, skip_nonfinite or ANN_GNORM_EVERY > 0,
** lm_adam.c:466], update.  Asynchronous on the compute stream: nothing is read back.  Two
** exceptions: the very first sum of squares on a device waits for the stream once (a self-check
** of its second stage), and with ANN_OP_PROF=1 every step ends with the reference's
** gpu_op_prof_dump (lm_adam.c:541), which waits for the events it prints.
*/
int	anni_adam_step_scaled(anni_adam *opt, double lr, double grad_scale);
/* lm_adam_step. */
int	anni_adam_step(anni_adam *opt, double lr);
/*
** lm_adam_set_offload (lm_adam.c:211-214) with adam_offload_mv (:314-334) and the re-upload of
** gpu_buffers_init (:295-307): with on != 0 the moments leave the device after every step --
** copied into two page-locked host buffers, their device blocks given back -- and the next step
** (or checkpoint call) brings them back first; results do not change.  While they are away d_m
** and d_v are NULL.  The first call with on != 0 moves m and v out of the arena's blocks into
** blocks of their own (gpu_malloc) and everything else into new blocks without room for them, so
** that the memory really is released: device pointers read from the handle before the call are
** stale after it.  The moments leave at once, not only after the next step.  A step with the
** moments offloaded allocates and waits, so it cannot be recorded into a HIP graph.  on == 0
** brings the moments back and keeps them.  0 done, -1 failed (then nothing has moved).
*/
int	anni_adam_set_offload(anni_adam *opt, int on);
/* 1 while m and v are on the device. */
int	anni_adam_mv_on_device(const anni_adam *opt);
/*
** Waits for the stream and fills last_sumsq / last_grad_norm / last_grad_scale / last_skipped /
** last_clipped; prints the reference's messages for that step on stderr (lm_adam.c:479-487):
** "[adam] step T skipped: grad norm G" for a skipped step, and with ANN_GNORM_EVERY=N
** "[adam] step T grad norm G (clipped)" every N steps.
*/
int	anni_adam_sync_stats(anni_adam *opt);

/*
** The optimizer block of the reference's checkpoint (lang/lm_serialize.c:263-331,526-587):
** five int32 {1, epoch, step, t, n} followed by n (m, v) float pairs in slot order, written
** from / read into the arena through an interleave kernel and page-locked staging in chunks
** of 2^21 slots.  bf16 moments widen exactly on export and round to nearest even on import.
** export / import move the pairs of slots [first, first+count) to / from host memory;
** write / read move the whole block through a file descriptor (read restores t).
*/
int	anni_adam_export_mv(anni_adam *opt, int64_t first, int64_t count, float *pairs);
int	anni_adam_import_mv(anni_adam *opt, int64_t first, int64_t count, const float *pairs);
int	anni_adam_write_state(anni_adam *opt, int fd, int epoch, int step);
int	anni_adam_read_state(anni_adam *opt, int fd, int *epoch, int *step);

/* lm_train_step_lr and its setters (lang/lm_train.c:98-124,398-411); kind "none" / "linear" / "cosine". */
void	anni_lr_set_schedule(int warmup_steps, int decay_steps, const char *kind);
void	anni_lr_set_sched_from(int from);
/*
** The live control of the reference's training loop (train_control.lr set through
** lm_train_set_control, lang/train_progress.h:46-56, lm_train.c:93-105): a value > 0 is returned
** by anni_lr_step whatever the schedule says; <= 0 gives the schedule back.
*/
void	anni_lr_set_override(double lr);
double	anni_lr_step(double base_lr, int step);

/* ---- stream plumbing ---------------------------------------------------- */

/*
** The compute stream (a hipStream_t); anni_gpu_set_stream(NULL) restores the library's own.
** anni_adam_step_scaled on a stream under capture is recorded, not run (it allocates nothing and
** waits for nothing); the recorded step keeps its lr, grad_scale, t and gradient flat.  Call
** gpu_stream_sync before the capture begins so that no batched small copy is recorded with it.
*/
void	*anni_gpu_stream(void);
void	anni_gpu_set_stream(void *hip_stream);
/*
** gpu_memcpy_h2d / gpu_memcpy_d2h_async of 64 KiB or less are batched: they reach the stream
** when the next entry point of this library enqueues something (lm_adam.c's per-vector copies
** become two kernels per step that way).  Work that a caller puts on the stream handle ITSELF
** (raw HIP calls, another library) does not pass through an entry point: call this first, it
** puts the pending batch on the stream.  Batched device-to-host copies are complete after any
** synchronising call of this library (gpu_stream_sync, gpu_device_sync, gpu_memcpy_d2h,
** gpu_grad_sumsq, anni_adam_sync_stats, the checkpoint calls), not after a hipStreamSynchronize
** of the caller's own.  ANNI_SMALL_COPY_BATCH=0 switches the batching off.
*/
void	anni_gpu_flush(void);

/* Name and architecture of the current device and the HIP driver version: what the reference's bench row records from nvidia-smi (lang/lm_bench.c:287-316). */
int	anni_gpu_device_info(char *name, size_t cap, int *driver_version);

/* ---- producers either side of the step (device utilities) ---------------- */

/* dst = bf16(src) round to nearest even (num/gpu_cuda.cu:1497-1513). */
int	anni_f32_to_bf16(void *d_dst, const float *d_src, int64_t n);
/*
** Per-tensor FP8 quantisation by the reference's convention (num/gpu_cuda.cu:796-851,927-938):
** scale = max(amax/448, 1e-12) (amax <= 0 or non-finite: 1e-8/448), q = satfinite_e4m3(x * (1/scale)).
** d_scale[0] receives the scale; d_src is only read.
*/
int	anni_fp8_quantize(void *d_q, float *d_scale, const float *d_src, int64_t n);
/*
** Bias / LayerNorm gradients straight into the gradient flat: d_acc[c] += column sums of the
** row-major rows x cols matrix d_x (d_y given: of the element-wise float product d_x * d_y), added
** one row after the other in float exactly as the reference's host loops do (lang/ffn.c:301-305,
** 358-362: db += rows of dout / dh; lang/layernorm.c:368-372: dbeta += dy, dgamma += dy * x_hat),
** so the result has the host path's bits and is the same on every run.  Stands where the
** reference's device path keeps per-bias accumulators that it flushes to host vectors before the
** optimizer gathers them again (gpu_mat_col_sum_add, num/gpu.h:195-199, gpu_cuda.cu:3131-3167):
** with d_acc = (float *)opt->d_grad + anni_adam_tensor_offset(opt, i) nothing leaves the device.
** rows == 0 leaves d_acc alone; cols up to 2^24.
*/
int	anni_colsum_add(float *d_acc, const float *d_x, const float *d_y, int64_t rows, int cols);
/*
** Up to 16 such sums at once (the bias and LayerNorm gradients of a block, say): a sum narrower
** than ~4000 columns occupies only cols / 64 of the 256 compute units, so sums launched one by
** one leave most of the chip idle; here the plain sums share one launch and the product sums
** another.  The jobs must not alias each other's d_acc.  Same results as one call per job.
*/
typedef struct anni_colsum {
	float		*d_acc;
	const float	*d_x;
	const float	*d_y;	/* NULL: plain column sums */
	int64_t		rows;
	int		cols;
} anni_colsum;
int	anni_colsum_add_batch(const anni_colsum *jobs, int n_jobs);

#ifdef __cplusplus
}
#endif
#endif

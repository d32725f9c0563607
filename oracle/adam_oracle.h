/*
** CPU oracle for the AnnI optimizer step.  TEST INFRASTRUCTURE ONLY.
**
** This is a plain-C restatement of the reference's host optimizer path; it is
** the checker the HIP kernels are compared with and the CPU leg of the bench.
** Nothing that ships (the HIP backend, the arena, the Python package) links,
** loads or calls it: only tests, the smoke check and the bench's cpu_baseline
** leg do.
**
** What each function follows in the reference:
**   oracle_lr                      lang/lm_train.c:98-124  (lm_train_step_lr)
**   oracle_adam_step_scaled        lang/lm_adam.c:522-533  (early-outs, t++)
**                                  lang/lm_adam.c:571-598  (clip + update math)
**                                  lang/lm_adam.c:474-483  (non-finite skip; the
**                                  reference has it on its device path only)
**   oracle_bf16_rne                num/gpu_cuda.cu:8578,1505 (__float2bfloat16 = RNE)
**   oracle_fp8_scale_from_amax     num/gpu_cuda.cu:927-938 (amax_to_scale_kernel)
**   oracle_fp8_quantize            num/gpu_cuda.cu:826-851 (x * (1/scale), satfinite E4M3)
**   oracle_colsum_add              lang/ffn.c:301-305,358-362, lang/layernorm.c:368-372
**                                  (bias / LayerNorm gradients as serial float column sums)
**
** Pinned by: the reference's compiled lm_adam_step_scaled (oracle/_ref, bit for
** bit on p/m/v), the golden vectors it wrote (the .npz files under tests/golden: oracle_adam_step_scaled
** and oracle_adam_step_slots, bit for bit), the reference's own LR known answers
** (tests/test_ann.c:866-879), closed forms (t=1, constant gradient, zero gradient), and
** brute-force exact sums; oracle_colsum_add by the reference's compiled layernorm_backward
** (dgamma / dbeta, bit for bit) and by inputs whose sum depends on the order.  The VALUE of
** the FP8 norm (oracle_sumsq's factored form) is pinned against the direct form
** SUM (float(decode(q) * scale_t) * grad_scale)^2 summed exactly (<= 1e-7 relative, multi-tensor
** lists) and by invariants a wrong factoring fails (a tensor's share scales with the square
** of its own scale only, one element gives the closed form, permutations inside a tensor
** change no bit, a NaN code gives NaN).
** PARITY UNPINNED by the reference (no implementation exists there, the oracle defines the
** rounding points): bf16-stored m/v, bf16 gradients, fp8-E4M3 gradients with a per-tensor
** scale, weight decay on selected tensors only, and the non-finite skip on the CPU path.
*/
#ifndef ADAM_ORACLE_H__
#define ADAM_ORACLE_H__

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage type of a flat array handed to the oracle. */
#define ORACLE_F32	0
#define ORACLE_BF16	1	/* uint16_t, upper half of an IEEE float */
#define ORACLE_FP8	2	/* uint8_t, OCP E4M3 (finite-only, 0x7F/0xFF = NaN) */

/* One tensor of the flat: elements [off, off+n). */
typedef struct oracle_seg {
	int64_t	off;
	int64_t	n;
	int	wd_on;		/* decoupled weight decay applies to this tensor */
	float	gscale;		/* fp8 gradients: per-tensor dequant scale (else unused) */
} oracle_seg;

/* Mirrors the fields of the reference's lm_adam that the step reads (lang/lm_adam.h:30-54). */
typedef struct oracle_adam {
	int64_t	n;
	int	t;
	double	beta1;
	double	beta2;
	double	eps;
	double	weight_decay;
	double	grad_clip;
	int	skip_nonfinite;	/* 1: a non-finite norm skips the update (lm_adam.c:474-483) */
	int	grad_type;	/* ORACLE_F32 / ORACLE_BF16 / ORACLE_FP8 */
	int	moment_type;	/* ORACLE_F32 / ORACLE_BF16 */
	int	norm_threads;	/* 0/1: serial norm in slot order (the reference); >1: ordered partials */
	/* outputs of the last step */
	double	last_sumsq;
	double	last_grad_norm;
	double	last_grad_scale;	/* grad_scale after the clip factor */
	int	last_clipped;
	int	last_skipped;
} oracle_adam;

void	oracle_adam_defaults(oracle_adam *o, int64_t n);

/*
** One optimizer step over the flat.  p is float[n]; g, m, v are typed by
** grad_type / moment_type; twin (may be NULL) receives RNE bf16 of the final p;
** segs == NULL means "one tensor, decay everywhere" (the reference's behaviour).
** sumsq_override (may be NULL) replaces the oracle's own sum of squares so the
** update can be compared bit for bit under a norm computed elsewhere.
** Returns 0 when an update (or a skip) happened, 1 for the lr <= 0 early-out.
*/
int	oracle_adam_step_scaled(oracle_adam *o, float *p, void *g, void *m, void *v,
		uint16_t *twin, const oracle_seg *segs, int nsegs, double lr,
		double grad_scale, const double *sumsq_override, int threads);

/*
** Sum over the flat of (g*grad_scale)^2 as the clip block computes it.  FP8 gradients use the
** factored form SUM_t (scale_t*grad_scale)^2 * SUM_i decode(q_i)^2 (within 1e-7 relative of the
** direct form the update consumes; tests/test_oracle.py).
*/
double	oracle_sumsq(const void *g, int grad_type, int64_t n, const oracle_seg *segs,
		int nsegs, double grad_scale, int threads);

/* lm_train_step_lr with its three globals passed explicitly. kind: 0 none, 1 linear, 2 cosine. */
double	oracle_lr(double base_lr, int step, int warmup, int decay_steps, int kind,
		int sched_from);

uint16_t	oracle_bf16_rne(float x);
float	oracle_bf16_widen(uint16_t h);
float	oracle_fp8_decode(uint8_t q);
uint8_t	oracle_fp8_encode(float x);	/* RNE, saturate to +-448, NaN -> 0x7F | sign */
float	oracle_fp8_scale_from_amax(float amax);
/* q[i] = encode(x[i] * (1/scale)) ; returns the scale used (from the tensor's amax). */
float	oracle_fp8_quantize(uint8_t *q, const float *x, int64_t n);
void	oracle_f32_to_bf16(uint16_t *dst, const float *src, int64_t n);

/*
** The reference's host loop as it is laid out in memory there: 24-byte slots
** {param*, grad*, m, v} walked serially (lang/lm_adam.h:9-14, lm_adam.c:571-598).
** Used only as the single-thread CPU timing leg; results equal the SoA path.
*/
typedef struct oracle_slot {
	float	*param;
	float	*grad;
	float	m;
	float	v;
} oracle_slot;
void	oracle_adam_step_slots(oracle_slot *slots, int64_t n, int t, double beta1,
		double beta2, double eps, double weight_decay, double grad_clip,
		double lr, double grad_scale);

/* acc[j] += column sums of x (y != NULL: of x * y), rows x cols row-major, the host loops' order. */
void	oracle_colsum_add(float *acc, const float *x, const float *y, int64_t rows, int cols);

/*
** Comparison helpers of the full-size tests: byte equality, and a against b with
** out[0] = max |a-b| / max(|b|, rms(b)), out[1] = number of elements with |a-b| > tol * |b|,
** out[2] = the largest |b| among those.  type ORACLE_F32 or ORACLE_BF16 (bit patterns, widened).
*/
int	oracle_same_bytes(const void *a, const void *b, int64_t nbytes);
void	oracle_compare(const void *a, const void *b, int type, int64_t n, double tol, double *out);

int	oracle_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif

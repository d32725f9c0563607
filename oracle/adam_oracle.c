/*
** CPU oracle for the AnnI optimizer step.  TEST INFRASTRUCTURE ONLY: see
** adam_oracle.h for what it is allowed to be used for and what pins it.
**
** Build: gcc -O2 -std=c99 -fopenmp (no -march, no FMA, no fast-math) -- the
** reference's own flags (Makefile:21), so every double operation below rounds
** exactly where the reference's does.
*/
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include "adam_oracle.h"

#define ALWAYS_INLINE static inline __attribute__((always_inline))

/* ---- storage codecs -------------------------------------------------- */

static uint32_t f32_bits(float x)
{
	uint32_t u;

	memcpy(&u, &x, 4);
	return u;
}

static float bits_f32(uint32_t u)
{
	float x;

	memcpy(&x, &u, 4);
	return x;
}

/* Round-to-nearest-even float -> bfloat16 (num/gpu_cuda.cu:8578 stores __float2bfloat16(p)). */
uint16_t oracle_bf16_rne(float x)
{
	uint32_t u = f32_bits(x);

	if ((u & 0x7fffffffu) > 0x7f800000u)	/* NaN: keep it a NaN */
		return (uint16_t)((u >> 16) | 0x0040u);
	u += 0x7fffu + ((u >> 16) & 1u);
	return (uint16_t)(u >> 16);
}

float oracle_bf16_widen(uint16_t h)
{
	return bits_f32((uint32_t)h << 16);
}

/* OCP E4M3 (finite + NaN, no infinities): 1 sign, 4 exponent (bias 7), 3 mantissa. */
float oracle_fp8_decode(uint8_t q)
{
	int e = (q >> 3) & 15;
	int f = q & 7;
	float a;

	if (e == 15 && f == 7)
		return bits_f32((q & 0x80) ? 0xffc00000u : 0x7fc00000u);
	if (e == 0)
		a = ldexpf((float)f, -9);		/* subnormal: f/8 * 2^-6 */
	else
		a = ldexpf((float)(8 + f), e - 10);	/* (1 + f/8) * 2^(e-7) */
	return (q & 0x80) ? -a : a;
}

/* RNE with saturation to +-448 (what __NV_SATFINITE E4M3 does, gpu_cuda.cu:845-846). */
uint8_t oracle_fp8_encode(float x)
{
	uint8_t s = (f32_bits(x) & 0x80000000u) ? 0x80 : 0;
	float a = fabsf(x);
	int e;
	int q;

	if (a != a)
		return (uint8_t)(s | 0x7f);
	if (a >= 448.0f)
		return (uint8_t)(s | 0x7e);
	if (a < 0.015625f) {			/* below 2^-6: subnormal grid, step 2^-9 */
		q = (int)rintf(ldexpf(a, 9));	/* 0..8; 8 lands on the first normal */
		return (uint8_t)(s | q);
	}
	(void)frexpf(a, &e);			/* a = f * 2^e, f in [0.5,1) */
	e -= 1;					/* a = 1.xxx * 2^e */
	q = (int)rintf(ldexpf(a, 3 - e));	/* 8..16 */
	if (q == 16) {
		q = 8;
		e += 1;
	}
	return (uint8_t)(s | ((e + 7) << 3) | (q - 8));
}

float oracle_fp8_scale_from_amax(float amax)
{
	float a = amax;

	if (!(a > 0.0f) || !isfinite(a))
		a = 1e-8f;
	a = a / 448.0f;
	if (a < 1e-12f)
		a = 1e-12f;
	return a;
}

float oracle_fp8_quantize(uint8_t *q, const float *x, int64_t n)
{
	float amax = 0.0f;
	float scale;
	float inv;
	int64_t i;

	for (i = 0; i < n; i++)
		amax = fmaxf(amax, fabsf(x[i]));	/* fmaxf drops NaNs, as the kernel's does */
	scale = oracle_fp8_scale_from_amax(amax);
	inv = 1.0f / scale;
	for (i = 0; i < n; i++)
		q[i] = oracle_fp8_encode(x[i] * inv);
	return scale;
}

void oracle_f32_to_bf16(uint16_t *dst, const float *src, int64_t n)
{
	int64_t i;

#pragma omp parallel for if (n > 1000000)
	for (i = 0; i < n; i++)
		dst[i] = oracle_bf16_rne(src[i]);
}

/* ---- comparison helpers of the full-size tests (plain arithmetic, nothing of the reference) ---- */

/* 1 when the two byte ranges are equal. */
int oracle_same_bytes(const void *a, const void *b, int64_t nbytes)
{
	const int64_t chunk = (int64_t)1 << 24;
	const int64_t n_chunks = (nbytes + chunk - 1) / chunk;
	int same = 1;
	int64_t c;

#pragma omp parallel for reduction(&& : same) if (n_chunks > 4)
	for (c = 0; c < n_chunks; c++) {
		const int64_t at = c * chunk;
		const int64_t len = nbytes - at < chunk ? nbytes - at : chunk;

		same = same && memcmp((const char *)a + at, (const char *)b + at, (size_t)len) == 0;
	}
	return same;
}

static double cmp_value(const void *x, int type, int64_t i)
{
	return type == ORACLE_BF16 ? (double)oracle_bf16_widen(((const uint16_t *)x)[i])
	    : (double)((const float *)x)[i];
}

/*
** a against b (float arrays, or bf16 bit patterns that are widened): out[0] = max over i of
** |a-b| / max(|b|, rms(b)); out[1] = how many elements have |a-b| > tol * |b|; out[2] = the largest
** |b| among those (0 when there is none).
*/
void oracle_compare(const void *a, const void *b, int type, int64_t n, double tol, double *out)
{
	double ss = 0.0, worst = 0.0, biggest = 0.0, floor_;
	int64_t count = 0;
	int64_t i;

#pragma omp parallel for reduction(+ : ss) if (n > 1000000)
	for (i = 0; i < n; i++) {
		const double y = cmp_value(b, type, i);

		ss += y * y;
	}
	floor_ = (n > 0 ? sqrt(ss / (double)n) : 0.0) + 1e-300;
#pragma omp parallel for reduction(max : worst, biggest) reduction(+ : count) if (n > 1000000)
	for (i = 0; i < n; i++) {
		const double x = cmp_value(a, type, i);
		const double y = cmp_value(b, type, i);
		const double d = fabs(x - y);
		const double ay = fabs(y);
		const double r = d / (ay > floor_ ? ay : floor_);

		if (r > worst || r != r)
			worst = r != r ? INFINITY : r;
		if (d > tol * ay || d != d) {
			count++;
			if (ay > biggest)
				biggest = ay;
		}
	}
	out[0] = worst;
	out[1] = (double)count;
	out[2] = biggest;
}

/* ---- learning-rate schedule (lang/lm_train.c:98-124) ------------------ */

double oracle_lr(double base_lr, int step, int warmup, int decay_steps, int kind,
	int sched_from)
{
	double q;
	int u;

	if (warmup < 0)
		warmup = 0;		/* lm_train_set_lr_schedule clamps (lm_train.c:398-401) */
	if (decay_steps < 0)
		decay_steps = 0;
	if (sched_from < 0)
		sched_from = 0;
	step -= sched_from;
	if (step < 0)
		step = 0;
	if (warmup > 0 && step < warmup)
		return base_lr * ((double)step + 1.0) / (double)warmup;
	if (decay_steps <= 0 || kind == 0)
		return base_lr;
	u = step - warmup;
	if (u < 0)
		u = 0;
	if (u > decay_steps)
		u = decay_steps;
	q = (double)u / (double)decay_steps;
	if (kind == 1)
		return base_lr * (1.0 - q);
	return base_lr * 0.5 * (1.0 + cos(3.14159265358979323846 * q));
}

/* ---- the step -------------------------------------------------------- */

void oracle_adam_defaults(oracle_adam *o, int64_t n)
{
	memset(o, 0, sizeof(*o));
	o->n = n;
	o->beta1 = 0.9;		/* lang/lm_adam.c:110-115 */
	o->beta2 = 0.999;
	o->eps = 1e-8;
	o->grad_type = ORACLE_F32;
	o->moment_type = ORACLE_F32;
}

int oracle_max_threads(void)
{
#ifdef _OPENMP
	return omp_get_max_threads();
#else
	return 1;
#endif
}

/* Gradient element i as the float the update sees (fp8: decode * scale in float). */
ALWAYS_INLINE float load_grad(const void *g, const int gt, int64_t i, float gscale)
{
	if (gt == ORACLE_F32)
		return ((const float *)g)[i];
	if (gt == ORACLE_BF16)
		return oracle_bf16_widen(((const uint16_t *)g)[i]);
	return oracle_fp8_decode(((const uint8_t *)g)[i]) * gscale;
}

ALWAYS_INLINE void zero_grad(void *g, const int gt, int64_t i)
{
	if (gt == ORACLE_F32)
		((float *)g)[i] = 0.0f;
	else if (gt == ORACLE_BF16)
		((uint16_t *)g)[i] = 0;
	else
		((uint8_t *)g)[i] = 0;
}

/* Continues the running sum `acc` over elements [lo, hi) (lm_adam.c:577-580). */
ALWAYS_INLINE double sumsq_range(double acc, const void *g, const int gt, int64_t lo,
	int64_t hi, float gscale, double grad_scale)
{
	double x;
	int64_t i;

	for (i = lo; i < hi; i++) {
		x = load_grad(g, gt, i, gscale) * grad_scale;
		acc += x * x;
	}
	return acc;
}

static double sumsq_dispatch(double acc, const void *g, int gt, int64_t lo, int64_t hi,
	float gscale, double grad_scale)
{
	if (gt == ORACLE_F32)
		return sumsq_range(acc, g, ORACLE_F32, lo, hi, gscale, grad_scale);
	if (gt == ORACLE_BF16)
		return sumsq_range(acc, g, ORACLE_BF16, lo, hi, gscale, grad_scale);
	return sumsq_range(acc, g, ORACLE_FP8, lo, hi, gscale, grad_scale);
}

double oracle_sumsq(const void *g, int grad_type, int64_t n, const oracle_seg *segs,
	int nsegs, double grad_scale, int threads)
{
	oracle_seg whole;
	double total = 0.0;
	int s;

	if (!segs) {
		whole.off = 0;
		whole.n = n;
		whole.wd_on = 1;
		whole.gscale = 1.0f;
		segs = &whole;
		nsegs = 1;
	}
	if (grad_type == ORACLE_FP8) {
		/*
		** FP8 gradients (no counterpart in the reference): the norm is defined in its
		** factored form, SUM_t (scale_t * grad_scale)^2 * SUM_i decode(q_i)^2.  The square of
		** an E4M3 value is exact in float and the inner sum is exact in double (multiples of
		** 2^-18 below 2^53), so its order does not matter; only the per-tensor products round.
		*/
		for (s = 0; s < nsegs; s++) {
			const uint8_t *q = (const uint8_t *)g + segs[s].off;
			const double sc = (double)segs[s].gscale * grad_scale;
			double inner = 0.0;
			int64_t i;

#pragma omp parallel for num_threads(threads > 1 ? threads : 1) reduction(+:inner) \
    if (threads > 1 && segs[s].n > 65536)
			for (i = 0; i < segs[s].n; i++) {
				const float d = oracle_fp8_decode(q[i]);

				inner += (double)(d * d);
			}
			total += (sc * sc) * inner;
		}
		return total;
	}
	if (threads <= 1) {
		/* One accumulator carried through every tensor in slot order: the reference's loop. */
		for (s = 0; s < nsegs; s++)
			total = sumsq_dispatch(total, g, grad_type, segs[s].off,
			    segs[s].off + segs[s].n, segs[s].gscale, grad_scale);
		return total;
	}
	/* Ordered partials: each tensor cut into `threads` runs, summed in run order. */
	for (s = 0; s < nsegs; s++) {
		double *part = calloc((size_t)threads, sizeof(double));
		int64_t per = (segs[s].n + threads - 1) / threads;
		int k;

		if (!part)
			return NAN;
#pragma omp parallel for num_threads(threads) schedule(static, 1)
		for (k = 0; k < threads; k++) {
			int64_t lo = segs[s].off + (int64_t)k * per;
			int64_t hi = lo + per;

			if (hi > segs[s].off + segs[s].n)
				hi = segs[s].off + segs[s].n;
			if (lo < hi)
				part[k] = sumsq_dispatch(0.0, g, grad_type, lo, hi,
				    segs[s].gscale, grad_scale);
		}
		for (k = 0; k < threads; k++)
			total += part[k];
		free(part);
	}
	return total;
}

/*
** Elements [lo, hi) of one tensor.  GT/MT are literals at every call site so
** the loads fold away.  Rounding points (-> float) are the stores to m32, v32
** and the two stores to p, exactly as lang/lm_adam.c:588-596.
*/
ALWAYS_INLINE void update_range(float *p, void *g, void *m, void *v, uint16_t *twin,
	const int GT, const int MT, int64_t lo, int64_t hi, float gscale, int wd_on,
	double beta1, double beta2, double eps, double wd, double bc1, double bc2,
	double lr, double grad_scale)
{
	int64_t i;

	for (i = lo; i < hi; i++) {
		double x = load_grad(g, GT, i, gscale) * grad_scale;
		float m32;
		float v32;
		double mhat;
		double vhat;

		if (MT == ORACLE_F32) {
			m32 = ((float *)m)[i];
			v32 = ((float *)v)[i];
		} else {
			m32 = oracle_bf16_widen(((uint16_t *)m)[i]);
			v32 = oracle_bf16_widen(((uint16_t *)v)[i]);
		}
		m32 = beta1 * m32 + (1.0 - beta1) * x;
		v32 = beta2 * v32 + (1.0 - beta2) * x * x;
		mhat = m32 / bc1;
		vhat = v32 / bc2;
		p[i] -= lr * mhat / (sqrt(vhat) + eps);
		if (wd_on && wd > 0.0)
			p[i] -= lr * wd * p[i];
		if (MT == ORACLE_F32) {
			((float *)m)[i] = m32;
			((float *)v)[i] = v32;
		} else {
			((uint16_t *)m)[i] = oracle_bf16_rne(m32);
			((uint16_t *)v)[i] = oracle_bf16_rne(v32);
		}
		zero_grad(g, GT, i);
		if (twin)
			twin[i] = oracle_bf16_rne(p[i]);
	}
}

#define UPDATE_CASE(GTV, MTV) \
	update_range(p, g, m, v, twin, GTV, MTV, lo, hi, gscale, wd_on, beta1, beta2, \
	    eps, wd, bc1, bc2, lr, grad_scale)

static void update_dispatch(float *p, void *g, void *m, void *v, uint16_t *twin, int gt,
	int mt, int64_t lo, int64_t hi, float gscale, int wd_on, double beta1, double beta2,
	double eps, double wd, double bc1, double bc2, double lr, double grad_scale)
{
	if (mt == ORACLE_F32) {
		if (gt == ORACLE_F32)
			UPDATE_CASE(ORACLE_F32, ORACLE_F32);
		else if (gt == ORACLE_BF16)
			UPDATE_CASE(ORACLE_BF16, ORACLE_F32);
		else
			UPDATE_CASE(ORACLE_FP8, ORACLE_F32);
	} else {
		if (gt == ORACLE_F32)
			UPDATE_CASE(ORACLE_F32, ORACLE_BF16);
		else if (gt == ORACLE_BF16)
			UPDATE_CASE(ORACLE_BF16, ORACLE_BF16);
		else
			UPDATE_CASE(ORACLE_FP8, ORACLE_BF16);
	}
}

int oracle_adam_step_scaled(oracle_adam *o, float *p, void *g, void *m, void *v,
	uint16_t *twin, const oracle_seg *segs, int nsegs, double lr, double grad_scale,
	const double *sumsq_override, int threads)
{
	oracle_seg whole;
	double bc1;
	double bc2;
	int s;

	if (!o || lr <= 0.0)
		return 1;			/* lm_adam.c:531-532: t is NOT advanced */
	o->t++;					/* lm_adam.c:533 */
	if (!segs) {
		whole.off = 0;
		whole.n = o->n;
		whole.wd_on = 1;
		whole.gscale = 1.0f;
		segs = &whole;
		nsegs = 1;
	}
	if (threads < 1)
		threads = 1;
	bc1 = 1.0 - pow(o->beta1, (double)o->t);	/* lm_adam.c:571-572 */
	bc2 = 1.0 - pow(o->beta2, (double)o->t);
	o->last_clipped = 0;
	o->last_skipped = 0;
	if (o->grad_clip > 0.0 || o->skip_nonfinite) {
		double ss;
		double norm;

		ss = sumsq_override ? *sumsq_override
		    : oracle_sumsq(g, o->grad_type, o->n, segs, nsegs, grad_scale,
		    o->norm_threads > 1 ? o->norm_threads : 1);
		norm = sqrt(ss);			/* lm_adam.c:581 */
		o->last_sumsq = ss;
		o->last_grad_norm = norm;
		if (o->skip_nonfinite && !isfinite(norm)) {
			/* lm_adam.c:474-483: keep p/m/v, zero the gradients, t stays advanced */
			for (s = 0; s < nsegs; s++) {
				size_t es = o->grad_type == ORACLE_F32 ? 4
				    : o->grad_type == ORACLE_BF16 ? 2 : 1;

				memset((char *)g + (size_t)segs[s].off * es, 0,
				    (size_t)segs[s].n * es);
			}
			o->last_skipped = 1;
			o->last_grad_scale = grad_scale;
			return 0;
		}
		if (o->grad_clip > 0.0 && norm > o->grad_clip) {	/* lm_adam.c:582-585 */
			grad_scale *= o->grad_clip / (norm + 1e-12);
			o->last_clipped = 1;
		}
	}
	o->last_grad_scale = grad_scale;
	for (s = 0; s < nsegs; s++) {
		int64_t lo0 = segs[s].off;
		int64_t hi0 = lo0 + segs[s].n;

		if (threads == 1 || segs[s].n < 65536) {
			update_dispatch(p, g, m, v, twin, o->grad_type, o->moment_type, lo0, hi0,
			    segs[s].gscale, segs[s].wd_on, o->beta1, o->beta2, o->eps,
			    o->weight_decay, bc1, bc2, lr, grad_scale);
		} else {
			int64_t per = (segs[s].n + threads - 1) / threads;
			int k;

#pragma omp parallel for num_threads(threads) schedule(static, 1)
			for (k = 0; k < threads; k++) {
				int64_t lo = lo0 + (int64_t)k * per;
				int64_t hi = lo + per > hi0 ? hi0 : lo + per;

				if (lo < hi)
					update_dispatch(p, g, m, v, twin, o->grad_type,
					    o->moment_type, lo, hi, segs[s].gscale,
					    segs[s].wd_on, o->beta1, o->beta2, o->eps,
					    o->weight_decay, bc1, bc2, lr, grad_scale);
			}
		}
	}
	return 0;
}

/* The reference's memory layout and loop, for the single-thread timing leg. */
void oracle_adam_step_slots(oracle_slot *slots, int64_t n, int t, double beta1,
	double beta2, double eps, double weight_decay, double grad_clip, double lr,
	double grad_scale)
{
	double bc1 = 1.0 - pow(beta1, (double)t);
	double bc2 = 1.0 - pow(beta2, (double)t);
	double g;
	double mhat;
	double vhat;
	int64_t i;

	if (grad_clip > 0.0) {
		double norm = 0.0;

		for (i = 0; i < n; i++) {
			g = *slots[i].grad * grad_scale;
			norm += g * g;
		}
		norm = sqrt(norm);
		if (norm > grad_clip)
			grad_scale *= grad_clip / (norm + 1e-12);
	}
	for (i = 0; i < n; i++) {
		g = *slots[i].grad * grad_scale;
		slots[i].m = beta1 * slots[i].m + (1.0 - beta1) * g;
		slots[i].v = beta2 * slots[i].v + (1.0 - beta2) * g * g;
		mhat = slots[i].m / bc1;
		vhat = slots[i].v / bc2;
		*slots[i].param -= lr * mhat / (sqrt(vhat) + eps);
		if (weight_decay > 0.0)
			*slots[i].param -= lr * weight_decay * *slots[i].param;
		*slots[i].grad = 0.0f;
	}
}

/*
** Column sums in the order of the reference's host loops (lang/ffn.c:301-305,358-362:
** db[j] += x[t * cols + j]; lang/layernorm.c:368-372: dbeta[j] += dy, dgamma[j] += dy * x_hat),
** rows outermost, everything in float: acc[j] = (acc[j] + t_0) + t_1 ... with t the element or the
** float product of the two elements.
*/
void oracle_colsum_add(float *acc, const float *x, const float *y, int64_t rows, int cols)
{
	int64_t t;
	int j;

	for (t = 0; t < rows; t++) {
		for (j = 0; j < cols; j++) {
			if (y)
				acc[j] += x[t * cols + j] * y[t * cols + j];
			else
				acc[j] += x[t * cols + j];
		}
	}
}

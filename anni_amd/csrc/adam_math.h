/*
** Per-element arithmetic of the AdamW step, shared by every kernel variant.
**
** The parity target is the reference's HOST loop (lang/lm_adam.c:587-598), which
** computes in double and stores float after each of m, v, the Adam step on p and
** the decay on p.  The device code below performs the same IEEE-754 double
** operations in the same order (this library is compiled with -ffp-contract=off,
** so no multiply-add is fused), which makes p, m and v bit-identical to the host
** loop whenever the effective gradient scale is the same double.
*/
#ifndef ANNI_ADAM_MATH_H__
#define ANNI_ADAM_MATH_H__

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace anni {

/* Scalars of one step, computed on the host in double as lm_adam.c:571-572 does. */
struct StepConsts {
	double	beta1;
	double	omb1;	/* 1.0 - beta1 */
	double	beta2;
	double	omb2;	/* 1.0 - beta2 */
	double	eps;
	double	bc1;	/* 1 - beta1^t */
	double	bc2;	/* 1 - beta2^t */
	double	lr;
	double	lr_wd;	/* lr * weight_decay (lm_adam.c:595 multiplies these first) */
	int	decay_on;	/* weight_decay > 0 (lm_adam.c:594); per-tensor flags select where */
	double	rbc1;	/* 1.0 / bc1 and 1.0 / bc2, correctly rounded (host division) */
	double	rbc2;
};

/* New p, m, v of one element. */
struct Elem {
	float	p;
	float	m;
	float	v;
};

/*
** a / b for a step constant b > 0 whose correctly rounded reciprocal rb the host supplies:
** q = a*rb, then one exact residual a - b*q folded back.  The result is a/b rounded to nearest
** unless a/b lies within ~2^-52 ulp of a rounding boundary (then it may be the other neighbour).
** Compared on the host with the IEEE quotient for b = 1 - beta^t, beta in {0.9, 0.95, 0.999},
** t = 1..10000, over 10^8 float-valued numerators from every binary exponent: no difference
** (tests/c/div_by_const_test.c).  The residual of a zero is +0 whatever the zero's sign, so the
** sign is put back: -0 / b is -0.  Not for an infinite a: the residual would be inf - inf
** (adam_elem sends those to the IEEE division).  Used only where the update is bound by
** arithmetic (narrow storage types); the all-f32 mode keeps the IEEE division.
*/
__device__ __forceinline__ double div_by_const(double a, double b, double rb)
{
	const double q = a * rb;

	return __builtin_copysign(__builtin_fma(__builtin_fma(-b, q, a), rb, q), a);
}

/*
** g is the gradient element as a float; gs the effective gradient scale.
** Rounding points: m, v (float), p after the step, p after the decay.
*/
template <bool FASTDIV>
__device__ __forceinline__ Elem adam_elem(float p, float g, float m, float v, double gs,
	const StepConsts &c, bool decay)
{
	Elem r;
	const double x = (double)g * gs;
	double mhat, vhat;

	r.m = (float)(c.beta1 * (double)m + c.omb1 * x);
	r.v = (float)(c.beta2 * (double)v + (c.omb2 * x) * x);
	if (FASTDIV) {
		mhat = div_by_const((double)r.m, c.bc1, c.rbc1);
		vhat = div_by_const((double)r.v, c.bc2, c.rbc2);
		/*
		** A moment that overflowed to infinity (or is NaN): the host loop divides it all the same
		** -- inf / bc2 = inf, sqrt(inf) = inf, the step is 0 -- while the residual above gives
		** NaN.  |m| + v is finite exactly when both are (or spuriously not, next to the largest
		** float: harmless); the wavefront leaves the fast path only when a lane needs to.
		*/
		const bool odd = !__builtin_isfinite(__builtin_fabsf(r.m) + r.v);

		if (__builtin_expect(__builtin_amdgcn_ballot_w64(odd) != 0, 0)) {
			float fm = r.m, fv = r.v;

			/* keeps the two divisions inside this block (they would be hoisted and selected otherwise) */
			asm volatile("" : "+v"(fm), "+v"(fv));
			if (odd) {
				mhat = (double)fm / c.bc1;
				vhat = (double)fv / c.bc2;
			}
		}
	} else {
		mhat = (double)r.m / c.bc1;
		vhat = (double)r.v / c.bc2;
	}
	r.p = (float)((double)p - (c.lr * mhat) / (sqrt(vhat) + c.eps));
	if (decay)
		r.p = (float)((double)r.p - c.lr_wd * (double)r.p);
	return r;
}

/* float -> bfloat16 bits, round to nearest even; NaN stays NaN (quiet bit set). */
__device__ __forceinline__ uint32_t bf16_rne(float x)
{
	uint32_t u = __float_as_uint(x);

	if ((u & 0x7fffffffu) > 0x7f800000u)
		return (u >> 16) | 0x0040u;
	u += 0x7fffu + ((u >> 16) & 1u);
	return u >> 16;
}

/*
** Two floats -> two bfloat16 in one word (x in the low half) with the gfx950 conversion
** instruction: round to nearest even, NaN quieted; the same bits as bf16_rne for every float
** (checked over all 2^32 patterns).
*/
typedef float f32x2_cv __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_cv __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_rne2(float x, float y)
{
	const f32x2_cv v = {x, y};

	return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_cv));
}

__device__ __forceinline__ float bf16_widen(uint32_t h)
{
	return __uint_as_float(h << 16);
}

/* OCP E4M3 byte -> float (exact): bias 7, subnormals f/8 * 2^-6, S.1111.111 = NaN, no infinities. */
__device__ __forceinline__ float fp8_e4m3_decode(uint32_t q)
{
	const uint32_t s = (q & 0x80u) << 24;
	const uint32_t e = (q >> 3) & 15u;
	const uint32_t f = q & 7u;
	uint32_t bits;

	if (e == 0u)
		bits = __float_as_uint((float)f * 0x1p-9f);
	else if (e == 15u && f == 7u)
		bits = 0x7fc00000u;
	else
		bits = ((e + 120u) << 23) | (f << 20);
	return __uint_as_float(s | bits);
}

/*
** Two / four OCP E4M3 bytes of a word -> floats with the gfx950 conversion instruction
** (exact, same values as fp8_e4m3_decode; checked against the table for all 256 codes).
*/
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ f32x2_t fp8_e4m3_decode2(uint32_t w, bool high)
{
	return high ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true)
	    : __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
}

/* float -> OCP E4M3 byte: round to nearest even, saturate to +-448, NaN -> S.1111.111. */
__device__ __forceinline__ uint32_t fp8_e4m3_encode(float x)
{
	const uint32_t u = __float_as_uint(x);
	const uint32_t s = (u >> 24) & 0x80u;
	const float a = __uint_as_float(u & 0x7fffffffu);
	int e;
	int q;

	if (a != a)
		return s | 0x7fu;
	if (a >= 448.0f)
		return s | 0x7eu;
	if (a < 0.015625f)
		return s | (uint32_t)(int)rintf(a * 512.0f);	/* subnormal grid, step 2^-9 */
	e = (int)((u >> 23) & 0xffu) - 127;			/* a = 1.xxx * 2^e, e in [-6, 8] */
	q = (int)rintf(ldexpf(a, 3 - e));			/* 8..16 */
	if (q == 16) {
		q = 8;
		e += 1;
	}
	return s | (uint32_t)((e + 7) << 3) | (uint32_t)(q - 8);
}

/*
** Four floats -> four OCP E4M3 bytes (x in the low byte) with the gfx950 conversion instruction:
** round to nearest even on the format's grid, subnormals included.  The instruction alone would
** turn an overflow into NaN, so the values are first clamped to +-448 (an infinity saturates);
** a NaN input is patched to S.1111.111 afterwards, whatever the clamp made of it.  Same bytes as
** fp8_e4m3_encode on every input (checked on every rounding boundary of the format).
*/
__device__ __forceinline__ uint32_t fp8_e4m3_encode4(float x, float y, float z, float w)
{
	const float lim = 448.0f;
	int r = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(x, -lim, lim),
	    __builtin_amdgcn_fmed3f(y, -lim, lim), 0, false);
	uint32_t out;

	r = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(z, -lim, lim),
	    __builtin_amdgcn_fmed3f(w, -lim, lim), r, true);
	out = (uint32_t)r;
	if (x != x || y != y || z != z || w != w) {
		if (x != x)
			out = (out & 0xffffff00u) | ((__float_as_uint(x) >> 24) & 0x80u) | 0x7fu;
		if (y != y)
			out = (out & 0xffff00ffu) | ((((__float_as_uint(y) >> 24) & 0x80u) | 0x7fu) << 8);
		if (z != z)
			out = (out & 0xff00ffffu) | ((((__float_as_uint(z) >> 24) & 0x80u) | 0x7fu) << 16);
		if (w != w)
			out = (out & 0x00ffffffu) | ((((__float_as_uint(w) >> 24) & 0x80u) | 0x7fu) << 24);
	}
	return out;
}

/*
** Per-tensor FP8 scale from the tensor's max |x| (num/gpu_cuda.cu:927-938): amax / 448, at
** least 1e-12; a zero, negative or non-finite amax counts as 1e-8.
*/
__device__ __forceinline__ float scale_from_amax(float a)
{
	if (!(a > 0.0f) || !(a <= 3.4028234663852886e38f))
		a = 1e-8f;
	a = a / 448.0f;
	if (a < 1e-12f)
		a = 1e-12f;
	return a;
}

} /* namespace anni */
#endif

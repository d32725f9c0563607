/*
** Host restatement of div_by_const (anni_amd/csrc/adam_math.h): a / b for a step constant
** b = 1 - beta^t whose correctly rounded reciprocal rb = 1.0 / b the host supplies:
**     q = a * rb;  q' = fma(fma(-b, q, a), rb, q)
** compared with the IEEE quotient a / b for every beta in {0.9, 0.95, 0.999}, every t in
** 1..10000 and, per (beta, t), float-valued numerators from every binary exponent a float has
** (subnormals included), both signs, several mantissas each -- the values the kernels divide are
** moments stored as float or bf16.  Prints the number of quotients compared and of mismatches;
** for a mismatch also whether the final float parameter (p - lr * mhat / (sqrt(vhat) + eps))
** differs for a few settings around it.
*/
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static double div_by_const(double a, double b, double rb)
{
	const double q = a * rb;

	return copysign(fma(fma(-b, q, a), rb, q), a);
}

static uint64_t mix64(uint64_t z)
{
	z += 0x9e3779b97f4a7c15ull;
	z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
	z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
	return z ^ (z >> 31);
}

static float from_bits(uint32_t u)
{
	float f;

	memcpy(&f, &u, 4);
	return f;
}

int main(int argc, char **argv)
{
	static const double betas[3] = { 0.9, 0.95, 0.999 };
	const int per_band = argc > 1 ? atoi(argv[1]) : 7;
	long long compared = 0, mismatches = 0, p_differs = 0;
	int bi, t;

	for (bi = 0; bi < 3; bi++) {
#pragma omp parallel for schedule(dynamic, 64) reduction(+ : compared, mismatches, p_differs)
		for (t = 1; t <= 10000; t++) {
			const double b = 1.0 - pow(betas[bi], (double)t);
			const double rb = 1.0 / b;
			uint32_t e;
			int k, s;

			for (e = 0; e < 255; e++)		/* 255 = inf / nan: the kernels divide those the IEEE way */
				for (k = 0; k < per_band; k++)
					for (s = 0; s < 2; s++) {
						/* mantissas: all zero, all ones, bf16-representable (low 16 bits zero), random */
						uint32_t man = (uint32_t)mix64(((uint64_t)bi << 56) ^ ((uint64_t)t << 32) ^ (e << 8) ^ (uint32_t)k) & 0x7fffffu;
						float a;
						double want, got;

						if (k == 0)
							man = 0;
						else if (k == 1)
							man = 0x7fffffu;
						else if (k & 1)
							man &= 0x7f0000u;
						a = from_bits(((uint32_t)s << 31) | (e << 23) | man);
						want = (double)a / b;
						got = div_by_const((double)a, b, rb);
						compared++;
						if (memcmp(&want, &got, 8) != 0) {
							static const double lrs[3] = { 3e-6, 3e-4, 1e-2 };
							int i;

							mismatches++;
							for (i = 0; i < 3; i++) {
								/* as mhat under a typical vhat, and as vhat under a typical mhat */
								const float p1 = (float)(0.02 - lrs[i] * want / (1e-3 + 1e-8));
								const float p2 = (float)(0.02 - lrs[i] * got / (1e-3 + 1e-8));
								const float p3 = (float)(0.02 - lrs[i] * 1e-3 / (sqrt(fabs(want)) + 1e-8));
								const float p4 = (float)(0.02 - lrs[i] * 1e-3 / (sqrt(fabs(got)) + 1e-8));

								if (memcmp(&p1, &p2, 4) != 0 || memcmp(&p3, &p4, 4) != 0)
									p_differs++;
							}
#pragma omp critical
							if (mismatches <= 5)
								printf("mismatch beta %.3f t %d a %.9g: a/b %.17g, by reciprocal %.17g\n",
								    betas[bi], t, (double)a, want, got);
						}
					}
		}
	}
	printf("compared %lld mismatches %lld final_p_differs %lld\n", compared, mismatches, p_differs);
	return 0;
}

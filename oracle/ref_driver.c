/*
** Drives the reference's own compiled optimizer (lang/lm_adam.c, lang/lm_train.c)
** over flat arrays, without a model.  TEST INFRASTRUCTURE ONLY.
**
** Compiled only where the reference tree is present, together with the
** reference's library sources, into oracle/_ref/libanni_ref.so (see Makefile).
** A lm_adam is filled in by hand: slot i points at p[i] / g[i]; with no
** segments and the CPU stub backend linked (gpu_available() == 0),
** lm_adam_step_scaled takes its host path, lang/lm_adam.c:559-606.
*/
#include <stdlib.h>
#include <string.h>
#include "lm_adam.h"
#include "lm_train.h"

typedef struct ref_adam {
	lm_adam	opt;
	float	*p;
	float	*g;
} ref_adam;

ref_adam *ref_adam_create(float *p, float *g, const float *m, const float *v, long n,
	int t, double beta1, double beta2, double eps, double wd, double clip)
{
	ref_adam *r = calloc(1, sizeof(*r));
	long i;

	if (!r)
		return NULL;
	r->opt.slots = calloc((size_t)n, sizeof(lm_adam_slot));
	if (!r->opt.slots) {
		free(r);
		return NULL;
	}
	for (i = 0; i < n; i++) {
		r->opt.slots[i].param = &p[i];
		r->opt.slots[i].grad = &g[i];
		r->opt.slots[i].m = m ? m[i] : 0.0f;
		r->opt.slots[i].v = v ? v[i] : 0.0f;
	}
	r->opt.n = (int)n;
	r->opt.t = t;
	r->opt.beta1 = beta1;
	r->opt.beta2 = beta2;
	r->opt.eps = eps;
	r->opt.weight_decay = wd;
	r->opt.grad_clip = clip;
	r->p = p;
	r->g = g;
	return r;
}

/* Returns opt->t after the call. */
int ref_adam_step(ref_adam *r, double lr, double grad_scale)
{
	lm_adam_step_scaled(&r->opt, lr, grad_scale);
	return r->opt.t;
}

void ref_adam_set(ref_adam *r, double wd, double clip)
{
	r->opt.weight_decay = wd;
	r->opt.grad_clip = clip;
}

void ref_adam_export(const ref_adam *r, float *m, float *v)
{
	long i;

	for (i = 0; i < r->opt.n; i++) {
		m[i] = r->opt.slots[i].m;
		v[i] = r->opt.slots[i].v;
	}
}

void ref_adam_free(ref_adam *r)
{
	if (!r)
		return;
	free(r->opt.slots);
	free(r);
}

double ref_step_lr(double base_lr, int step, int warmup, int decay_steps,
	const char *kind, int sched_from)
{
	double lr;

	lm_train_set_lr_schedule(warmup, decay_steps, kind);
	lm_train_set_lr_sched_from(sched_from);
	lr = lm_train_step_lr(base_lr, step);
	lm_train_set_lr_sched_from(0);
	lm_train_set_lr_schedule(0, 0, "none");
	return lr;
}

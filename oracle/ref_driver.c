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
#include "gpu.h"
#include "lm_adam.h"
#include "lm_serialize.h"
#include "lm_train.h"
#include "train_progress.h"
#include "layernorm.h"
#include "lm_bench.h"
#include "bpe.h"

typedef struct ref_adam {
	lm_adam	opt;
	float	*p;
	float	*g;
	vec	wv;	/* one bias-style segment over the whole flat (device path only) */
	vec	dwv;
	lm_adam_seg	seg;
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

/*
** Same, but registered as one host-resident vector segment (the kind lm_adam.c keeps for
** biases and LayerNorm vectors, lm_adam.c:43-57): when the library is linked against a real
** backend, lm_adam_step_scaled then takes its DEVICE path (lm_adam.c:452-515) -- gpu_malloc,
** H2D gather, gpu_grad_sumsq, clip, gpu_adam_step_dev_bf16, async D2H scatter -- unchanged.
*/
ref_adam *ref_adam_create_device(float *p, float *g, long n, double beta1, double beta2,
	double eps, double wd, double clip)
{
	ref_adam *r = ref_adam_create(p, g, NULL, NULL, n, 0, beta1, beta2, eps, wd, clip);

	if (!r)
		return NULL;
	r->wv.data = p;
	r->wv.n = (int)n;
	r->dwv.data = g;
	r->dwv.n = (int)n;
	r->seg.wv = &r->wv;
	r->seg.dwv = &r->dwv;
	r->seg.off = 0;
	r->seg.n = (int)n;
	r->opt.segs = &r->seg;
	r->opt.n_segs = 1;
	return r;
}

/* Pulls the device-resident moments into the slots (lm_adam.c:336-358). */
void ref_adam_sync_host(ref_adam *r)
{
	lm_adam_sync_host(&r->opt);
}

double ref_adam_last_norm(const ref_adam *r)
{
	return r->opt.last_grad_norm;
}

int ref_adam_on_device(const ref_adam *r)
{
	return r->opt.d_param != NULL;
}

/* Frees the device flats the reference allocated (what lm_adam_free does, lm_adam.c:185-194). */
void ref_adam_release_device(ref_adam *r)
{
	if (r->opt.d_param) {
		gpu_adam_set_bf16_flat(NULL, NULL, 0);
		gpu_free(r->opt.d_param);
		gpu_free(r->opt.d_param_bf16);
		gpu_free(r->opt.d_grad);
		gpu_free(r->opt.d_m);
		gpu_free(r->opt.d_v);
		free(r->opt.h_m);
		free(r->opt.h_v);
		r->opt.d_param = r->opt.d_grad = r->opt.d_m = r->opt.d_v = NULL;
		r->opt.d_param_bf16 = NULL;
		r->opt.h_m = r->opt.h_v = NULL;
	}
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

/*
** The production flow: a real lm (the reference's compile-time sizes: D=1024, 16 heads, FF
** 4096, 12 blocks, lang/lm_config.h:8-24; untied embedding) and lm_adam_create over it
** (lang/lm_adam.c:79-139).  With a real backend linked, lm_adam_step_scaled aliases every
** weight / gradient matrix into its flats and keeps bias / LayerNorm vectors on the host,
** exactly as in training.
*/
typedef struct ref_model {
	lm	*model;
	lm_adam	*opt;
} ref_model;

ref_model *ref_model_create(int vocab, double beta2, double wd, double clip)
{
	ref_model *r = calloc(1, sizeof(*r));

	if (!r)
		return NULL;
	r->model = lm_create_vocab(vocab);
	if (r->model)
		r->opt = lm_adam_create(r->model);
	if (!r->opt) {
		lm_free(&r->model);
		free(r);
		return NULL;
	}
	r->opt->beta2 = beta2;
	r->opt->weight_decay = wd;
	r->opt->grad_clip = clip;
	return r;
}

/*
** The same with the head matrix shared with the embedding, the way the reference trains its
** larger models (`--tokenizer bpe --vocab V --tied`, scripts/run555m.sh:61-63): lm_create_bpe_tied
** wants a tokenizer, so one with V - 260 synthetic merges is made (pairs of raw bytes first, then
** byte + earlier merge: all distinct, every expansion at most three bytes); only its size matters
** to the optimizer.  The model owns the tokenizer afterwards (lm_free releases it).
*/
ref_model *ref_model_create_tied(int vocab, double beta2, double wd, double clip)
{
	ref_model *r = calloc(1, sizeof(*r));
	const int n_merges = vocab - BPE_BASE;
	int *left = NULL;
	int *right = NULL;
	bpe *tok = NULL;
	int i;

	if (!r || n_merges < 0 || n_merges > 65536 * 2)
		goto fail;
	left = malloc((size_t)(n_merges ? n_merges : 1) * sizeof(int));
	right = malloc((size_t)(n_merges ? n_merges : 1) * sizeof(int));
	if (!left || !right)
		goto fail;
	for (i = 0; i < n_merges; i++) {
		if (i < 65536) {
			left[i] = VOCAB_SPECIALS + i / 256;
			right[i] = VOCAB_SPECIALS + i % 256;
		} else {
			left[i] = VOCAB_SPECIALS + (i - 65536) % 256;
			right[i] = BPE_BASE + (i - 65536) / 256;
		}
	}
	tok = bpe_create(left, right, n_merges);
	if (!tok)
		goto fail;
	r->model = lm_create_bpe_tied(tok);
	if (!r->model) {
		bpe_free(&tok);
		goto fail;
	}
	r->opt = lm_adam_create(r->model);
	if (!r->opt) {
		lm_free(&r->model);
		goto fail;
	}
	free(left);
	free(right);
	r->opt->beta2 = beta2;
	r->opt->weight_decay = wd;
	r->opt->grad_clip = clip;
	return r;
fail:
	free(left);
	free(right);
	free(r);
	return NULL;
}

/* The compile-time model sizes this library was built with (lang/lm_config.h:8-24). */
void ref_model_dims(int *d_model, int *n_heads, int *d_ff, int *n_blocks)
{
	*d_model = LM_D_MODEL;
	*n_heads = LM_N_HEADS;
	*d_ff = LM_D_FF;
	*n_blocks = LM_N_BLOCKS;
}

long ref_model_n(const ref_model *r) { return r->opt->n; }
int ref_model_n_segs(const ref_model *r) { return r->opt->n_segs; }
int ref_model_t(const ref_model *r) { return r->opt->t; }
int ref_model_on_device(const ref_model *r) { return r->opt->d_param != NULL; }
double ref_model_last_norm(const ref_model *r) { return r->opt->last_grad_norm; }
/* The caller's device flats (lang/lm_adam.h:43-44), for tests of what the backend serves from them. */
void *ref_model_d_param(const ref_model *r) { return r->opt->d_param; }
void *ref_model_d_param_bf16(const ref_model *r) { return r->opt->d_param_bf16; }

/* seg i: off, n, 1 for a matrix / 0 for a vector. */
void ref_model_seg(const ref_model *r, int i, long *off, long *n, int *is_mat)
{
	*off = r->opt->segs[i].off;
	*n = r->opt->segs[i].n;
	*is_mat = r->opt->segs[i].w != NULL;
}

/* Parameters (host view) into / out of one flat array in slot order. */
void ref_model_get_params(ref_model *r, float *flat)
{
	long i;

	lm_adam_sync_host(r->opt);	/* device-authoritative weights and m/v -> host */
	for (i = 0; i < r->opt->n; i++)
		flat[i] = *r->opt->slots[i].param;
}

void ref_model_get_moments(ref_model *r, float *m, float *v)
{
	long i;

	lm_adam_sync_host(r->opt);
	for (i = 0; i < r->opt->n; i++) {
		m[i] = r->opt->slots[i].m;
		v[i] = r->opt->slots[i].v;
	}
}

/*
** New gradients from one flat array: host dW / db everywhere (what the first step and the
** vector segments read), and straight into the device flat once the matrices are aliased
** there (where backward would have written them).
*/
int ref_model_set_grads(ref_model *r, const float *flat)
{
	long i;

	for (i = 0; i < r->opt->n; i++)
		*r->opt->slots[i].grad = flat[i];
	/* host writes leave a mat host-authoritative (num/mat.h: mat_host_dirty) unless it is aliased */
	for (i = 0; i < r->opt->n_segs; i++)
		if (r->opt->segs[i].dw && r->opt->segs[i].dw->on_device != MAT_DEV_ALIASED)
			mat_host_dirty(r->opt->segs[i].dw);
	if (r->opt->d_grad)
		return gpu_memcpy_h2d(r->opt->d_grad, flat, (size_t)r->opt->n * sizeof(float));
	return 0;
}

/* lm_adam_set_offload (lang/lm_adam.c:211-214): m and v leave the device after every step. */
void ref_set_offload(int on)
{
	lm_adam_set_offload(on);
}

int ref_model_mv_on_device(const ref_model *r)
{
	return r->opt->d_m != NULL && r->opt->d_v != NULL;
}

int ref_model_step(ref_model *r, double lr, double grad_scale)
{
	lm_adam_step_scaled(r->opt, lr, grad_scale);
	return r->opt->t;
}

/* lm_save_checkpoint / lm_load_checkpoint (lang/lm_serialize.c:300-331,526-587) on this model. */
int ref_model_save_checkpoint(ref_model *r, int epoch, int step, const char *path)
{
	return lm_save_checkpoint(r->model, r->opt, epoch, step, path);
}

ref_model *ref_model_load_checkpoint(const char *path, int *epoch, int *step)
{
	ref_model *r = calloc(1, sizeof(*r));

	if (!r)
		return NULL;
	r->model = lm_load_checkpoint(path, &r->opt, epoch, step);
	if (!r->model) {
		free(r);
		return NULL;
	}
	return r;
}

void ref_model_free(ref_model *r)
{
	if (!r)
		return;
	lm_adam_free(&r->opt);
	lm_free(&r->model);
	free(r);
}

/*
** dgamma / dbeta as the reference's host layernorm_backward accumulates them
** (lang/layernorm.c:312-376; model width LM_D_MODEL is a compile-time constant): both start
** from the given values, dy and x_hat are T x LM_D_MODEL row-major.  Returns LM_D_MODEL, -1 on failure.
*/
int ref_ln_backward_grads(const float *dy, const float *x_hat, int T, float *dgamma, float *dbeta)
{
	layernorm *ln = layernorm_create();
	ln_cache *c = ln_cache_create(T);
	mat *mdy = mat_create(T, LM_D_MODEL);
	mat *mdx = mat_create(T, LM_D_MODEL);
	int rc = -1;
	int i;

	if (c && !c->x_hat)		/* not stored when the device recomputes it (layernorm.c:116-121) */
		c->x_hat = mat_create(T, LM_D_MODEL);
	if (ln && c && mdy && mdx && c->x_hat && c->inv_std) {
		memcpy(mdy->data, dy, (size_t)T * LM_D_MODEL * sizeof(float));
		memcpy(c->x_hat->data, x_hat, (size_t)T * LM_D_MODEL * sizeof(float));
		for (i = 0; i < T; i++)
			c->inv_std->data[i] = 1.0f;
		c->T = T;
		c->x_src = NULL;
		memcpy(ln->dgamma->data, dgamma, LM_D_MODEL * sizeof(float));
		memcpy(ln->dbeta->data, dbeta, LM_D_MODEL * sizeof(float));
		if (layernorm_backward(mdx, mdy, ln, c) == 0) {
			memcpy(dgamma, ln->dgamma->data, LM_D_MODEL * sizeof(float));
			memcpy(dbeta, ln->dbeta->data, LM_D_MODEL * sizeof(float));
			rc = LM_D_MODEL;
		}
	}
	mat_free(&mdy);
	mat_free(&mdx);
	ln_cache_free(&c);
	layernorm_free(&ln);
	return rc;
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

/* lm_train_step_lr under a live control whose lr field is `ctl_lr` (lang/train_progress.h:46-56). */
double ref_step_lr_controlled(double base_lr, int step, int warmup, int decay_steps,
	const char *kind, double ctl_lr)
{
	train_control ctl;
	double lr;

	memset(&ctl, 0, sizeof(ctl));
	ctl.lr = ctl_lr;
	lm_train_set_control(&ctl);
	lr = ref_step_lr(base_lr, step, warmup, decay_steps, kind, 0);
	lm_train_set_control(NULL);
	return lr;
}

/*
** The reference's own bench harness, `anni lm bench step --profile --json FILE`
** (lang/lm_bench.c:619-643): one packed training step per iteration on whatever backend is
** linked, one JSON line appended to `json`.  Returns lm_bench_step's result (0 done, 1 loss
** check failed, 2 refused: its harness refuses to run on the CPU stub).
*/
int ref_bench_step(const char *json, int B, int T, int vocab, int warmup, int steps)
{
	lm_bench_cfg cfg;

	lm_bench_cfg_defaults(&cfg);
	cfg.B = B;
	cfg.T = T;
	cfg.vocab = vocab;
	cfg.prec = LM_BENCH_FP32;
	cfg.graphs = 0;
	cfg.warmup = warmup;
	cfg.steps = steps;
	cfg.profile = 1;
	cfg.ceiling = 0;
	cfg.allow_busy = 1;
	cfg.json = json;
	return lm_bench_step(&cfg);
}

/*
** The device-resident optimizer arena and its multi-tensor step: the MI355X
** counterpart of lang/lm_adam.c (registration lm_adam.c:79-139, arena
** lm_adam.c:217-311, step lm_adam.c:452-515,522-607) and of lm_train_step_lr
** (lang/lm_train.c:98-124).  See include/anni_adam.h.
*/
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <new>
#include <vector>
#include "adam_kernels.h"
#include "anni_adam.h"
#include "backend_state.h"

using namespace anni;

struct anni_adam_priv {
	void			*arena;
	size_t			arena_bytes;
	Seg			*d_segs;
	int32_t			*d_tile_seg;
	double			*d_partials;
	StepState		*d_state;
	StepState		*h_state;	/* page-locked */
	void			*own_grad;	/* the arena's gradient flat (NULL when external) */
	std::vector<int64_t>	offsets;
	std::vector<uint32_t>	flags;
	bool			any_decay_off;
};

static size_t elem_bytes(int type)
{
	return type == ANNI_F32 ? 4 : type == ANNI_BF16 ? 2 : 1;
}

static size_t round_up(size_t x, size_t a)
{
	return (x + a - 1) / a * a;
}

extern "C" {

anni_adam *anni_adam_create(const anni_tensor *tensors, int n_tensors,
	const anni_adam_config *cfg)
{
	const size_t big = (size_t)2 << 20;	/* each flat starts on a 2 MiB boundary */
	anni_adam *opt;
	anni_adam_priv *pv;
	int64_t n = 0;
	size_t off_p, off_m, off_v, off_twin, off_g, off_gscale, off_segs, off_tiles, off_part,
	    off_state, total;
	int64_t n_tiles;
	std::vector<Seg> segs;
	std::vector<int32_t> tile_seg;
	std::vector<float> ones;

	if (!tensors || n_tensors <= 0 || !cfg || !device_ready())
		return nullptr;
	if (cfg->grad_type < ANNI_F32 || cfg->grad_type > ANNI_FP8_E4M3
	    || (cfg->moment_type != ANNI_F32 && cfg->moment_type != ANNI_BF16))
		return nullptr;
	for (int i = 0; i < n_tensors; i++) {
		if (tensors[i].n < 0)
			return nullptr;
		n += tensors[i].n;
	}
	if (n <= 0)
		return nullptr;
	opt = (anni_adam *)calloc(1, sizeof(*opt));
	pv = new (std::nothrow) anni_adam_priv();
	if (!opt || !pv) {
		free(opt);
		delete pv;
		return nullptr;
	}
	opt->priv = pv;
	opt->n = n;
	opt->n_tensors = n_tensors;
	opt->beta1 = 0.9;	/* lm_adam.c:110-115 */
	opt->beta2 = 0.999;
	opt->eps = 1e-8;
	opt->cfg = *cfg;

	/* Registration: packed offsets in order, as add_mat / add_vec lay the slots out. */
	segs.resize((size_t)n_tensors);
	pv->offsets.resize((size_t)n_tensors);
	pv->flags.resize((size_t)n_tensors);
	{
		int64_t at = 0;

		for (int i = 0; i < n_tensors; i++) {
			segs[(size_t)i].begin = at;
			segs[(size_t)i].end = at + tensors[i].n;
			segs[(size_t)i].flags = tensors[i].flags;
			segs[(size_t)i].pad = 0;
			pv->offsets[(size_t)i] = at;
			pv->flags[(size_t)i] = tensors[i].flags;
			at += tensors[i].n;
		}
	}
	/* Launch table: the tensor that holds the first element of each tile. */
	n_tiles = (n + kTile - 1) / kTile;
	tile_seg.resize((size_t)n_tiles);
	{
		int s = 0;

		for (int64_t k = 0; k < n_tiles; k++) {
			while (segs[(size_t)s].end <= k * kTile)
				s++;
			tile_seg[(size_t)k] = s;
		}
	}

	off_p = 0;
	off_m = round_up(off_p + (size_t)n * 4, big);
	off_v = round_up(off_m + (size_t)n * elem_bytes(cfg->moment_type), big);
	off_twin = round_up(off_v + (size_t)n * elem_bytes(cfg->moment_type), big);
	off_g = round_up(off_twin + (cfg->twins ? (size_t)n * 2 : 0), big);
	off_gscale = round_up(off_g + (cfg->own_grad ? (size_t)n * elem_bytes(cfg->grad_type) : 0),
	    big);
	off_segs = round_up(off_gscale + (size_t)n_tensors * sizeof(float), 256);
	off_tiles = round_up(off_segs + (size_t)n_tensors * sizeof(Seg), 256);
	off_part = round_up(off_tiles + (size_t)n_tiles * sizeof(int32_t), 256);
	off_state = round_up(off_part + (size_t)kMaxPartials * sizeof(double), 256);
	total = off_state + 256;

	if (!hip_ok(hipMalloc(&pv->arena, total), "arena hipMalloc")
	    || !hip_ok(hipHostMalloc((void **)&pv->h_state, sizeof(StepState),
	    hipHostMallocDefault), "arena hipHostMalloc")) {
		(void)hipGetLastError();
		anni_adam_free(&opt);
		return nullptr;
	}
	pv->arena_bytes = total;
	{
		char *base = (char *)pv->arena;
		hipStream_t st = compute_stream();

		opt->d_param = (float *)(base + off_p);
		opt->d_m = base + off_m;
		opt->d_v = base + off_v;
		opt->d_param_bf16 = cfg->twins ? base + off_twin : nullptr;
		pv->own_grad = cfg->own_grad ? base + off_g : nullptr;
		opt->d_grad = pv->own_grad;
		opt->d_gscale = (float *)(base + off_gscale);
		pv->d_segs = (Seg *)(base + off_segs);
		pv->d_tile_seg = (int32_t *)(base + off_tiles);
		pv->d_partials = (double *)(base + off_part);
		pv->d_state = (StepState *)(base + off_state);

		ones.assign((size_t)n_tensors, 1.0f);
		/* State starts at zero (slots are calloc'ed, lm_adam.c:92); the fills run on the stream. */
		if (launch_fill_bytes(st, base + off_p, 0, off_twin) != 0
		    || (cfg->twins && launch_fill_bytes(st, base + off_twin, 0, (size_t)n * 2) != 0)
		    || (cfg->own_grad && launch_fill_bytes(st, base + off_g, 0,
		    (size_t)n * elem_bytes(cfg->grad_type)) != 0)
		    || launch_fill_bytes(st, base + off_part, 0, total - off_part) != 0
		    || !hip_ok(hipMemcpyAsync(opt->d_gscale, ones.data(),
		    (size_t)n_tensors * sizeof(float), hipMemcpyHostToDevice, st), "gscale")
		    || !hip_ok(hipMemcpyAsync(pv->d_segs, segs.data(),
		    (size_t)n_tensors * sizeof(Seg), hipMemcpyHostToDevice, st), "segs")
		    || !hip_ok(hipMemcpyAsync(pv->d_tile_seg, tile_seg.data(),
		    (size_t)n_tiles * sizeof(int32_t), hipMemcpyHostToDevice, st), "tiles")
		    || !hip_ok(hipStreamSynchronize(st), "arena init")) {
			anni_adam_free(&opt);
			return nullptr;
		}
	}
	memset(pv->h_state, 0, sizeof(StepState));
	return opt;
}

void anni_adam_free(anni_adam **popt)
{
	anni_adam *opt;

	if (!popt || !*popt)
		return;
	opt = *popt;
	if (opt->priv) {
		if (device_ready())
			(void)hipStreamSynchronize(compute_stream());
		if (opt->priv->arena)
			(void)hip_ok(hipFree(opt->priv->arena), "arena hipFree");
		if (opt->priv->h_state)
			(void)hip_ok(hipHostFree(opt->priv->h_state), "arena hipHostFree");
		delete opt->priv;
	}
	free(opt);
	*popt = nullptr;
}

int64_t anni_adam_tensor_offset(const anni_adam *opt, int i)
{
	if (!opt || !opt->priv || i < 0 || i >= opt->n_tensors)
		return -1;
	return opt->priv->offsets[(size_t)i];
}

int anni_adam_bind_grad(anni_adam *opt, void *d_grad)
{
	if (!opt || !opt->priv)
		return -1;
	opt->d_grad = d_grad ? d_grad : opt->priv->own_grad;
	return opt->d_grad ? 0 : -1;
}

int anni_adam_seed_twins(anni_adam *opt)
{
	if (!opt || !opt->d_param_bf16)
		return -1;
	return launch_f32_to_bf16(compute_stream(), (uint16_t *)opt->d_param_bf16, opt->d_param,
	    opt->n);
}

int anni_adam_zero_grad(anni_adam *opt)
{
	if (!opt || !opt->d_grad)
		return -1;
	return launch_fill_bytes(compute_stream(), opt->d_grad, 0,
	    (size_t)opt->n * elem_bytes(opt->cfg.grad_type));
}

} /* extern "C" */

/* Fills the kernel-side description of the arena. */
static void describe(const anni_adam *opt, Flat *f)
{
	const anni_adam_priv *pv = opt->priv;

	memset(f, 0, sizeof(*f));
	f->p = opt->d_param;
	f->g = opt->d_grad;
	f->m = opt->d_m;
	f->v = opt->d_v;
	f->twin = (uint16_t *)opt->d_param_bf16;
	f->n = opt->n;
	f->grad_type = opt->cfg.grad_type;
	f->moment_type = opt->cfg.moment_type;
	f->segs = pv->d_segs;
	f->tile_seg = pv->d_tile_seg;
	f->gscale = opt->d_gscale;
}

/* One step; ev (may be NULL) = three events recorded before, between and after the two launches. */
static int step_impl(anni_adam *opt, double lr, double grad_scale, hipEvent_t *ev)
{
	anni_adam_priv *pv;
	hipStream_t st;
	StepConsts c;
	NormIn norm;
	Flat f;
	int np = 0;

	if (!opt || !opt->priv)
		return -1;
	if (lr <= 0.0)
		return 1;			/* lm_adam.c:531-532: t is not advanced */
	if (!opt->d_grad || !device_ready())
		return -1;
	pv = opt->priv;
	st = compute_stream();
	opt->t++;				/* lm_adam.c:533 */
	c.bc1 = 1.0 - pow(opt->beta1, (double)opt->t);	/* lm_adam.c:571-572 */
	c.bc2 = 1.0 - pow(opt->beta2, (double)opt->t);
	if (c.bc1 <= 0.0 || c.bc2 <= 0.0)
		return -1;			/* gpu_cuda.cu:8681-8682 */
	c.beta1 = opt->beta1;
	c.omb1 = 1.0 - opt->beta1;
	c.beta2 = opt->beta2;
	c.omb2 = 1.0 - opt->beta2;
	c.eps = opt->eps;
	c.lr = lr;
	c.decay_on = opt->weight_decay > 0.0 ? 1 : 0;	/* lm_adam.c:594 */
	c.lr_wd = c.decay_on ? lr * opt->weight_decay : 0.0;
	describe(opt, &f);
	memset(&norm, 0, sizeof(norm));
	norm.use_norm = (opt->grad_clip > 0.0 || opt->cfg.skip_nonfinite) ? 1 : 0;
	norm.clip = opt->grad_clip > 0.0 ? opt->grad_clip : 0.0;
	norm.skip_nonfinite = opt->cfg.skip_nonfinite;
	norm.state = pv->d_state;
	if (ev)
		(void)hipEventRecord(ev[0], st);
	if (norm.use_norm) {
		if (launch_sumsq(st, f, grad_scale, pv->d_partials, &np) != 0)
			return -1;
		norm.partials = pv->d_partials;
		norm.n_partials = np;
	}
	if (ev)
		(void)hipEventRecord(ev[1], st);
	if (launch_update(st, f, c, grad_scale, norm) != 0)
		return -1;
	if (ev)
		(void)hipEventRecord(ev[2], st);
	return 0;
}

extern "C" {

int anni_adam_step_scaled(anni_adam *opt, double lr, double grad_scale)
{
	return step_impl(opt, lr, grad_scale, nullptr);
}

int anni_adam_step(anni_adam *opt, double lr)
{
	return step_impl(opt, lr, 1.0, nullptr);
}

int anni_adam_sync_stats(anni_adam *opt)
{
	anni_adam_priv *pv;
	hipStream_t st;

	if (!opt || !opt->priv || !device_ready())
		return -1;
	pv = opt->priv;
	st = compute_stream();
	if (!hip_ok(hipMemcpyAsync(pv->h_state, pv->d_state, sizeof(StepState),
	    hipMemcpyDeviceToHost, st), "stats d2h")
	    || !hip_ok(hipStreamSynchronize(st), "stats sync"))
		return -1;
	opt->last_sumsq = pv->h_state->sumsq;
	opt->last_grad_norm = pv->h_state->norm;
	opt->last_grad_scale = pv->h_state->grad_scale;
	opt->last_skipped = pv->h_state->skipped;
	opt->last_clipped = pv->h_state->clipped;
	return 0;
}

int anni_adam_time_steps(anni_adam *opt, int count, void *const *grads, int n_grads,
	const double *lr, const double *grad_scale, float *ms_total, float *ms_sumsq,
	float *ms_update)
{
	std::vector<hipEvent_t> ev;
	hipStream_t st;
	int rc = 0;
	bool per_kernel = ms_sumsq || ms_update;

	if (!opt || count <= 0 || !lr || !grad_scale || !ms_total || !device_ready())
		return -1;
	if (grads && n_grads <= 0)
		return -1;
	st = compute_stream();
	ev.resize(per_kernel ? (size_t)count * 3 : 2);
	for (size_t i = 0; i < ev.size(); i++)
		if (hipEventCreate(&ev[i]) != hipSuccess) {
			for (size_t k = 0; k < i; k++)
				(void)hipEventDestroy(ev[k]);
			return -1;
		}
	if (!per_kernel)
		(void)hipEventRecord(ev[0], st);
	for (int i = 0; i < count && rc == 0; i++) {
		if (grads)
			(void)anni_adam_bind_grad(opt, grads[i % n_grads]);
		rc = step_impl(opt, lr[i], grad_scale[i], per_kernel ? &ev[(size_t)i * 3] : nullptr);
		if (rc == 1)
			rc = -1;		/* a timed run must not contain no-op steps */
	}
	if (!per_kernel)
		(void)hipEventRecord(ev[1], st);
	if (!hip_ok(hipStreamSynchronize(st), "time_steps sync"))
		rc = -1;
	if (rc == 0) {
		float ms = 0.0f;

		if (per_kernel) {
			float a = 0.0f, b = 0.0f;

			for (int i = 0; i < count; i++) {
				float x = 0.0f, y = 0.0f;

				(void)hipEventElapsedTime(&x, ev[(size_t)i * 3], ev[(size_t)i * 3 + 1]);
				(void)hipEventElapsedTime(&y, ev[(size_t)i * 3 + 1], ev[(size_t)i * 3 + 2]);
				a += x;
				b += y;
			}
			(void)hipEventElapsedTime(&ms, ev[0], ev[(size_t)count * 3 - 1]);
			if (ms_sumsq)
				*ms_sumsq = a;
			if (ms_update)
				*ms_update = b;
		} else {
			(void)hipEventElapsedTime(&ms, ev[0], ev[1]);
		}
		*ms_total = ms;
	}
	for (size_t i = 0; i < ev.size(); i++)
		(void)hipEventDestroy(ev[i]);
	return rc;
}

/* ---- learning-rate schedule (lang/lm_train.c:98-124,398-411) ------------------ */

static int g_warmup_steps;
static int g_decay_steps;
static int g_decay_kind;	/* 0 none, 1 linear, 2 cosine (any other name: cosine, as the reference) */
static int g_sched_from;

void anni_lr_set_schedule(int warmup_steps, int decay_steps, const char *kind)
{
	g_warmup_steps = warmup_steps < 0 ? 0 : warmup_steps;
	g_decay_steps = decay_steps < 0 ? 0 : decay_steps;
	if (!kind || strcmp(kind, "none") == 0)
		g_decay_kind = 0;
	else if (strcmp(kind, "linear") == 0)
		g_decay_kind = 1;
	else
		g_decay_kind = 2;
}

void anni_lr_set_sched_from(int from)
{
	g_sched_from = from < 0 ? 0 : from;
}

double anni_lr_step(double base_lr, int step)
{
	double q;
	int u;

	step -= g_sched_from;
	if (step < 0)
		step = 0;
	if (g_warmup_steps > 0 && step < g_warmup_steps)
		return base_lr * ((double)step + 1.0) / (double)g_warmup_steps;
	if (g_decay_steps <= 0 || g_decay_kind == 0)
		return base_lr;
	u = step - g_warmup_steps;
	if (u < 0)
		u = 0;
	if (u > g_decay_steps)
		u = g_decay_steps;
	q = (double)u / (double)g_decay_steps;
	if (g_decay_kind == 1)
		return base_lr * (1.0 - q);
	return base_lr * 0.5 * (1.0 + cos(3.14159265358979323846 * q));
}

void *anni_gpu_stream(void)
{
	return device_ready() ? (void *)compute_stream() : nullptr;
}

void anni_gpu_set_stream(void *hip_stream)
{
	if (device_ready())
		set_compute_stream((hipStream_t)hip_stream);
}

} /* extern "C" */

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
#include <unistd.h>
#include <mutex>
#include <new>
#include <vector>
#include "adam_kernels.h"
#include "anni_adam.h"
#include "anni_gpu.h"
#include "anni_hooks.h"
#include "backend_state.h"
#include "placement.h"

using namespace anni;

/* Step state (128 bytes) + the ticket counters of the norm's second stage. */
static const size_t kStateBytes = 128 + ((kTicketBytes + 255) / 256) * 256;

static size_t elem_bytes(int type)
{
	return type == ANNI_F32 ? 4 : type == ANNI_BF16 ? 2 : 1;
}

static size_t round_up(size_t x, size_t a)
{
	return (x + a - 1) / a * a;
}

/* Byte sizes of the flats of one arena. */
struct Sizes {
	int64_t	n;
	int	n_tensors;
	int64_t	n_tiles;
	int	n_slots;
	size_t	p_bytes;
	size_t	mv_bytes;
	size_t	tw_bytes;
	size_t	g_bytes;	/* one gradient slot, rounded up to 2 MiB */
};

struct anni_adam_priv {
	void			*arena;		/* p, m and the tables (split), or everything (compact) */
	void			*arena2;	/* split: v, the twins and the gradient slots */
	size_t			arena_bytes;	/* both allocations together */
	size_t			resident_bytes;	/* what a step touches: p, m, v, twins, one gradient flat, the tables */
	double			apart_ratio;	/* split: time(all flats in one block) / time(this placement) on the probe */
	Seg			*d_segs;
	int32_t			*d_tile_seg;
	double			*d_partials;
	StepState		*d_state;
	StepState		*h_state;	/* page-locked */
	char			*grad_slots;	/* the arena's gradient flats (NULL when external) */
	size_t			grad_slot_bytes;	/* distance between consecutive slots */
	int			n_grad_slots;
	int			logged_t;	/* the step whose messages anni_adam_sync_stats has printed */
	int			split;		/* 1: two allocations (see the layout note in anni_adam_create) */
	double			probe_gbps;	/* update throughput measured at creation (0: not measured) */
	PlaceStats		search;		/* split: what the search for the second block cost */
	std::vector<int64_t>	offsets;
	std::vector<uint32_t>	flags;
	/* derived outputs (anni_adam_enable_derived): one more allocation */
	std::vector<Seg>	segs;		/* host copy of the device table */
	void			*derived;
	int			derived_owned;	/* 1: derived is an allocation of its own */
	uint32_t		*d_wamax;	/* max |p| of each flagged tensor, cleared by a fill kernel before every step */
	PackDesc		*d_packs;
	float			*d_tile_amax;	/* per-wavefront max |p| of every whole tile */
	int			fp8_twins;	/* 1: some tensor keeps an E4M3 twin */
	/* scratch of anni_adam_quantize_grads, allocated at its first call: per-tensor max words, then the tile maxima */
	void			*gq_scratch;
	/* anni_adam_set_offload */
	Sizes			z;		/* what the arena was laid out for */
	int			mv_apart;	/* 1: m and v are blocks of their own (gpu_malloc), not parts of the arena's */
	int			offload;	/* 1: m and v leave the device after every step */
	void			*h_m;		/* page-locked homes of m and v while they are away */
	void			*h_v;
};

/* One or two device allocations with the flats laid out in them. */
struct Placement {
	char	*a;		/* p, m, tables (split) or everything (compact) */
	char	*b;		/* split: v, twins, gradient slots; NULL when compact */
	size_t	a_bytes, b_bytes;
	/* offsets from a: */
	size_t	off_p, off_m, off_gscale, off_segs, off_tiles, off_part, off_state;
	/* offsets from b (from a when compact): */
	size_t	off_v, off_twin, off_g;
	int	split;
	double	ratio;		/* split: what alloc_apart_from measured */
	double	gbps;		/* what the full-size probe measured (0: not probed) */
	PlaceStats	search;	/* split: what the search for the second block cost */
};

/*
** Layout.  MI355X's device memory behaves as three sections of 96 GiB, and a kernel that
** streams several arrays at once runs about 15 % faster when its arrays are split over two
** sections than when one section holds them all (placement.h).  SPLIT therefore uses TWO
** allocations of exactly the size of their contents: p, m and the small tables in one, v, the
** twins and the gradient slots in the other (16 + 18 of the update's 34 bytes per parameter),
** the second one searched for in another section by timing the update on the zero-filled flats
** themselves (alloc_apart_from).  Nothing is reserved beyond what the arena holds.  COMPACT is
** one allocation with the flats at 2 MiB boundaries.
*/
static size_t tables_bytes(const Sizes &z)
{
	return round_up((size_t)z.n_tensors * sizeof(float), 256)
	    + round_up((size_t)z.n_tensors * sizeof(Seg), 256)
	    + round_up((size_t)z.n_tiles * sizeof(int32_t), 256)
	    + round_up((size_t)kMaxPartials * sizeof(double), 256) + kStateBytes;
}

static bool place(const Sizes &z, bool split, Placement *pl)
{
	const size_t big = (size_t)2 << 20;
	void *mem = nullptr;

	memset(pl, 0, sizeof(*pl));
	pl->ratio = 1.0;
	pl->off_p = 0;
	pl->off_m = round_up(pl->off_p + z.p_bytes, big);
	if (split) {
		pl->off_gscale = round_up(pl->off_m + z.mv_bytes, big);
		pl->off_v = 0;
	} else {
		pl->off_v = round_up(pl->off_m + z.mv_bytes, big);
	}
	pl->off_twin = round_up(pl->off_v + z.mv_bytes, big);
	pl->off_g = round_up(pl->off_twin + z.tw_bytes, big);
	if (split)
		pl->b_bytes = pl->off_g + (size_t)z.n_slots * z.g_bytes + big;
	else
		pl->off_gscale = round_up(pl->off_g + (size_t)z.n_slots * z.g_bytes, big);
	pl->off_segs = pl->off_gscale + round_up((size_t)z.n_tensors * sizeof(float), 256);
	pl->off_tiles = pl->off_segs + round_up((size_t)z.n_tensors * sizeof(Seg), 256);
	pl->off_part = pl->off_tiles + round_up((size_t)z.n_tiles * sizeof(int32_t), 256);
	pl->off_state = pl->off_part + round_up((size_t)kMaxPartials * sizeof(double), 256);
	pl->a_bytes = pl->off_gscale + tables_bytes(z);
	pl->split = split ? 1 : 0;
	if (hipMalloc(&mem, pl->a_bytes) != hipSuccess) {
		(void)hipGetLastError();
		return false;
	}
	pl->a = (char *)mem;
	if (split) {
		/* p and m are still scratch: the search times the update on them and on each candidate */
		pl->b = (char *)alloc_apart_from(pl->a, pl->off_gscale, pl->b_bytes, &pl->ratio, &pl->search);
		if (!pl->b) {
			(void)hipFree(pl->a);
			pl->a = nullptr;
			return false;
		}
	}
	return true;
}

static void unplace(Placement *pl)
{
	if (pl->a)
		(void)hip_ok(hipFree(pl->a), "arena hipFree");
	if (pl->b)
		(void)hip_ok(hipFree(pl->b), "arena hipFree");
	pl->a = nullptr;
	pl->b = nullptr;
}

/* Points the handle at a placement. */
static void adopt(anni_adam *opt, const Sizes &z, const Placement &pl)
{
	anni_adam_priv *pv = opt->priv;
	char *base = pl.a;
	char *second = pl.b ? pl.b : pl.a;

	pv->arena = pl.a;
	pv->arena2 = pl.b;
	pv->arena_bytes = pl.a_bytes + pl.b_bytes;
	pv->resident_bytes = z.p_bytes + 2 * z.mv_bytes + z.tw_bytes
	    + (size_t)z.n * elem_bytes(opt->cfg.grad_type) + tables_bytes(z);
	pv->split = pl.split;
	pv->apart_ratio = pl.ratio;
	pv->probe_gbps = pl.gbps;
	pv->search = pl.search;
	opt->d_param = (float *)(base + pl.off_p);
	opt->d_m = base + pl.off_m;
	opt->d_v = second + pl.off_v;
	opt->d_param_bf16 = z.tw_bytes ? second + pl.off_twin : nullptr;
	pv->grad_slots = z.n_slots ? second + pl.off_g : nullptr;
	pv->grad_slot_bytes = z.g_bytes;
	pv->n_grad_slots = z.n_slots;
	opt->d_grad = pv->grad_slots;
	opt->d_gscale = (float *)(base + pl.off_gscale);
	pv->d_segs = (Seg *)(base + pl.off_segs);
	pv->d_tile_seg = (int32_t *)(base + pl.off_tiles);
	pv->d_partials = (double *)(base + pl.off_part);
	pv->d_state = (StepState *)(base + pl.off_state);
}

/* State starts at zero (slots are calloc'ed, lm_adam.c:92); tables are uploaded; all on the stream. */
static bool init_contents(anni_adam *opt, const Sizes &z, const Placement &pl,
	const std::vector<Seg> &segs, const std::vector<int32_t> &tile_seg)
{
	char *base = pl.a;
	char *second = pl.b ? pl.b : pl.a;
	hipStream_t st = compute_stream();
	std::vector<float> ones((size_t)z.n_tensors, 1.0f);

	return launch_fill_bytes(st, base + pl.off_p, 0, z.p_bytes) == 0
	    && launch_fill_bytes(st, base + pl.off_m, 0, z.mv_bytes) == 0
	    && launch_fill_bytes(st, second + pl.off_v, 0, z.mv_bytes) == 0
	    && (!z.tw_bytes || launch_fill_bytes(st, second + pl.off_twin, 0, z.tw_bytes) == 0)
	    && (!z.n_slots || launch_fill_bytes(st, second + pl.off_g, 0,
	    (size_t)z.n_slots * z.g_bytes) == 0)
	    && launch_fill_bytes(st, base + pl.off_part, 0, pl.off_state + kStateBytes - pl.off_part) == 0
	    && hip_ok(hipMemcpyAsync(opt->d_gscale, ones.data(), (size_t)z.n_tensors * sizeof(float),
	    hipMemcpyHostToDevice, st), "gscale")
	    && hip_ok(hipMemcpyAsync(opt->priv->d_segs, segs.data(), (size_t)z.n_tensors * sizeof(Seg),
	    hipMemcpyHostToDevice, st), "segs")
	    && hip_ok(hipMemcpyAsync(opt->priv->d_tile_seg, tile_seg.data(),
	    (size_t)z.n_tiles * sizeof(int32_t), hipMemcpyHostToDevice, st), "tiles")
	    && hip_ok(sync_stream_and_deliver(), "arena init");
}

static void describe(const anni_adam *opt, Flat *f);

/*
** Throughput of the update on this placement, in GB/s of algorithmic traffic.  Run on
** the all-zero state it leaves every flat as it is (0 stays 0 under the update).
*/
static double probe(const anni_adam *opt)
{
	hipStream_t st = compute_stream();
	hipEvent_t e0, e1;
	StepConsts c;
	NormIn norm;
	Flat f;
	float ms = 0.0f;
	const double bytes = (double)opt->n * (8.0 + 2.0 * elem_bytes(opt->cfg.grad_type)
	    + 4.0 * elem_bytes(opt->cfg.moment_type) + (opt->d_param_bf16 ? 2.0 : 0.0));

	if (!opt->d_grad)
		return 0.0;
	memset(&c, 0, sizeof(c));
	c.beta1 = 0.9;
	c.omb1 = 1.0 - 0.9;
	c.beta2 = 0.95;
	c.omb2 = 1.0 - 0.95;
	c.eps = 1e-8;
	c.bc1 = c.omb1;
	c.bc2 = c.omb2;
	c.rbc1 = 1.0 / c.bc1;
	c.rbc2 = 1.0 / c.bc2;
	c.lr = 1e-3;
	memset(&norm, 0, sizeof(norm));
	describe(opt, &f);
	if (hipEventCreate(&e0) != hipSuccess)
		return 0.0;
	if (hipEventCreate(&e1) != hipSuccess) {
		(void)hipEventDestroy(e0);
		return 0.0;
	}
	if (launch_update(st, f, c, 1.0, norm) == 0) {
		/* the timed launches run on the middle and the last gradient slot: the slots lie in other
		** regions than the state and can be slow when the state is not */
		const anni_adam_priv *pv = opt->priv;
		const int last = pv->n_grad_slots > 0 ? pv->n_grad_slots - 1 : 0;

		(void)hipEventRecord(e0, st);
		if (pv->grad_slots)
			f.g = pv->grad_slots + (size_t)(last / 2) * pv->grad_slot_bytes;
		(void)launch_update(st, f, c, 1.0, norm);
		if (pv->grad_slots)
			f.g = pv->grad_slots + (size_t)last * pv->grad_slot_bytes;
		(void)launch_update(st, f, c, 1.0, norm);
		(void)hipEventRecord(e1, st);
		if (hipStreamSynchronize(st) != hipSuccess
		    || hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
			ms = 0.0f;
	}
	(void)hipGetLastError();
	(void)hipEventDestroy(e0);
	(void)hipEventDestroy(e1);
	return ms > 0.0f ? 2.0 * bytes / (ms * 1e-3) / 1e9 : 0.0;
}

static void *scratch_on_this_device(void);

extern "C" {

/* *made holds the handle as soon as it exists, so the caller can release it if this throws. */
static anni_adam *create_body(const anni_tensor *tensors, int n_tensors,
	const anni_adam_config *cfg, anni_adam **made)
{
	const size_t big = (size_t)2 << 20;	/* each flat starts on a 2 MiB boundary */
	anni_adam *opt;
	anni_adam_priv *pv;
	Sizes z;
	std::vector<Seg> segs;
	std::vector<int32_t> tile_seg;
	Placement pl;
	int64_t n = 0;
	bool want_split;
	bool ok = false;

	if (!tensors || n_tensors <= 0 || !cfg || !device_ready())
		return nullptr;
	(void)release_idle_pools();	/* the search for the arena's second half looks at what is free */
	if (cfg->grad_type < ANNI_F32 || cfg->grad_type > ANNI_FP8_E4M3
	    || (cfg->moment_type != ANNI_F32 && cfg->moment_type != ANNI_BF16)
	    || cfg->grad_slots < 0 || cfg->grad_slots > 4096
	    || cfg->layout < ANNI_LAYOUT_AUTO || cfg->layout > ANNI_LAYOUT_SPLIT)
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
	*made = opt;
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
			segs[(size_t)i].flags = tensors[i].flags
			    & (ANNI_T_DECAY | ANNI_T_TWIN | ANNI_T_FP8TWIN);
			segs[(size_t)i].pad = 0;
			pv->offsets[(size_t)i] = at;
			pv->flags[(size_t)i] = tensors[i].flags;
			at += tensors[i].n;
		}
	}
	pv->segs = segs;
	/* Launch table: the tensor that holds the first element of each tile. */
	z.n = n;
	z.n_tensors = n_tensors;
	z.n_tiles = (n + kTile - 1) / kTile;
	z.n_slots = cfg->grad_slots;
	z.p_bytes = (size_t)n * 4;
	z.mv_bytes = (size_t)n * elem_bytes(cfg->moment_type);
	z.tw_bytes = cfg->twins ? (size_t)n * 2 : 0;
	z.g_bytes = round_up((size_t)n * elem_bytes(cfg->grad_type), big);
	pv->z = z;
	tile_seg.resize((size_t)z.n_tiles);
	{
		int s = 0;

		for (int64_t k = 0; k < z.n_tiles; k++) {
			while (segs[(size_t)s].end <= k * kTile)
				s++;
			tile_seg[(size_t)k] = s;
		}
	}
	if (!hip_ok(hipHostMalloc((void **)&pv->h_state, sizeof(StepState), hipHostMallocDefault),
	    "arena hipHostMalloc")) {
		(void)hipGetLastError();
		*made = nullptr;
		anni_adam_free(&opt);
		return nullptr;
	}
	memset(pv->h_state, 0, sizeof(StepState));
	if (cfg->grad_type == ANNI_FP8_E4M3)
		(void)scratch_on_this_device();	/* set-up of anni_adam_quantize_grads_static on this device */

	/*
	** AUTO splits arenas whose parameter flat has 256 MiB or more (smaller ones are not
	** bandwidth critical, and their probe launches would be too short to tell placements apart).
	*/
	want_split = cfg->layout == ANNI_LAYOUT_SPLIT
	    || (cfg->layout == ANNI_LAYOUT_AUTO && z.p_bytes >= kPlaceMin);
	if (want_split && place(z, true, &pl)) {
		adopt(opt, z, pl);
		if (init_contents(opt, z, pl, segs, tile_seg)) {
			ok = true;
			/* the update's throughput on the whole arena, for the record */
			if (z.n_slots > 0 && z.p_bytes >= kPlaceMin) {
				pl.gbps = probe(opt);
				pv->probe_gbps = pl.gbps;
			}
		} else {
			unplace(&pl);
			pv->arena = nullptr;
			pv->arena2 = nullptr;
		}
	}
	if (!ok && cfg->layout != ANNI_LAYOUT_SPLIT) {
		if (place(z, false, &pl)) {
			adopt(opt, z, pl);
			ok = init_contents(opt, z, pl, segs, tile_seg);
			if (!ok) {
				unplace(&pl);
				pv->arena = nullptr;
			} else if (z.n_slots > 0 && z.p_bytes >= kPlaceMin) {
				pl.gbps = probe(opt);
				pv->probe_gbps = pl.gbps;
			}
		}
	}
	if (!ok) {
		(void)hip_ok(hipErrorOutOfMemory, "arena hipMalloc");
		*made = nullptr;
		anni_adam_free(&opt);
		return nullptr;
	}
	return opt;
}

void anni_adam_free(anni_adam **popt);

/* No C++ exception (a failed host allocation) crosses the C boundary: the answer is NULL / -1. */
anni_adam *anni_adam_create(const anni_tensor *tensors, int n_tensors,
	const anni_adam_config *cfg)
{
	anni_adam *made = nullptr;

	try {
		return create_body(tensors, n_tensors, cfg, &made);
	} catch (...) {
		anni_adam_free(&made);
		return nullptr;
	}
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
		if (opt->priv->mv_apart) {
			gpu_free(opt->d_m);
			gpu_free(opt->d_v);
		}
		if (opt->priv->h_m)
			(void)hip_ok(hipHostFree(opt->priv->h_m), "offload hipHostFree");
		if (opt->priv->h_v)
			(void)hip_ok(hipHostFree(opt->priv->h_v), "offload hipHostFree");
		if (opt->priv->arena)
			(void)hip_ok(hipFree(opt->priv->arena), "arena hipFree");
		if (opt->priv->arena2)
			(void)hip_ok(hipFree(opt->priv->arena2), "arena hipFree");
		if (opt->priv->derived && opt->priv->derived_owned)
			(void)hip_ok(hipFree(opt->priv->derived), "derived hipFree");
		if (opt->priv->gq_scratch)
			(void)hip_ok(hipFree(opt->priv->gq_scratch), "quantizer hipFree");
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
	opt->d_grad = d_grad ? d_grad : (void *)opt->priv->grad_slots;
	return opt->d_grad ? 0 : -1;
}

void *anni_adam_grad_slot(const anni_adam *opt, int k)
{
	if (!opt || !opt->priv || k < 0 || k >= opt->priv->n_grad_slots)
		return nullptr;
	return opt->priv->grad_slots + (size_t)k * opt->priv->grad_slot_bytes;
}

int anni_adam_is_split(const anni_adam *opt)
{
	return opt && opt->priv ? opt->priv->split : 0;
}

double anni_adam_apart_ratio(const anni_adam *opt)
{
	return opt && opt->priv ? opt->priv->apart_ratio : 0.0;
}

size_t anni_adam_arena_bytes(const anni_adam *opt)
{
	return opt && opt->priv ? opt->priv->arena_bytes : 0;
}

size_t anni_adam_resident_bytes(const anni_adam *opt)
{
	return opt && opt->priv ? opt->priv->resident_bytes : 0;
}

double anni_adam_probe_gbps(const anni_adam *opt)
{
	return opt && opt->priv ? opt->priv->probe_gbps : 0.0;
}

int anni_adam_placement_cost(const anni_adam *opt, double *walked_gib, double *ms)
{
	if (!opt || !opt->priv)
		return -1;
	if (walked_gib)
		*walked_gib = opt->priv->search.walked_gib;
	if (ms)
		*ms = opt->priv->search.ms;
	return opt->priv->search.timed;
}

static void describe(const anni_adam *opt, Flat *f);

/* The derived outputs as the update would leave them, straight from p. */
static int derive_now(anni_adam *opt)
{
	anni_adam_priv *pv = opt->priv;
	hipStream_t st = compute_stream();
	Flat f;

	describe(opt, &f);
	if (pv->fp8_twins && launch_fill_bytes(st, pv->d_wamax, 0,
	    (size_t)opt->n_tensors * sizeof(uint32_t)) != 0)
		return -1;
	if (launch_derive(st, f) != 0)
		return -1;
	if (pv->fp8_twins) {
		if (launch_amax_fold(st, f, nullptr) != 0)
			return -1;
		if (launch_fp8_twins(st, f, (uint8_t *)opt->d_param_fp8, opt->d_wscale, pv->d_wamax,
		    opt->n_tensors, nullptr) != 0)
			return -1;
	}
	return 0;
}

int anni_adam_seed_twins(anni_adam *opt)
{
	if (!opt || !opt->priv || (!opt->d_param_bf16 && !opt->priv->derived))
		return -1;
	if (opt->d_param_bf16 && launch_f32_to_bf16(compute_stream(),
	    (uint16_t *)opt->d_param_bf16, opt->d_param, opt->n) != 0)
		return -1;
	return opt->priv->derived ? derive_now(opt) : 0;
}

static int enable_derived_body(anni_adam *opt, const anni_pack *packs, int n_packs,
	int64_t pack_elems)
{
	anni_adam_priv *pv;
	hipStream_t st;
	std::vector<PackDesc> descs;
	std::vector<Seg> segs;
	std::vector<float> ones;
	size_t off_q, off_scale, off_amax, off_packs, off_tamax, off_pack, total;
	char *base;
	bool fp8 = false;

	if (!opt || !opt->priv || opt->priv->derived || n_packs < 0 || (n_packs > 0 && !packs)
	    || pack_elems < 0 || (n_packs > 0 && pack_elems <= 0) || !device_ready())
		return -1;
	pv = opt->priv;
	segs = pv->segs;
	descs.assign((size_t)opt->n_tensors, PackDesc{0, 1u, 0u});
	for (int i = 0; i < opt->n_tensors; i++)
		if (segs[(size_t)i].flags & kSegFp8Twin)
			fp8 = true;
	for (int k = 0; k < n_packs; k++) {
		const anni_pack &pk = packs[k];
		int64_t cnt, rows;

		if (pk.tensor < 0 || pk.tensor >= opt->n_tensors || pk.cols <= 0
		    || pk.dst_stride < pk.cols || pk.dst_offset < 0)
			return -1;
		if (segs[(size_t)pk.tensor].flags & kSegPack)
			return -1;		/* one target per tensor */
		cnt = segs[(size_t)pk.tensor].end - segs[(size_t)pk.tensor].begin;
		if (cnt <= 0 || cnt >= ((int64_t)1 << 32) || cnt % pk.cols != 0)
			return -1;
		rows = cnt / pk.cols;
		if (pk.dst_offset + (rows - 1) * (int64_t)pk.dst_stride + pk.cols > pack_elems)
			return -1;
		descs[(size_t)pk.tensor].dst_off = pk.dst_offset;
		descs[(size_t)pk.tensor].cols = (uint32_t)pk.cols;
		descs[(size_t)pk.tensor].dst_stride = (uint32_t)pk.dst_stride;
		segs[(size_t)pk.tensor].flags |= kSegPack;
	}
	if (!fp8 && n_packs == 0)
		return -1;		/* nothing to derive */
	off_q = 0;
	off_scale = round_up(fp8 ? (size_t)opt->n : 0, 256);
	off_amax = off_scale + round_up((size_t)opt->n_tensors * sizeof(float), 256);
	off_packs = off_amax + round_up((size_t)opt->n_tensors * sizeof(uint32_t), 256);
	off_tamax = round_up(off_packs + (size_t)opt->n_tensors * sizeof(PackDesc), 256);
	off_pack = round_up(off_tamax + (fp8 ? (size_t)((opt->n + kTile - 1) / kTile) * kWaves
	    * sizeof(float) : 0), (size_t)2 << 20);
	total = off_pack + round_up((size_t)pack_elems * 2, 256) + 256;
	if (device_alloc(&pv->derived, total) != hipSuccess) {
		pv->derived = nullptr;
		return -1;
	} else {
		pv->derived_owned = 1;
	}
	base = (char *)pv->derived;
	st = compute_stream();
	ones.assign((size_t)opt->n_tensors, 1.0f);
	pv->d_wamax = (uint32_t *)(base + off_amax);
	pv->d_packs = (PackDesc *)(base + off_packs);
	pv->d_tile_amax = fp8 ? (float *)(base + off_tamax) : nullptr;
	pv->fp8_twins = fp8 ? 1 : 0;
	if (launch_fill_bytes(st, base, 0, total) != 0
	    || !hip_ok(hipMemcpyAsync(base + off_scale, ones.data(),
	    (size_t)opt->n_tensors * sizeof(float), hipMemcpyHostToDevice, st), "wscale")
	    || !hip_ok(hipMemcpyAsync(pv->d_packs, descs.data(),
	    (size_t)opt->n_tensors * sizeof(PackDesc), hipMemcpyHostToDevice, st), "packs")
	    || !hip_ok(hipMemcpyAsync(pv->d_segs, segs.data(), (size_t)opt->n_tensors * sizeof(Seg),
	    hipMemcpyHostToDevice, st), "segs")
	    || !hip_ok(hipStreamSynchronize(st), "derived init")) {
		if (pv->derived_owned)
			(void)hipFree(pv->derived);
		pv->derived = nullptr;
		return -1;
	}
	pv->segs = segs;
	opt->d_param_fp8 = fp8 ? base + off_q : nullptr;
	opt->d_wscale = (float *)(base + off_scale);
	opt->d_pack_bf16 = n_packs ? base + off_pack : nullptr;
	return 0;
}

int anni_adam_enable_derived(anni_adam *opt, const anni_pack *packs, int n_packs,
	int64_t pack_elems)
{
	try {
		return enable_derived_body(opt, packs, n_packs, pack_elems);
	} catch (...) {
		return -1;
	}
}

int anni_adam_zero_grad(anni_adam *opt)
{
	if (!opt || !opt->d_grad)
		return -1;
	return launch_fill_bytes(compute_stream(), opt->d_grad, 0,
	    (size_t)opt->n * elem_bytes(opt->cfg.grad_type));
}

/*
** The passes that keep the E4M3 weight twins, pointed at the gradients and at every tensor:
** maxima of whole tiles per wavefront (tiles shared by tensors raise the tensors' words
** directly), folded into one word per tensor, then scale_t = max(amax_t / 448, 1e-12) and
** q = E4M3(x * (1 / scale_t)) -- the arithmetic of anni_fp8_quantize on each tensor.  `work` holds
** one word per tensor (cleared here, on the stream) and, 256-byte aligned behind them, the tile
** maxima (every one that is read was written by this call).
*/
static int quantize_grads_into(anni_adam *opt, const float *d_src, void *work)
{
	anni_adam_priv *pv = opt->priv;
	hipStream_t st = compute_stream();
	const size_t amax_bytes = round_up((size_t)opt->n_tensors * sizeof(uint32_t), 256);
	Flat f;

	memset(&f, 0, sizeof(f));
	f.p = const_cast<float *>(d_src);
	f.n = opt->n;
	f.segs = pv->d_segs;
	f.tile_seg = pv->d_tile_seg;
	f.der.wamax = (uint32_t *)work;
	f.der.tile_amax = (float *)((char *)work + amax_bytes);
	if (launch_fill_bytes(st, f.der.wamax, 0, (size_t)opt->n_tensors * sizeof(uint32_t)) != 0
	    || launch_derive(st, f, 0u) != 0
	    || launch_amax_fold(st, f, nullptr, 0u) != 0
	    || launch_fp8_twins(st, f, (uint8_t *)opt->d_grad, opt->d_gscale, f.der.wamax,
	    opt->n_tensors, nullptr, 0u) != 0)
		return -1;
	return 0;
}

int anni_adam_quantize_grads(anni_adam *opt, const float *d_src)
{
	anni_adam_priv *pv;

	if (!opt || !opt->priv || !d_src || !opt->d_grad || !opt->d_gscale || !device_ready()
	    || opt->cfg.grad_type != ANNI_FP8_E4M3 || ((uintptr_t)d_src & 15) != 0)
		return -1;
	pv = opt->priv;
	if (!pv->gq_scratch) {
		const size_t n_tiles = (size_t)((opt->n + kTile - 1) / kTile);
		const size_t amax_bytes = round_up((size_t)opt->n_tensors * sizeof(uint32_t), 256);
		void *d = nullptr;

		if (!hip_ok(device_alloc(&d, amax_bytes + n_tiles * kWaves * sizeof(float)),
		    "quantizer hipMalloc"))
			return -1;
		pv->gq_scratch = d;
	}
	return quantize_grads_into(opt, d_src, pv->gq_scratch);
}

/*
** The same without any allocation: the work area is a fixed array in device memory that every
** GPU the library runs on holds from the moment the library is loaded until the process ends.
*/
static __device__ __align__(256) unsigned char scratch[ANNI_QUANT_STATIC_BYTES];

static const int kScratchDevices = 64;
static void *g_scratch_ptr[kScratchDevices];	/* the array's address on each device (the name itself is no device address) */
static std::mutex g_scratch_mu;

/* The address of `scratch` on the current device, looked up once per device; NULL on failure. */
static void *scratch_on_this_device(void)
{
	int dev = -1;
	void *ptr = nullptr;

	if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchDevices) {
		(void)hipGetLastError();
		return nullptr;
	}
	std::lock_guard<std::mutex> lk(g_scratch_mu);

	if (g_scratch_ptr[dev])
		return g_scratch_ptr[dev];
	if (!hip_ok(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) {
		(void)hipGetLastError();
		return nullptr;
	}
	g_scratch_ptr[dev] = ptr;
	return ptr;
}

int anni_adam_quantize_grads_static(anni_adam *opt, const float *d_src)
{
	void *work;
	size_t need;

	if (!opt || !opt->priv || !d_src || !opt->d_grad || !opt->d_gscale || !device_ready()
	    || opt->cfg.grad_type != ANNI_FP8_E4M3 || ((uintptr_t)d_src & 15) != 0)
		return -1;
	need = round_up((size_t)opt->n_tensors * sizeof(uint32_t), 256)
	    + (size_t)((opt->n + kTile - 1) / kTile) * kWaves * sizeof(float);
	if (opt->n > ANNI_QUANT_STATIC_MAX_ELEMS || opt->n_tensors > ANNI_QUANT_STATIC_MAX_TENSORS
	    || need > sizeof(scratch)) {
		(void)hip_ok(hipErrorInvalidValue, "anni_adam_quantize_grads_static: more than "
		    "ANNI_QUANT_STATIC_MAX_ELEMS elements or ANNI_QUANT_STATIC_MAX_TENSORS tensors");
		return -1;
	}
	work = scratch_on_this_device();
	if (!work)
		return -1;
	return quantize_grads_into(opt, d_src, work);
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
	if (pv->derived) {
		f->der.wamax = pv->fp8_twins ? pv->d_wamax : nullptr;
		f->der.tile_amax = pv->d_tile_amax;
		f->der.packs = pv->d_packs;
		f->der.pack = (uint16_t *)opt->d_pack_bf16;
	}
}

/* The ticket counters of the norm's second stage lie behind the step state (reserved and zeroed with it). */
static unsigned int *ticket_word(const anni_adam_priv *pv)
{
	static_assert(sizeof(StepState) <= 128, "the tickets start 128 bytes behind the state");
	return (unsigned int *)((char *)pv->d_state + 128);
}

/*
** One step; ev (may be NULL) = four events recorded before the step, after the sum of squares, after
** the update and after the derived outputs; an entry that is NULL is not recorded.
*/
/* ---- m and v off the device between steps (lm_adam.c:211-214,295-334) ----------------------- */

/*
** The reference can park the moments on the host between steps (lm_adam_set_offload): after a
** step adam_offload_mv reads d_m and d_v back and frees them, the next step allocates and uploads
** them again -- two of the five flats leave the device while forward and backward need the room.
** Here m and v normally are parts of the arena's two blocks, which cannot be freed piecemeal, so
** the first anni_adam_set_offload(opt, 1) re-houses the arena: m and v move into blocks of
** their own (gpu_malloc: its pools keep the emptied chunks, so taking the blocks again costs
** nothing and gpu_mem_info reads the same before and after every step), everything else into
** two new blocks without room for them.  While the moments are away opt->d_m and opt->d_v are
** NULL; their homes are two page-locked host buffers, raw copies of the stored type.
*/
static int mv_bring(anni_adam *opt)
{
	anni_adam_priv *pv = opt->priv;
	hipStream_t st;

	if (opt->d_m && opt->d_v)
		return 0;
	if (!pv->mv_apart || !pv->h_m || !pv->h_v)
		return -1;
	opt->d_m = gpu_malloc(pv->z.mv_bytes);
	opt->d_v = gpu_malloc(pv->z.mv_bytes);
	if (!opt->d_m || !opt->d_v) {
		gpu_free(opt->d_m);
		gpu_free(opt->d_v);
		opt->d_m = opt->d_v = nullptr;
		return -1;
	}
	st = compute_stream();
	if (!hip_ok(hipMemcpyAsync(opt->d_m, pv->h_m, pv->z.mv_bytes, hipMemcpyHostToDevice, st), "offload h2d")
	    || !hip_ok(hipMemcpyAsync(opt->d_v, pv->h_v, pv->z.mv_bytes, hipMemcpyHostToDevice, st), "offload h2d")) {
		/* the host copies stay the valid ones: nothing half-filled may pass for the moments */
		(void)sync_stream_and_deliver();
		gpu_free(opt->d_m);
		gpu_free(opt->d_v);
		opt->d_m = opt->d_v = nullptr;
		return -1;
	}
	return 0;
}

static int mv_send(anni_adam *opt)
{
	anni_adam_priv *pv = opt->priv;
	hipStream_t st;

	if (!opt->d_m || !opt->d_v)
		return 0;
	if (!pv->mv_apart || !pv->h_m || !pv->h_v)
		return -1;
	st = compute_stream();
	if (!hip_ok(hipMemcpyAsync(pv->h_m, opt->d_m, pv->z.mv_bytes, hipMemcpyDeviceToHost, st), "offload d2h")
	    || !hip_ok(hipMemcpyAsync(pv->h_v, opt->d_v, pv->z.mv_bytes, hipMemcpyDeviceToHost, st), "offload d2h")
	    || !hip_ok(sync_stream_and_deliver(), "offload sync"))
		return -1;
	gpu_free(opt->d_m);
	gpu_free(opt->d_v);
	opt->d_m = opt->d_v = nullptr;
	return 0;
}

/* Runs `work` with the moments on the device: offloaded ones are brought back for it and sent away again. */
template <typename F>
static int with_moments(anni_adam *opt, F work)
{
	int rc;

	if (mv_bring(opt) != 0)
		return -1;
	rc = work();
	if (opt->priv->offload && mv_send(opt) != 0)
		rc = -1;
	return rc;
}

/* Moves m and v into blocks of their own and everything else into two new blocks without them. */
static int rehouse_without_mv(anni_adam *opt)
{
	anni_adam_priv *pv = opt->priv;
	hipStream_t st = compute_stream();
	Sizes z = pv->z;
	Placement pl;
	void *m2, *v2;
	char *old_a = (char *)pv->arena;
	char *old_b = (char *)pv->arena2;
	const float *old_gscale = (const float *)((char *)pv->d_segs
	    - round_up((size_t)z.n_tensors * sizeof(float), 256));
	const bool own_gscale = opt->d_gscale == old_gscale;
	const size_t slots_bytes = (size_t)z.n_slots * z.g_bytes;
	const size_t tables = tables_bytes(z);
	long bound_slot = -1;
	bool ok;

	if (!hip_ok(sync_stream_and_deliver(), "offload sync"))
		return -1;
	if (pv->grad_slots && (char *)opt->d_grad >= pv->grad_slots
	    && (char *)opt->d_grad < pv->grad_slots + slots_bytes)
		bound_slot = (long)(((char *)opt->d_grad - pv->grad_slots) / (long)pv->grad_slot_bytes);
	m2 = gpu_malloc(z.mv_bytes);
	v2 = gpu_malloc(z.mv_bytes);
	z.mv_bytes = 0;			/* the new blocks have no room for the moments */
	if (!m2 || !v2 || !place(z, pv->split != 0, &pl)) {
		gpu_free(m2);
		gpu_free(v2);
		return -1;
	}
	{
		char *second = pl.b ? pl.b : pl.a;
		char *old_second = old_b ? old_b : old_a;

		ok = hip_ok(hipMemcpyAsync(m2, opt->d_m, pv->z.mv_bytes, hipMemcpyDeviceToDevice, st), "rehouse")
		    && hip_ok(hipMemcpyAsync(v2, opt->d_v, pv->z.mv_bytes, hipMemcpyDeviceToDevice, st), "rehouse")
		    && hip_ok(hipMemcpyAsync(pl.a + pl.off_p, opt->d_param, z.p_bytes, hipMemcpyDeviceToDevice, st), "rehouse")
		    /* the tables, the partials and the step state lie in one run behind the per-tensor scales */
		    && hip_ok(hipMemcpyAsync(pl.a + pl.off_gscale, old_gscale, tables, hipMemcpyDeviceToDevice, st), "rehouse")
		    && (!z.tw_bytes || hip_ok(hipMemcpyAsync(second + pl.off_twin, opt->d_param_bf16, z.tw_bytes,
		    hipMemcpyDeviceToDevice, st), "rehouse"))
		    && (!slots_bytes || hip_ok(hipMemcpyAsync(second + pl.off_g, pv->grad_slots, slots_bytes,
		    hipMemcpyDeviceToDevice, st), "rehouse"))
		    && hip_ok(hipStreamSynchronize(st), "rehouse sync");
		(void)old_second;
	}
	if (!ok) {
		unplace(&pl);
		gpu_free(m2);
		gpu_free(v2);
		return -1;
	}
	{
		void *ext_grad = bound_slot < 0 ? opt->d_grad : nullptr;
		float *ext_gscale = own_gscale ? nullptr : opt->d_gscale;
		const size_t real_mv = pv->z.mv_bytes;

		adopt(opt, z, pl);
		pv->z.mv_bytes = real_mv;
		pv->resident_bytes += 2 * real_mv;
		opt->d_m = m2;
		opt->d_v = v2;
		pv->mv_apart = 1;
		if (bound_slot >= 0)
			opt->d_grad = pv->grad_slots + (size_t)bound_slot * pv->grad_slot_bytes;
		else
			opt->d_grad = ext_grad;
		if (ext_gscale)
			opt->d_gscale = ext_gscale;
	}
	(void)hip_ok(hipFree(old_a), "arena hipFree");
	if (old_b)
		(void)hip_ok(hipFree(old_b), "arena hipFree");
	return 0;
}

extern "C" int anni_adam_set_offload(anni_adam *opt, int on)
{
	anni_adam_priv *pv;

	if (!opt || !opt->priv || !device_ready())
		return -1;
	pv = opt->priv;
	if (!on) {
		pv->offload = 0;
		return pv->mv_apart ? mv_bring(opt) : 0;
	}
	try {
		if (!pv->h_m && !hip_ok(hipHostMalloc(&pv->h_m, pv->z.mv_bytes, hipHostMallocDefault),
		    "offload hipHostMalloc")) {
			(void)hipGetLastError();
			pv->h_m = nullptr;
			return -1;
		}
		if (!pv->h_v && !hip_ok(hipHostMalloc(&pv->h_v, pv->z.mv_bytes, hipHostMallocDefault),
		    "offload hipHostMalloc")) {
			(void)hipGetLastError();
			pv->h_v = nullptr;
			return -1;
		}
		if (!pv->mv_apart && rehouse_without_mv(opt) != 0)
			return -1;
	} catch (...) {
		return -1;
	}
	pv->offload = 1;
	return mv_send(opt);
}

extern "C" int anni_adam_mv_on_device(const anni_adam *opt)
{
	return opt && opt->d_m && opt->d_v ? 1 : 0;
}

/* ANN_GNORM_EVERY=N (lm_adam.c:438-450): the gradient norm is computed, and printed every N steps, also when nothing clips. */
static int gnorm_every(void)
{
	static int every = -1;

	if (every < 0) {
		const char *e = getenv("ANN_GNORM_EVERY");

		every = e ? atoi(e) : 0;
		if (every < 0)
			every = 0;
	}
	return every;
}

static int mv_bring(anni_adam *opt);
static int mv_send(anni_adam *opt);

static int step_impl(anni_adam *opt, double lr, double grad_scale, hipEvent_t *ev)
{
	anni_adam_priv *pv;
	hipStream_t st;
	StepConsts c;
	NormIn norm;
	Flat f;
	int np = 0;
	int t;
	int slot;

	if (!opt || !opt->priv)
		return -1;
	if (lr <= 0.0)
		return 1;			/* lm_adam.c:531-532: t is not advanced */
	if (!opt->d_grad || !device_ready())
		return -1;
	pv = opt->priv;
	if (mv_bring(opt) != 0)			/* offloaded moments come back first (lm_adam.c:295-307) */
		return -1;
	st = compute_stream();
	t = opt->t + 1;				/* lm_adam.c:533; kept only when the step was launched */
	c.bc1 = 1.0 - pow(opt->beta1, (double)t);	/* lm_adam.c:571-572 */
	c.bc2 = 1.0 - pow(opt->beta2, (double)t);
	if (c.bc1 <= 0.0 || c.bc2 <= 0.0)
		return -1;			/* gpu_cuda.cu:8681-8682 */
	c.rbc1 = 1.0 / c.bc1;
	c.rbc2 = 1.0 / c.bc2;
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
	/* lm_adam.c:466: the norm is wanted for the clip, for the skip, or just to be printed */
	norm.use_norm = (opt->grad_clip > 0.0 || opt->cfg.skip_nonfinite || gnorm_every() > 0) ? 1 : 0;
	norm.state = pv->d_state;
	if (ev && ev[0])
		(void)hipEventRecord(ev[0], st);
	if (norm.use_norm) {
		SumsqFinish fin;
		int rc;

		fin.ticket = ticket_word(pv);
		fin.clip = opt->grad_clip > 0.0 ? opt->grad_clip : 0.0;
		fin.skip_nonfinite = opt->cfg.skip_nonfinite;
		fin.state = pv->d_state;
		slot = prof_begin(kProfSumsq, st);
		rc = launch_sumsq(st, f, grad_scale, pv->d_partials, &np, &fin);
		prof_end(slot, st);
		if (rc != 0)
			return -1;
	}
	if (ev && ev[1])
		(void)hipEventRecord(ev[1], st);
	/*
	** The words the update raises start every step at zero, cleared on the stream by a fill
	** kernel (not a memset node, and no state kept on the host: the step can be recorded into a
	** graph and replayed).
	*/
	if (pv->fp8_twins && launch_fill_bytes(st, pv->d_wamax, 0,
	    (size_t)opt->n_tensors * sizeof(uint32_t)) != 0)
		return -1;
	slot = prof_begin(kProfUpdate, st);
	if (launch_update(st, f, c, grad_scale, norm) != 0)
		return -1;
	prof_end(slot, st);
	opt->t = t;
	if (ev && ev[2])
		(void)hipEventRecord(ev[2], st);
	if (pv->fp8_twins) {
		slot = prof_begin(kProfDerived, st);
		if (launch_amax_fold(st, f, norm.use_norm ? pv->d_state : nullptr) != 0)
			return -1;
		if (launch_fp8_twins(st, f, (uint8_t *)opt->d_param_fp8, opt->d_wscale, pv->d_wamax,
		    opt->n_tensors, norm.use_norm ? pv->d_state : nullptr) != 0)
			return -1;
		prof_end(slot, st);
	}
	if (ev && ev[3])
		(void)hipEventRecord(ev[3], st);
	/*
	** The weights moved: consumers that cache derived copies keyed on the weight epoch rebuild
	** them (lm_adam.c:541-547 does this after every device step, a skipped one included).
	*/
	gpu_half_wt_invalidate(nullptr);
	if (pv->offload && mv_send(opt) != 0)	/* lm_adam.c:508-510 */
		return -1;
	if (prof_on())
		gpu_op_prof_dump();		/* lm_adam.c:541 */
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
	    || !hip_ok(sync_stream_and_deliver(), "stats sync"))
		return -1;
	opt->last_sumsq = pv->h_state->sumsq;
	opt->last_grad_norm = pv->h_state->norm;
	opt->last_grad_scale = pv->h_state->grad_scale;
	opt->last_skipped = pv->h_state->skipped;
	opt->last_clipped = pv->h_state->clipped;
	/*
	** The reference's messages for the step just read back (lm_adam.c:479-487), once per step:
	** a skipped step always, the norm every ANN_GNORM_EVERY steps.  The step itself never waits
	** for the host, so they appear when the caller asks for the numbers.
	*/
	if (pv->logged_t != opt->t
	    && (opt->grad_clip > 0.0 || opt->cfg.skip_nonfinite || gnorm_every() > 0)) {
		const int every = gnorm_every();

		pv->logged_t = opt->t;
		if (opt->last_skipped)
			fprintf(stderr, "[adam] step %d skipped: grad norm %g\n", opt->t, opt->last_grad_norm);
		else if (every > 0 && opt->t % every == 0)
			fprintf(stderr, "[adam] step %d grad norm %.4g%s\n", opt->t, opt->last_grad_norm,
			    opt->last_clipped ? " (clipped)" : "");
	}
	return 0;
}

/* ---- optimizer block of a checkpoint (lang/lm_serialize.c:263-331,526-587) ----------- */

/* Slots per staging round: the reference's ADAM_CHUNK (lm_serialize.c:261), 16 MiB of pairs. */
static const int64_t kCkptChunk = (int64_t)1 << 21;

/*
** Two page-locked + two device staging buffers of one chunk each and an event per buffer, for
** the lifetime of one call.
*/
struct CkptStage {
	float		*host[2];
	float		*dev[2];
	hipEvent_t	ev[2];
	bool		have_ev[2];

	CkptStage() : host{nullptr, nullptr}, dev{nullptr, nullptr}, ev{}, have_ev{false, false} {}
	bool init(void)
	{
		const size_t bytes = (size_t)kCkptChunk * 2 * sizeof(float);

		for (int i = 0; i < 2; i++) {
			if (hipHostMalloc((void **)&host[i], bytes, hipHostMallocDefault) != hipSuccess
			    || device_alloc((void **)&dev[i], bytes) != hipSuccess
			    || hipEventCreateWithFlags(&ev[i], hipEventDisableTiming) != hipSuccess) {
				(void)hipGetLastError();
				return false;
			}
			have_ev[i] = true;
		}
		return true;
	}
	~CkptStage()
	{
		for (int i = 0; i < 2; i++) {
			if (have_ev[i])
				(void)hipEventDestroy(ev[i]);
			if (host[i])
				(void)hipHostFree(host[i]);
			if (dev[i])
				(void)hipFree(dev[i]);
		}
	}
};

/* Where exported pairs go / imported pairs come from: a host array or a file descriptor. */
struct PairIo {
	float	*mem;		/* NULL: use fd */
	int	fd;
};

static int write_all(int fd, const void *buf, size_t n);
static int read_all(int fd, void *buf, size_t n);

/*
** Slots [first, first + count) as (m, v) pairs, chunk by chunk: while the host consumes chunk k
** out of one page-locked buffer (a copy into the caller's array, or write(2) straight from the
** buffer) the device interleaves chunk k + 1 and sends it into the other.
*/
static int export_pairs(anni_adam *opt, int64_t first, int64_t count, const PairIo &io)
{
	hipStream_t st;
	CkptStage sg;
	const int64_t n_chunks = (count + kCkptChunk - 1) / kCkptChunk;

	if (count == 0)
		return 0;
	if (!sg.init())
		return -1;
	st = compute_stream();
	for (int64_t k = -1; k < n_chunks; k++) {
		if (k + 1 < n_chunks) {		/* issue chunk k + 1 */
			const int64_t at = (k + 1) * kCkptChunk;
			const int64_t c = count - at < kCkptChunk ? count - at : kCkptChunk;
			const int b = (int)((k + 1) & 1);

			if (launch_mv_interleave(st, sg.dev[b], opt->d_m, opt->d_v, opt->cfg.moment_type,
			    first + at, c) != 0
			    || !hip_ok(hipMemcpyAsync(sg.host[b], sg.dev[b], (size_t)c * 2 * sizeof(float),
			    hipMemcpyDeviceToHost, st), "export d2h")
			    || !hip_ok(hipEventRecord(sg.ev[b], st), "export event")) {
				(void)hipStreamSynchronize(st);
				return -1;
			}
		}
		if (k >= 0) {			/* consume chunk k */
			const int64_t at = k * kCkptChunk;
			const int64_t c = count - at < kCkptChunk ? count - at : kCkptChunk;
			const int b = (int)(k & 1);
			const size_t bytes = (size_t)c * 2 * sizeof(float);

			if (!hip_ok(hipEventSynchronize(sg.ev[b]), "export wait")) {
				(void)hipStreamSynchronize(st);
				return -1;
			}
			if (io.mem)
				memcpy(io.mem + 2 * at, sg.host[b], bytes);
			else if (write_all(io.fd, sg.host[b], bytes) != 0) {
				(void)hipStreamSynchronize(st);
				return -1;
			}
		}
	}
	return 0;
}

/* The other way: the host fills one page-locked buffer while the device scatters the other. */
static int import_pairs(anni_adam *opt, int64_t first, int64_t count, const PairIo &io)
{
	hipStream_t st;
	CkptStage sg;
	int rc = 0;

	if (count == 0)
		return 0;
	if (!sg.init())
		return -1;
	st = compute_stream();
	for (int64_t at = 0, k = 0; at < count && rc == 0; at += kCkptChunk, k++) {
		const int64_t c = count - at < kCkptChunk ? count - at : kCkptChunk;
		const int b = (int)(k & 1);
		const size_t bytes = (size_t)c * 2 * sizeof(float);

		/* buffer b was last used two chunks ago: its upload must be over before it is refilled */
		if (k >= 2 && !hip_ok(hipEventSynchronize(sg.ev[b]), "import wait"))
			rc = -1;
		if (rc == 0) {
			if (io.mem)
				memcpy(sg.host[b], io.mem + 2 * at, bytes);
			else if (read_all(io.fd, sg.host[b], bytes) != 0)
				rc = -1;
		}
		if (rc == 0 && (!hip_ok(hipMemcpyAsync(sg.dev[b], sg.host[b], bytes, hipMemcpyHostToDevice,
		    st), "import h2d")
		    || launch_mv_deinterleave(st, opt->d_m, opt->d_v, opt->cfg.moment_type, sg.dev[b],
		    first + at, c) != 0
		    || !hip_ok(hipEventRecord(sg.ev[b], st), "import event")))
			rc = -1;
	}
	if (!hip_ok(sync_stream_and_deliver(), "import sync"))
		rc = -1;
	return rc;
}

int anni_adam_export_mv(anni_adam *opt, int64_t first, int64_t count, float *pairs)
{
	PairIo io;

	if (!opt || !opt->priv || !pairs || first < 0 || count < 0 || first + count > opt->n
	    || !device_ready())
		return -1;
	io.mem = pairs;
	io.fd = -1;
	return with_moments(opt, [&] { return export_pairs(opt, first, count, io); });
}

int anni_adam_import_mv(anni_adam *opt, int64_t first, int64_t count, const float *pairs)
{
	PairIo io;

	if (!opt || !opt->priv || !pairs || first < 0 || count < 0 || first + count > opt->n
	    || !device_ready())
		return -1;
	io.mem = const_cast<float *>(pairs);
	io.fd = -1;
	return with_moments(opt, [&] { return import_pairs(opt, first, count, io); });
}

static int write_all(int fd, const void *buf, size_t n)
{
	const char *p = (const char *)buf;

	while (n > 0) {
		const ssize_t w = write(fd, p, n);

		if (w <= 0)
			return -1;
		p += w;
		n -= (size_t)w;
	}
	return 0;
}

static int read_all(int fd, void *buf, size_t n)
{
	char *p = (char *)buf;

	while (n > 0) {
		const ssize_t r = read(fd, p, n);

		if (r <= 0)
			return -1;
		p += r;
		n -= (size_t)r;
	}
	return 0;
}

int anni_adam_write_state(anni_adam *opt, int fd, int epoch, int step)
{
	int32_t head[5];
	PairIo io;

	if (!opt || !opt->priv || fd < 0 || opt->n > INT32_MAX || !device_ready())
		return -1;
	head[0] = 1;			/* lm_serialize.c:319-321: has_adam, epoch, step, t, n */
	head[1] = epoch;
	head[2] = step;
	head[3] = opt->t;
	head[4] = (int32_t)opt->n;
	if (write_all(fd, head, sizeof(head)) != 0)
		return -1;
	io.mem = nullptr;
	io.fd = fd;
	return with_moments(opt, [&] { return export_pairs(opt, 0, opt->n, io); });	/* write(2) straight from the page-locked buffers */
}

int anni_adam_read_state(anni_adam *opt, int fd, int *epoch, int *step)
{
	int32_t head[5];
	PairIo io;

	if (!opt || !opt->priv || fd < 0 || !device_ready())
		return -1;
	if (read_all(fd, head, sizeof(head)) != 0 || head[0] != 1 || head[4] != opt->n)
		return -1;		/* lm_serialize.c:546-562: has_adam == 1 and the same slot count */
	io.mem = nullptr;
	io.fd = fd;
	if (with_moments(opt, [&] { return import_pairs(opt, 0, opt->n, io); }) != 0)
		return -1;		/* a short file: the moments read so far are in place, t is not */
	opt->t = head[3];		/* so the learning-rate schedule continues (lm_serialize.c:564) */
	if (epoch)
		*epoch = head[1];
	if (step)
		*step = head[2];
	return 0;
}

/* ---- learning-rate schedule (lang/lm_train.c:98-124,398-411) ------------------ */

static int g_warmup_steps;
static int g_decay_steps;
static int g_decay_kind;	/* 0 none, 1 linear, 2 cosine (any other name: cosine, as the reference) */
static int g_sched_from;
static double g_lr_override;	/* the lr field of the reference's train_control (lm_train.c:104-105); <= 0: none */

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

void anni_lr_set_override(double lr)
{
	g_lr_override = lr;
}

double anni_lr_step(double base_lr, int step)
{
	double q;
	int u;

	if (g_lr_override > 0.0)
		return g_lr_override;		/* lm_train.c:104-105 */
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

void anni_gpu_flush(void)
{
	if (device_ready())
		(void)compute_stream();		/* launches the pending batch of small copies, if any */
}

/* ---- what libanni_bench.so needs from inside this library (anni_hooks.h) ------------------ */

int anni_hook_step_events(anni_adam *opt, double lr, double grad_scale, void *const events[4])
{
	return step_impl(opt, lr, grad_scale, (hipEvent_t *)events);
}

void anni_hook_reload_switches(void)
{
	reload_switches();
}

long anni_hook_counter(const char *name)
{
	int runs = 0, bad = 0;
	long used = 0, dropped = 0;

	if (!name)
		return -1;
	fold_guard_stats(&runs, &bad);
	early_sum_stats(&used, &dropped);
	if (strcmp(name, "fold_guard_runs") == 0)
		return runs;
	if (strcmp(name, "fold_guard_mismatches") == 0)
		return bad;
	if (strcmp(name, "early_sum_used") == 0)
		return used;
	if (strcmp(name, "early_sum_dropped") == 0)
		return dropped;
	if (strcmp(name, "second_stream") == 0)
		return second_stream_state();
	if (strcmp(name, "vectors_first_steps") == 0 || strcmp(name, "vectors_first_served") == 0) {
		long steps = 0, served = 0;

		vectors_first_stats(&steps, &served);
		return strcmp(name, "vectors_first_steps") == 0 ? steps : served;
	}
	return -1;
}

int anni_gpu_device_info(char *name, size_t cap, int *driver_version)
{
	hipDeviceProp_t prop;
	int dev = 0;

	if (!device_ready() || !name || cap == 0 || hipGetDevice(&dev) != hipSuccess
	    || hipGetDeviceProperties(&prop, dev) != hipSuccess)
		return -1;
	snprintf(name, cap, "%s (%s)", prop.name[0] ? prop.name : "AMD GPU", prop.gcnArchName);
	if (driver_version && hipDriverGetVersion(driver_version) != hipSuccess)
		*driver_version = 0;
	return 0;
}

} /* extern "C" */

/*
** Internal C++ interface between the C-ABI entry points and the gfx950 kernels
** of the optimizer step.  Not installed; the public surface is the headers under include/.
**
** Work decomposition.  The flat of n elements is cut into tiles of kTile
** elements counted from the start of the flat (not from the start of a
** tensor), so vector accesses are aligned whenever the flat's base pointers
** are.  A launch table maps each tile to the tensor that holds its first
** element; a tile that lies wholly inside one tensor runs the 16-byte vector
** path with that tensor's attributes held in scalars, a tile that crosses a
** tensor boundary (or the ragged end of the flat) runs an element-wise path
** that looks the tensor up per element.  One launch therefore covers every
** tensor, however small, and the long tail of bias / LayerNorm vectors costs
** no extra launches.
*/
#ifndef ANNI_ADAM_KERNELS_H__
#define ANNI_ADAM_KERNELS_H__

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "adam_math.h"

namespace anni {

enum { kF32 = 0, kBF16 = 1, kFP8 = 2 };

constexpr int kThreads = 256;			/* four 64-lane wavefronts */
constexpr int kQuad = 4;			/* elements per lane per access */
constexpr int kTile = 4096;			/* elements per tile */
constexpr int kQuadsPerTile = kTile / (kThreads * kQuad);	/* 4 */
constexpr int kWaves = kThreads / 64;
constexpr int kMaxPartials = 8192;		/* upper bound on the sum-of-squares grid */

constexpr uint32_t kSegDecay = 1u;		/* decoupled weight decay applies */
constexpr uint32_t kSegTwin = 2u;		/* bf16 twin is written */
constexpr uint32_t kSegFp8Twin = 4u;		/* E4M3 twin with a per-tensor scale is kept current */
constexpr uint32_t kSegPack = 8u;		/* bf16 of the tensor also goes into a packed matrix */

/* One tensor of the flat: elements [begin, end). */
struct Seg {
	int64_t		begin;
	int64_t		end;
	uint32_t	flags;
	uint32_t	pad;
};

/*
** Where the bf16 of a row-major matrix of `cols` columns also goes: element (r, c) lands at
** pack[dst_off + r * dst_stride + c] (the [Wq | Wk | Wv] operand of num/gpu_cuda.cu:6456-6470).
*/
struct PackDesc {
	int64_t		dst_off;
	uint32_t	cols;
	uint32_t	dst_stride;
};

/*
** Outputs derived from the new weights in the same pass (all NULL: none).  Max |p| of the
** tensors flagged kSegFp8Twin: every wavefront leaves the maximum of its quarter of a whole tile
** in tile_amax[tile * kWaves + wave] (a plain store; tens of thousands of wavefronts raising
** one word per tensor were measured to cost the update 3-7 %), the few elements of tiles that
** straddle tensors raise wamax[s] directly (the caller clears wamax on the stream before
** every launch_update / launch_derive), and launch_amax_fold folds the tile maxima into wamax.  A maximum does not depend on the order, so the result is deterministic.
*/
struct Derived {
	uint32_t	*wamax;
	float		*tile_amax;	/* kWaves floats per tile of the flat */
	const PackDesc	*packs;		/* one per tensor, read for tensors flagged kSegPack */
	uint16_t	*pack;
};

/* Written by the step on the device; read back only when the host asks. */
struct StepState {
	double	sumsq;
	double	norm;
	double	grad_scale;	/* after the clip factor */
	int	skipped;
	int	clipped;
};

/* The arrays and launch table one launch works on (all device pointers). */
struct Flat {
	float		*p;
	void		*g;
	void		*m;
	void		*v;
	uint16_t	*twin;		/* may be NULL */
	int64_t		n;
	int		grad_type;
	int		moment_type;
	const Seg	*segs;		/* NULL: one tensor with uniform_flags */
	const int32_t	*tile_seg;	/* NULL when segs is NULL */
	const float	*gscale;	/* per-tensor dequant scale (fp8 gradients) */
	uint32_t	uniform_flags;
	Derived		der;
};

/* How the update obtains the global norm (use_norm == 0: grad_scale is final). */
/* The update takes its gradient scale and its skip decision from *state (use_norm) or from its arguments. */
struct NormIn {
	int		use_norm;
	const StepState	*state;		/* stored by launch_sumsq with a SumsqFinish on the same stream */
};

/*
** Ticket counters of the norm's second stage: one per group of workgroups and one above them,
** each on a 128-byte line of its own.  kTicketBytes of device memory, zero between launches, one
** block per partials array.
*/
constexpr int kTicketGroups = 64;
constexpr int kTicketStride = 32;		/* in words */
constexpr size_t kTicketBytes = (size_t)(1 + kTicketGroups) * kTicketStride * sizeof(unsigned int);

/* Second stage of the norm inside the sum-of-squares launch. */
struct SumsqFinish {
	unsigned int	*ticket;	/* kTicketBytes, 128-byte aligned */
	double		clip;		/* > 0: norm > clip scales the gradients by clip / (norm + 1e-12) */
	int		skip_nonfinite;
	StepState	*state;		/* device or page-locked host memory */
};

/* Reads the ANNI_* tuning switches from the environment again (they are read once, on first use). */
void	reload_switches(void);

/* How often the self-check of launch_sumsq's second stage has run in this process, and how often its two forms disagreed. */
void	fold_guard_stats(int *runs, int *mismatches);

/* Workgroups of a resident grid for a flat of n elements on the current device. */
int	grid_for(int64_t n);

/*
** partials[0..*n_partials) = per-workgroup sums of (g * grad_scale)^2, fixed order.  With `fin`
** the last workgroup to finish also folds them in index order into fin->state = {sum, sqrt,
** clip-adjusted scale, flags}.  The first such call on a device (and the first after
** reload_switches) launches the sum twice more and waits for the stream once: the self-check of
** the second stage (adam_kernels.hip, fold_guard); every other call is asynchronous.
*/
int	launch_sumsq(hipStream_t st, const Flat &f, double grad_scale, double *partials,
		int *n_partials, const SumsqFinish *fin);
int	launch_update(hipStream_t st, const Flat &f, const StepConsts &c, double grad_scale,
		const NormIn &norm);
/*
** The same update for the tiles (kTile elements each) order[0 .. turns) only, in that order;
** `order` is device memory.  Two such launches over disjoint tiles may run side by side.  -1 when
** the storage mode would take a software-pipelined kernel, which has no such form.
*/
int	update_walks_backwards(void);	/* launch_update takes the tiles from the last to the first */
int	launch_update_tiles(hipStream_t st, const Flat &f, const StepConsts &c, double grad_scale,
		const NormIn &norm, const int32_t *order, int64_t turns);
/*
** The sum of squares of a float flat in separable steps (the flat entry point gpu_grad_sumsq):
** launch_chunk_sums writes one partial sum for every 16 KiB chunk of x (list == NULL) or for
** the n_list chunks named in `list` (device-readable memory) into part[chunk];
** launch_chunk_fold adds all chunk_sums_count(n) partials in index order, through at most
** kChunkRuns intermediate sums (of kChunkPer partials or a power of two times that) in `runs`,
** and stores {sum, sqrt(sum), 1, 0, 0} into *state.
** The sum is a function of x alone: partials recomputed for some chunks after their elements
** changed give the bits a pass over the whole flat would.
*/
constexpr size_t kSumChunkBytes = 16384;	/* a chunk; callers that track rewritten chunks count in these */
constexpr int kChunkRuns = 1024;
constexpr int kChunkPer = 512;		/* two partials per lane of the workgroup that folds a run */
int	chunk_sums_count(int64_t n);
int	launch_chunk_sums(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *list,
		int n_list, int beside);	/* beside != 0: other kernels run at the same time, leave them room */
int	launch_chunk_fold(hipStream_t st, const double *part, int64_t n, double *runs, StepState *state);
/*
** The end of the sum in one launch: the partials of the n_fix chunks in `fix` (rising, no chunk
** twice; host memory, `fix_dev` the same list where the device can read it) are computed anew,
** then everything is folded as launch_chunk_fold does, with the same bits.  ticket: kTicketBytes
** of zeroed device memory, 128-byte aligned, left zeroed.  The first call per device checks the
** one launch against the separate kernels and waits for the stream once; calls must not overlap.
** stamp (may be NULL; page-locked host memory): receives `token` after *state has been stored, for
** a host that would rather watch a word than wait for the stream.  Returns 0 when the stamp will
** be written, 1 when the launch went the way of the separate kernels, which write none, -1 on error.
*/
int	launch_chunk_finish(hipStream_t st, const float *x, int64_t n, double *part, const int32_t *fix,
		const int32_t *fix_dev, int n_fix, double *runs, unsigned int *ticket, StepState *state,
		unsigned long long *stamp, unsigned long long token);
/*
** Derived outputs straight from p, without an update (after weights were loaded):
** wamax and the packed matrices as the update would leave them.
*/
int	launch_derive(hipStream_t st, const Flat &f, uint32_t need = kSegFp8Twin);
/*
** wamax[s] = max(wamax[s], tile maxima of tensor s) for the flagged tensors, after
** launch_update or launch_derive on the same stream.  state (may be NULL): nothing to do
** after a skipped step.
*/
int	launch_amax_fold(hipStream_t st, const Flat &f, const StepState *state,
		uint32_t need = kSegFp8Twin);
/*
** q = E4M3(p * (1 / scale_s)) for the tensors flagged `need` (0: every tensor), scale_s from
** wamax[s] (num/gpu_cuda.cu:826-851,927-938); wscale[s] receives the scale.  state (may be
** NULL): a skipped step leaves q and wscale alone.
*/
int	launch_fp8_twins(hipStream_t st, const Flat &f, uint8_t *q, float *wscale,
		const uint32_t *wamax, int n_tensors, const StepState *state,
		uint32_t need = kSegFp8Twin);
int	launch_f32_to_bf16(hipStream_t st, uint16_t *dst, const float *src, int64_t n);
/* pairs[2k] = m[first+k], pairs[2k+1] = v[first+k] as floats (bf16 moments widen exactly). */
int	launch_mv_interleave(hipStream_t st, float *pairs, const void *m, const void *v,
		int moment_type, int64_t first, int64_t count);
/* The inverse: m[first+k] = pairs[2k], v[first+k] = pairs[2k+1] (bf16 moments: round to nearest even). */
int	launch_mv_deinterleave(hipStream_t st, void *m, void *v, int moment_type, const float *pairs,
		int64_t first, int64_t count);
int	launch_fill_bytes(hipStream_t st, void *dst, int value, size_t nbytes);

} /* namespace anni */
#endif

/*
** anni_bench.h -- libanni_bench.so: what measures and tests libanni_gpu_hip.so.  Event-timed
** step loops, synthetic input generators, a calibration copy kernel, re-reading of the tuning
** switches.  A library of its own, linked against libanni_gpu_hip.so: a training program links
** only the latter (anni_gpu.h, anni_adam.h); bench.py and the tests load both.  None of these has
** a counterpart in the reference.
*/
#ifndef ANNI_BENCH_H__
#define ANNI_BENCH_H__

#include <stddef.h>
#include <stdint.h>
#include "anni_adam.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
** Times `count` back-to-back steps with HIP events recorded on the compute
** stream: per step, the gradient flat grads[i % n_grads] is bound (NULL array =
** keep the bound one), lr[i] and grad_scale[i] are used.  ms_total receives the
** elapsed time of the whole run, ms_sumsq / ms_update (may be NULL) the summed
** durations of the two kernels.  Allocates nothing on the device.
*/
int	anni_adam_time_steps(anni_adam *opt, int count, void *const *grads, int n_grads,
		const double *lr, const double *grad_scale, float *ms_total,
		float *ms_sumsq, float *ms_update);
/* Summed duration of the E4M3 twin launches of the last anni_adam_time_steps run that asked for per-kernel times. */
float	anni_adam_timed_derived_ms(const anni_adam *opt);

/* x[i] = mean + std * N(0,1), counter-based (seed, stream, i): same values for any launch shape. */
int	anni_fill_normal_f32(float *d_x, int64_t n, uint64_t seed, uint64_t stream,
		float mean, float std);
/* Plain 16-byte-vector copy kernel of nbytes (a multiple of 16, 16-byte aligned): reads and writes exactly nbytes. */
int	anni_copy_bytes(void *d_dst, const void *d_src, size_t nbytes);
/*
** The same copy in the shape of the update kernel (one workgroup per 16 KiB, four 16-byte words
** per lane in flight, as many workgroups as pieces); nontemporal != 0 uses non-temporal loads and
** stores.  For `bench.py --ceilings`: what a copy shaped like the update reaches on this device.
*/
int	anni_copy_bytes_tiled(void *d_dst, const void *d_src, size_t nbytes, int nontemporal);
/*
** Reads the kernels' tuning switches (ANNI_TILES_PER_WG, ANNI_KEEP_MB, ANNI_REVERSE, ANNI_PIPE,
** ANNI_NT, ANNI_BLOCKS_PER_CU) from the environment again; without this call they are read once,
** on first use.  For sweeps that compare settings on one arena inside one process (two
** processes differ by the memory they were given, by more than most settings do); results never
** depend on the switches.
*/
void	anni_gpu_reload_switches(void);
/*
** The sum of squares checks its second stage against a conservative form of itself at its first
** launch on a device and again after anni_gpu_reload_switches (two extra launches, one wait):
** how often that check has run in this process and how often the two forms disagreed (then the
** process has gone over to the conservative form and said so on stderr).  Returns 0.
*/
int	anni_fold_guard_stats(int *runs, int *mismatches);
/*
** gpu_grad_sumsq may begin its sum before it is called, when the caller has shown the pattern of
** lang/lm_adam.c twice in a row (small uploads of vectors, then the sum of the same flat): how
** often such an early sum was used by the call that followed, and how often it had to be thrown
** away because something else had gone onto the stream or another flat was named.  Returns 0.
*/
int	anni_early_sum_stats(long *used, long *dropped);
/*
** gpu_adam_step_dev_bf16 may update the tiles that hold the caller's bias / LayerNorm vectors in a
** launch of their own and copy those vectors out ahead of the rest, when the caller has read the
** same list of small ranges back after two updates in a row (lang/lm_adam.c:407-413): the steps
** in which read-backs were served that way, and how many read-backs.  Returns 0.
*/
int	anni_vectors_first_stats(long *steps, long *served);
/*
** Both of the above need a stream whose kernels run beside those of the compute stream; which of
** the runtime's streams do is measured when the first of them is about to be used.  -1: not
** looked for yet, 0: none found (then neither ever happens), 1: found.
*/
int	anni_second_stream_state(void);

#ifdef __cplusplus
}
#endif
#endif

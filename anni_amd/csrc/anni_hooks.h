/*
** Private to this source tree: the three entry points libanni_gpu_hip.so exports for
** libanni_bench.so (the measuring and testing utilities of include/anni_bench.h), which lives in a
** library of its own so that the product library carries nothing a training program does not
** call.  Not installed, not part of the ABI a caller may rely on.
*/
#ifndef ANNI_HOOKS_H__
#define ANNI_HOOKS_H__

#include "anni_adam.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
** anni_adam_step_scaled with up to four HIP events (hipEvent_t, NULL = not recorded) recorded on
** the compute stream: before the step, after the sum of squares, after the update, after the
** derived outputs.
*/
int	anni_hook_step_events(anni_adam *opt, double lr, double grad_scale, void *const events[4]);
/* Reads the ANNI_* tuning switches from the environment again; the next sum of squares re-runs its self-check. */
void	anni_hook_reload_switches(void);
/*
** Counters the library keeps for the record, by name; -1 for a name it does not know:
**   "fold_guard_runs", "fold_guard_mismatches"   the self-check of the arena's sum of squares
**   "early_sum_used", "early_sum_dropped"        gpu_grad_sumsq's sum begun early, taken / thrown away
*/
long	anni_hook_counter(const char *name);

#ifdef __cplusplus
}
#endif
#endif

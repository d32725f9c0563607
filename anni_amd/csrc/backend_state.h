/*
** State shared by the C-ABI translation units of libanni_gpu_hip.so: the one
** in-order compute stream every operation is issued on (the reference's g_st,
** num/gpu_cuda.cu:36-44) and a couple of helpers.
*/
#ifndef ANNI_BACKEND_STATE_H__
#define ANNI_BACKEND_STATE_H__

#include <hip/hip_runtime.h>

namespace anni {

/* True once a device is present and the compute stream exists. */
bool		device_ready(void);
hipStream_t	compute_stream(void);
/*
** Puts the pending batch of small copies on the stream, waits for the stream and hands the
** batched device-to-host copies to their destinations: what every synchronisation inside the
** library must do, so that a small gpu_memcpy_d2h_async is complete after ANY of them.
*/
hipError_t	sync_stream_and_deliver(void);
/* NULL restores the library's own stream. */
void		set_compute_stream(hipStream_t st);
/* Remembers the first HIP error for gpu_debug_last_error; returns err == hipSuccess. */
bool		hip_ok(hipError_t err, const char *what);
/*
** gpu_malloc keeps the chunks of its two pools reserved after the last block in them was freed;
** this gives the empty ones back to the driver (true when there was one).  Called before other
** large reservations.
*/
bool		release_idle_pools(void);
/*
** hipMalloc for the library's own blocks (scratch, derived outputs, staging): when the driver
** has nothing left, the empty chunks of gpu_malloc's pools are given back and the request is
** made once more.  *p is NULL on failure; the error is cleared.
*/
hipError_t	device_alloc(void **p, size_t nbytes);

/* How often the sum of squares begun early (gpu_backend.hip) was used by the call that followed, and how often dropped. */
void		early_sum_stats(long *used, long *dropped);
/* Steps whose small read-backs were served by a split update (gpu_backend.hip, "the vectors first"), and how many read-backs. */
void		vectors_first_stats(long *steps, long *served);
/* The search for a stream that runs beside the compute stream: -1 not made yet, 0 none found, 1 found. */
int		second_stream_state(void);

/*
** ANN_OP_PROF=1 (num/gpu_cuda.cu:3205-3409): an event pair around an operation of the optimizer
** step, summed per kind and printed by gpu_op_prof_dump.  prof_begin records the first event on
** `st` and returns the pair's slot (-1: profiling is off), prof_end records the second.
*/
enum { kProfSumsq = 0, kProfUpdate = 1, kProfDerived = 2, kProfKinds = 3 };
bool		prof_on(void);
int		prof_begin(int kind, hipStream_t st);
void		prof_end(int slot, hipStream_t st);

} /* namespace anni */
#endif

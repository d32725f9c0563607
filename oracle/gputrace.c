/*
** An interposer that timestamps the backend calls of one optimizer step.  TEST INFRASTRUCTURE
** ONLY: built into oracle/_ref/libgputrace.so and linked IN FRONT of libanni_gpu_hip.so into the
** "_trace" flavours of the compiled reference (see Makefile), so that the unchanged
** lang/lm_adam.c binds its gpu_* calls here; every call is forwarded to the real library
** (named by the environment variable ANNI_HIP_SO) and its start and end are recorded.  bench.py
** --reference-caller-only --call-trace prints the timeline: where the host spends the step
** between the kernels.  Costs two clock reads per call (about 40 ns).
*/
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

enum { F_DEVSYNC, F_AVAIL, F_H2D, F_SUMSQ, F_SETWD, F_STEP, F_PIN, F_D2HA, F_SSYNC, F_PROF, F_INVAL,
	F_MEMSET, F_D2H, F_N };
static const char *names[F_N] = { "gpu_device_sync", "gpu_available", "gpu_memcpy_h2d",
	"gpu_grad_sumsq", "gpu_adam_set_weight_decay", "gpu_adam_step_dev_bf16", "gpu_host_pin",
	"gpu_memcpy_d2h_async", "gpu_stream_sync", "gpu_op_prof_dump", "gpu_half_wt_invalidate",
	"gpu_memset", "gpu_memcpy_d2h" };
#define MAX_EVENTS (1 << 16)
typedef struct {
	int	id;
	double	t0;
	double	t1;
	size_t	bytes;
} event;
static event ev[MAX_EVENTS];
static int nev;
static int recording;
static void *real_lib;

static double now_us(void)
{
	struct timespec ts;

	clock_gettime(CLOCK_MONOTONIC, &ts);
	return (double)ts.tv_sec * 1e6 + (double)ts.tv_nsec * 1e-3;
}

static void *real(const char *name)
{
	void *s;

	if (!real_lib) {
		const char *path = getenv("ANNI_HIP_SO");

		real_lib = path ? dlopen(path, RTLD_NOW) : NULL;
		if (!real_lib) {
			fprintf(stderr, "gputrace: cannot open ANNI_HIP_SO=%s: %s\n", path ? path : "(unset)",
			    dlerror());
			abort();
		}
	}
	s = dlsym(real_lib, name);
	if (!s) {
		fprintf(stderr, "gputrace: %s not found\n", name);
		abort();
	}
	return s;
}

#define RECORD(which, nbytes, call) \
	do { \
		const double t0_ = now_us(); \
		call; \
		if (recording && nev < MAX_EVENTS) { \
			ev[nev].id = which; \
			ev[nev].t0 = t0_; \
			ev[nev].t1 = now_us(); \
			ev[nev].bytes = nbytes; \
			nev++; \
		} \
	} while (0)

void gputrace_start(void) { nev = 0; recording = 1; }
void gputrace_stop(void) { recording = 0; }
int gputrace_count(void) { return nev; }
const char *gputrace_name(int id) { return id >= 0 && id < F_N ? names[id] : "?"; }
void gputrace_get(int i, int *id, double *t0, double *t1, size_t *bytes)
{
	*id = ev[i].id;
	*t0 = ev[i].t0;
	*t1 = ev[i].t1;
	*bytes = ev[i].bytes;
}

void gpu_device_sync(void)
{
	static void (*f)(void);

	if (!f)
		f = (void (*)(void))real("gpu_device_sync");
	RECORD(F_DEVSYNC, 0, f());
}

int gpu_available(void)
{
	static int (*f)(void);
	int r;

	if (!f)
		f = (int (*)(void))real("gpu_available");
	RECORD(F_AVAIL, 0, r = f());
	return r;
}

int gpu_memcpy_h2d(void *d, const void *s, size_t n)
{
	static int (*f)(void *, const void *, size_t);
	int r;

	if (!f)
		f = (int (*)(void *, const void *, size_t))real("gpu_memcpy_h2d");
	RECORD(F_H2D, n, r = f(d, s, n));
	return r;
}

int gpu_grad_sumsq(const float *x, int n, double *out)
{
	static int (*f)(const float *, int, double *);
	int r;

	if (!f)
		f = (int (*)(const float *, int, double *))real("gpu_grad_sumsq");
	RECORD(F_SUMSQ, 0, r = f(x, n, out));
	return r;
}

void gpu_adam_set_weight_decay(double wd)
{
	static void (*f)(double);

	if (!f)
		f = (void (*)(double))real("gpu_adam_set_weight_decay");
	RECORD(F_SETWD, 0, f(wd));
}

int gpu_adam_step_dev_bf16(float *p, void *tw, float *g, float *m, float *v, int n, double lr,
	double b1, double b2, double eps, int t, double gs)
{
	static int (*f)(float *, void *, float *, float *, float *, int, double, double, double, double,
	    int, double);
	int r;

	if (!f)
		f = (int (*)(float *, void *, float *, float *, float *, int, double, double, double,
		    double, int, double))real("gpu_adam_step_dev_bf16");
	RECORD(F_STEP, 0, r = f(p, tw, g, m, v, n, lr, b1, b2, eps, t, gs));
	return r;
}

int gpu_host_pin(void *p, size_t n)
{
	static int (*f)(void *, size_t);
	int r;

	if (!f)
		f = (int (*)(void *, size_t))real("gpu_host_pin");
	RECORD(F_PIN, n, r = f(p, n));
	return r;
}

int gpu_memcpy_d2h_async(void *d, const void *s, size_t n)
{
	static int (*f)(void *, const void *, size_t);
	int r;

	if (!f)
		f = (int (*)(void *, const void *, size_t))real("gpu_memcpy_d2h_async");
	RECORD(F_D2HA, n, r = f(d, s, n));
	return r;
}

int gpu_stream_sync(void)
{
	static int (*f)(void);
	int r;

	if (!f)
		f = (int (*)(void))real("gpu_stream_sync");
	RECORD(F_SSYNC, 0, r = f());
	return r;
}

void gpu_op_prof_dump(void)
{
	static void (*f)(void);

	if (!f)
		f = (void (*)(void))real("gpu_op_prof_dump");
	RECORD(F_PROF, 0, f());
}

void gpu_half_wt_invalidate(const float *p)
{
	static void (*f)(const float *);

	if (!f)
		f = (void (*)(const float *))real("gpu_half_wt_invalidate");
	RECORD(F_INVAL, 0, f(p));
}

int gpu_memset(void *d, int v, size_t n)
{
	static int (*f)(void *, int, size_t);
	int r;

	if (!f)
		f = (int (*)(void *, int, size_t))real("gpu_memset");
	RECORD(F_MEMSET, n, r = f(d, v, n));
	return r;
}

int gpu_memcpy_d2h(void *d, const void *s, size_t n)
{
	static int (*f)(void *, const void *, size_t);
	int r;

	if (!f)
		f = (int (*)(void *, const void *, size_t))real("gpu_memcpy_d2h");
	RECORD(F_D2H, n, r = f(d, s, n));
	return r;
}

/*
** Placement of large blocks over the sections of device memory, found by timing the update
** on scratch flats (see placement.h).  No counterpart in the reference.
*/
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <chrono>
#include <vector>
#include "adam_kernels.h"
#include "backend_state.h"
#include "placement.h"

namespace anni {

static const int64_t kProbeElems = (int64_t)64 << 20;	/* 0.34 ms per launch; shorter launches tell less */
static const int64_t kProbeMinElems = (int64_t)8 << 20;
static const size_t kProbeEvery = (size_t)8 << 30;	/* a block is timed about every 8 GiB of blocks */
static const size_t kSection = (size_t)96 << 30;	/* the walk crosses a section boundary within one section's worth of blocks */
static const double kApartRatio = 1.07;			/* measured 1.13 - 1.17 across a section boundary */

/*
** Milliseconds per launch of the all-f32 update over n elements of zero state (which it leaves
** zero): p, m at a0 and a0 + 4n; v, g, twin at b0, b0 + 4n, b0 + 8n.  0 on failure.
*/
static double probe_ms(char *a0, char *b0, int64_t n)
{
	hipStream_t st = compute_stream();
	hipEvent_t e0, e1;
	StepConsts c;
	NormIn norm;
	Flat f;
	float ms = 0.0f;
	const int reps = 3;

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
	memset(&f, 0, sizeof(f));
	f.p = (float *)a0;
	f.m = a0 + 4 * n;
	f.v = b0;
	f.g = b0 + 4 * n;
	f.twin = (uint16_t *)(b0 + 8 * n);
	f.n = n;
	f.grad_type = kF32;
	f.moment_type = kF32;
	f.uniform_flags = kSegTwin;
	if (hipEventCreate(&e0) != hipSuccess)
		return 0.0;
	if (hipEventCreate(&e1) != hipSuccess) {
		(void)hipEventDestroy(e0);
		return 0.0;
	}
	if (launch_update(st, f, c, 1.0, norm) == 0) {
		(void)hipEventRecord(e0, st);
		for (int i = 0; i < reps; i++)
			(void)launch_update(st, f, c, 1.0, norm);
		(void)hipEventRecord(e1, st);
		if (hipStreamSynchronize(st) != hipSuccess
		    || hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
			ms = 0.0f;
	}
	(void)hipGetLastError();
	(void)hipEventDestroy(e0);
	(void)hipEventDestroy(e1);
	return (double)ms / reps;
}

/* ANNI_PLACE_LOG=1: one line per candidate on stderr. */
static bool place_log(void)
{
	static int on = -1;

	if (on < 0) {
		const char *e = getenv("ANNI_PLACE_LOG");

		on = (e && e[0] == '1') ? 1 : 0;
	}
	return on == 1;
}

/*
** How far the walk may go: one section and one block, or ANNI_PLACE_MAX_GIB GiB when that is set
** (0 = no walk, the first block is taken).
*/
static size_t walk_max(size_t bytes)
{
	static long gib = -2;

	if (gib == -2) {
		const char *e = getenv("ANNI_PLACE_MAX_GIB");

		gib = e && *e ? atol(e) : -1;
		if (gib < -1 || gib > 1024)
			gib = -1;
	}
	return gib >= 0 ? (size_t)gib << 30 : kSection + bytes;
}

static size_t free_bytes_now(size_t *total)
{
	size_t fr = 0, tt = 0;

	if (hipMemGetInfo(&fr, &tt) != hipSuccess) {
		(void)hipGetLastError();
		fr = 0;
		tt = 0;
	}
	if (total)
		*total = tt;
	return fr;
}

void *alloc_apart_from(void *ref, size_t ref_bytes, size_t bytes, double *ratio, PlaceStats *stats)
{
	hipStream_t st = compute_stream();
	const auto t_begin = std::chrono::steady_clock::now();
	std::vector<void *> blocks;
	size_t walked = 0;
	size_t total = 0;
	int timed = 0;
	double t_same = 0.0;
	double best_ratio = 0.0;
	int best = -1;
	int64_t n;

	if (ratio)
		*ratio = 1.0;
	if (stats)
		memset(stats, 0, sizeof(*stats));
	/* probe size: 18 bytes per element inside ref and inside a candidate (for the one-block timings) */
	n = kProbeElems;
	if ((size_t)n * 18 > ref_bytes)
		n = (int64_t)(ref_bytes / 18);
	if ((size_t)n * 18 > bytes)
		n = (int64_t)(bytes / 18);
	n = n / kTile * kTile;
	if (!ref || n < kProbeMinElems) {
		void *p = nullptr;

		if (hipMalloc(&p, bytes) != hipSuccess) {
			(void)hipGetLastError();
			return nullptr;
		}
		if (stats)
			stats->walked_gib = (double)bytes / 1073741824.0;
		return p;
	}
	const size_t free_at_entry = free_bytes_now(&total);
	const size_t margin = total / 20 > ((size_t)8 << 30) ? total / 20 : ((size_t)8 << 30);
	/* never more than half of what is free now: others allocate while this runs */
	const size_t limit = walk_max(bytes) < free_at_entry / 2 ? walk_max(bytes) : free_at_entry / 2;
	/*
	** The walk: blocks of `bytes` are requested one after the other and kept, so the allocator
	** works its way down through device memory; about every 8 GiB one of them is timed.  The
	** blocks in between are ballast of the SAME size as the candidates on purpose: requests of
	** one size fill the gaps the allocator has in the order it would fill them for the
	** candidates too, whereas large aligned ballast leaves gaps near the top in which small
	** candidates then all end up (seen with 1.5 GiB candidates and 16 GiB ballast: eight
	** candidates, 112 GiB walked, none of them out of the first section).
	*/
	const size_t every = bytes >= kProbeEvery ? 1 : (kProbeEvery + bytes - 1) / bytes;

	if (launch_fill_bytes(st, ref, 0, (size_t)n * 18) != 0)
		return nullptr;
	for (size_t it = 0; it == 0 || walked + bytes <= limit; it++) {
		void *c = nullptr;
		double t_pair;

		if (it > 0 && free_bytes_now(nullptr) < bytes + margin)
			break;
		if (hipMalloc(&c, bytes) != hipSuccess) {
			(void)hipGetLastError();
			break;
		}
		blocks.push_back(c);
		walked += bytes;
		if (it % every != 0)
			continue;
		if (launch_fill_bytes(st, c, 0, (size_t)n * 18) != 0)
			break;
		if (it == 0) {
			/*
			** All five flats in one block, timed inside `ref` and inside the first candidate:
			** the slower of the two is the reference.  (A block that the driver pieced together
			** from memory of several sections -- it does so when it reuses freed memory -- is
			** fast by itself and would make every pair look no better than "one block".)
			*/
			const double t_ref = probe_ms((char *)ref + 10 * n, (char *)ref, n);
			const double t_c = probe_ms((char *)c + 10 * n, (char *)c, n);

			t_same = t_ref > t_c ? t_ref : t_c;
			if (t_ref <= 0.0 || t_c <= 0.0)
				break;
		}
		t_pair = probe_ms((char *)ref, (char *)c, n);
		if (t_pair <= 0.0)
			break;
		timed++;
		if (place_log())
			fprintf(stderr, "[place] block %zu at %p (%.2f GiB): one block %.4f ms, with ref %p %.4f ms, "
			    "ratio %.3f, walked %.0f GiB, free %.1f GiB\n", it, c, (double)bytes / 1073741824.0,
			    t_same, ref, t_pair, t_same / t_pair, (double)walked / 1073741824.0,
			    (double)free_bytes_now(nullptr) / 1073741824.0);
		if (best < 0 || t_same / t_pair > best_ratio) {
			best = (int)it;
			best_ratio = t_same / t_pair;
		}
		if (best_ratio >= kApartRatio)
			break;
	}
	(void)hipStreamSynchronize(st);
	if (best < 0 && !blocks.empty())
		best = 0;
	for (size_t i = 0; i < blocks.size(); i++)
		if ((int)i != best)
			(void)hipFree(blocks[i]);
	(void)hipGetLastError();
	if (stats) {
		stats->walked_gib = (double)walked / 1073741824.0;
		stats->ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now()
		    - t_begin).count();
		stats->timed = timed;
	}
	if (place_log())
		fprintf(stderr, "[place] search over: %.1f GiB walked in %zu blocks, %d timed, %.1f ms, best ratio %.3f\n",
		    (double)walked / 1073741824.0, blocks.size(), timed,
		    std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t_begin).count(),
		    best_ratio);
	if (best < 0)
		return nullptr;
	if (ratio && best_ratio > 0.0)
		*ratio = best_ratio;
	return blocks[(size_t)best];
}

} /* namespace anni */

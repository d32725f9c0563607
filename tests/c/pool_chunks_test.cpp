/*
** Host-only exercise of the first-fit chunk bookkeeping behind gpu_malloc's pools
** (anni_amd/csrc/pool_chunks.h): a random sequence of takes and gives checked against a byte map,
** and the invariants after every operation -- blocks sorted, covering the chunk, no two free
** neighbours, live bytes right.  Prints "ok" and the operation counts.
*/
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "pool_chunks.h"

using namespace anni;

static unsigned long long rng_state = 88172645463325252ull;
static unsigned long long rnd(void)
{
	rng_state ^= rng_state << 13;
	rng_state ^= rng_state >> 7;
	rng_state ^= rng_state << 17;
	return rng_state;
}

static void check(const PoolChunk &c, const std::vector<unsigned char> &map)
{
	size_t at = 0, live = 0;

	for (size_t i = 0; i < c.blocks.size(); i++) {
		const PoolBlock &b = c.blocks[i];

		if (b.off != at || b.bytes == 0) { printf("FAIL: block %zu at %zu, expected %zu\n", i, b.off, at); exit(1); }
		if (i > 0 && !b.used && !c.blocks[i - 1].used) { printf("FAIL: free neighbours at %zu\n", b.off); exit(1); }
		for (size_t k = 0; k < b.bytes; k++)
			if ((map[b.off + k] != 0) != b.used) { printf("FAIL: map differs at %zu\n", b.off + k); exit(1); }
		if (b.used)
			live += b.bytes;
		at += b.bytes;
	}
	if (at != c.bytes || live != c.live) { printf("FAIL: cover %zu of %zu, live %zu vs %zu\n", at, c.bytes, live, c.live); exit(1); }
}

int main(void)
{
	const size_t N = 4096;				/* units; the real code hands out multiples of 2 MiB */
	PoolChunk c((char *)0, N, 0);
	std::vector<unsigned char> map(N, 0);
	std::vector<std::pair<size_t, size_t> > held;	/* (offset, bytes) */
	long takes = 0, refused = 0, gives = 0;

	for (int op = 0; op < 20000; op++) {
		if (held.empty() || rnd() % 100 < 55) {
			const size_t need = 1 + rnd() % (op % 7 == 0 ? 1500 : 300);
			const size_t off = c.take(need);
			size_t run = 0, best = 0;

			/* first fit must succeed exactly when the byte map has a free run of `need`, at the first such run */
			size_t first = (size_t)-1;
			for (size_t k = 0; k < N; k++) {
				run = map[k] ? 0 : run + 1;
				if (run > best) best = run;
				if (run >= need && first == (size_t)-1) first = k + 1 - need;
			}
			if ((off == (size_t)-1) != (first == (size_t)-1) || (off != (size_t)-1 && off != first)) {
				printf("FAIL: take(%zu) gave %zu, the map says %zu\n", need, off, first);
				return 1;
			}
			if (off == (size_t)-1) { refused++; continue; }
			memset(&map[off], 1, need);
			held.push_back(std::make_pair(off, need));
			takes++;
		} else {
			const size_t k = rnd() % held.size();

			if (held[k].second > 1 && c.give(held[k].first + 1) != 0) { printf("FAIL: interior pointer accepted\n"); return 1; }
			if (c.give(held[k].first) != held[k].second) { printf("FAIL: give\n"); return 1; }
			if (c.give(held[k].first) != 0) { printf("FAIL: double give accepted\n"); return 1; }
			memset(&map[held[k].first], 0, held[k].second);
			held.erase(held.begin() + (long)k);
			gives++;
		}
		/* now and then: reserve the largest free block whole (what the placement search uses as scratch) and hand it back */
		if (op % 97 == 0) {
			size_t big = 0;
			const size_t at = c.largest_free(&big);

			if (big > 0) {
				if (c.take_block(at + 1) != 0) { printf("FAIL: take_block of an interior offset\n"); return 1; }
				if (c.take_block(at) != big) { printf("FAIL: take_block\n"); return 1; }
				if (c.take_block(at) != 0) { printf("FAIL: take_block of a used block\n"); return 1; }
				memset(&map[at], 1, big);
				check(c, map);
				if (c.give(at) != big) { printf("FAIL: give after take_block\n"); return 1; }
				memset(&map[at], 0, big);
			}
		}
		check(c, map);
	}
	while (!held.empty()) { c.give(held.back().first); held.pop_back(); }
	if (c.blocks.size() != 1 || c.blocks[0].used || c.live != 0) { printf("FAIL: not one free block at the end\n"); return 1; }
	size_t n = 0;
	if (c.largest_free(&n) != 0 || n != N) { printf("FAIL: largest_free\n"); return 1; }
	printf("ok takes %ld refused %ld gives %ld\n", takes, refused, gives);
	return 0;
}

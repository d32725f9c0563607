/*
** Where large blocks of device memory should lie relative to each other.
**
** MI355X's 288 GiB of HBM3E behave as three sections of 96 GiB (consecutive physical
** addresses; a 12-high stack is three ranks of four dies).  A kernel that reads and writes
** several arrays at once -- the update streams nine -- runs about 15 % slower when ALL of its
** arrays lie in one section than when they are split over two or three (5.6 against 6.4 - 6.6
** TB/s for the update; which arrays share a section hardly matters as long as neither side
** holds much more than half of the traffic, and where a block lies INSIDE a section does not
** matter at all).  A kernel with a single stream, or one that only reads, does not care.
**
** Physical addresses cannot be asked for, and the driver's allocator (largest fitting
** power-of-two blocks, highest address first, gaps filled later) does not put consecutive
** requests at predictable places.  So placement is found by measurement: the update is timed on
** scratch flats inside the candidate blocks, against the same launch with all flats in one
** block.  No reference code does this (the reference has one allocation per flat and no notion of placement).
*/
#ifndef ANNI_PLACEMENT_H__
#define ANNI_PLACEMENT_H__

#include <stddef.h>
#include <stdint.h>

namespace anni {

/* Blocks smaller than this are not worth placing (their streams are short). */
constexpr size_t kPlaceMin = (size_t)256 << 20;

/* What a search did, for the record (anni_adam_placement_stats, ANNI_PLACE_LOG=1). */
struct PlaceStats {
	double	walked_gib;	/* device memory requested and held during the walk, the result included */
	double	ms;		/* wall clock of the whole search */
	int	timed;		/* candidates that were timed */
};

/*
** Allocates `bytes` of device memory that streams well together with the block
** [ref, ref + ref_bytes): memory of another section when one can be had.  Blocks of `bytes` are
** requested one after the other and kept (the allocator works its way down through the
** sections), about every 8 GiB one of them is timed against `ref`, until one is at least 7 %
** faster than the same launch inside a single block or the walk has reached its limit; the best
** one is kept, all others are returned.  The limit: one section and one block (96 GiB + `bytes`;
** ANNI_PLACE_MAX_GIB sets another figure, 0 = no walk), and never more than half of what was
** free when the search began, so that the process and its neighbours on the device keep room
** to allocate while it runs.  Both probe areas -- the first 18 bytes per probe element of `ref`
** and of every candidate -- are zero-filled and left zero, so `ref` must not hold data there.
** *ratio (may be NULL) receives time(one block) / time(ref + result), "one block" being the
** slower of `ref` alone and the first candidate alone; 1.0 when nothing was measured.  A ratio
** near 1 with a fast arena happens too: memory the driver reuses after frees is often pieced
** together from several sections already, and then there is nothing left to gain.  NULL when the
** allocation itself fails.  Synchronises the compute stream.  Takes no lock of this library.
*/
void	*alloc_apart_from(void *ref, size_t ref_bytes, size_t bytes, double *ratio,
		PlaceStats *stats = nullptr);

} /* namespace anni */
#endif

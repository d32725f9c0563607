/*
** First-fit blocks inside one chunk of device memory: the bookkeeping of gpu_malloc's two pools
** (gpu_backend.hip), kept free of any device call so that it can be exercised on the host.
** Blocks are sorted by offset and always cover the chunk; neighbours that are both free are
** merged at once, so a chunk all of whose blocks were freed is one free block again.
*/
#ifndef ANNI_POOL_CHUNKS_H__
#define ANNI_POOL_CHUNKS_H__

#include <stddef.h>
#include <vector>

namespace anni {

struct PoolBlock {
	size_t	off;
	size_t	bytes;
	bool	used;
};

struct PoolChunk {
	char			*base;
	size_t			bytes;
	int			pool;
	size_t			live;		/* bytes handed out */
	std::vector<PoolBlock>	blocks;		/* sorted by offset, covering the chunk */

	PoolChunk(char *b, size_t n, int which) : base(b), bytes(n), pool(which), live(0)
	{
		blocks.push_back(PoolBlock{ 0, n, false });
	}

	/* Offset of a block of `need` bytes taken first-fit, or (size_t)-1. */
	size_t take(size_t need)
	{
		for (size_t i = 0; i < blocks.size(); i++) {
			if (blocks[i].used || blocks[i].bytes < need)
				continue;
			if (blocks[i].bytes > need) {
				const PoolBlock rest = { blocks[i].off + need, blocks[i].bytes - need, false };

				blocks[i].bytes = need;
				blocks.insert(blocks.begin() + (long)i + 1, rest);
			}
			blocks[i].used = true;
			live += need;
			return blocks[i].off;
		}
		return (size_t)-1;
	}

	/*
	** Takes the whole free block that starts at `off` (what largest_free reported): its size, or
	** 0 when no free block starts there.  For a reservation that is handed back with give().
	*/
	size_t take_block(size_t off)
	{
		for (size_t i = 0; i < blocks.size(); i++) {
			if (blocks[i].off != off || blocks[i].used)
				continue;
			blocks[i].used = true;
			live += blocks[i].bytes;
			return blocks[i].bytes;
		}
		return 0;
	}

	/* Bytes given back by freeing the live block that starts at `off`; 0 when there is none. */
	size_t give(size_t off)
	{
		for (size_t i = 0; i < blocks.size(); i++) {
			if (blocks[i].off != off || !blocks[i].used)
				continue;
			const size_t n = blocks[i].bytes;

			blocks[i].used = false;
			live -= n;
			if (i + 1 < blocks.size() && !blocks[i + 1].used) {
				blocks[i].bytes += blocks[i + 1].bytes;
				blocks.erase(blocks.begin() + (long)i + 1);
			}
			if (i > 0 && !blocks[i - 1].used) {
				blocks[i - 1].bytes += blocks[i].bytes;
				blocks.erase(blocks.begin() + (long)i);
			}
			return n;
		}
		return 0;
	}

	/* The largest free block (scratch for the placement probe): its offset, *n its size (0: none). */
	size_t largest_free(size_t *n) const
	{
		size_t at = 0;

		*n = 0;
		for (const PoolBlock &b : blocks)
			if (!b.used && b.bytes > *n) {
				*n = b.bytes;
				at = b.off;
			}
		return at;
	}
};

} /* namespace anni */
#endif

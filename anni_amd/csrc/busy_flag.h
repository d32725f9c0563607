/*
** A flag that lets one caller at a time into a section whose state is shared by all callers
** and turns the others away instead of making them wait (the flat sum of squares has one result
** slot per process, as the reference's static accumulator, num/gpu_cuda.cu:8485-8486).  No device
** call in here, so it can be exercised on the host.
*/
#ifndef ANNI_BUSY_FLAG_H__
#define ANNI_BUSY_FLAG_H__

#include <atomic>

namespace anni {

struct BusyFlag {
	std::atomic<int>	held;

	BusyFlag() : held(0) {}
	/* true: the caller is inside and must call leave(); false: somebody else is. */
	bool enter(void)
	{
		int expect = 0;

		return held.compare_exchange_strong(expect, 1, std::memory_order_acquire,
		    std::memory_order_relaxed);
	}
	void leave(void)
	{
		held.store(0, std::memory_order_release);
	}
};

/* Enters on construction when it can; leaves on destruction when it did. */
struct BusyScope {
	BusyFlag	&flag;
	const bool	entered;

	explicit BusyScope(BusyFlag &f) : flag(f), entered(f.enter()) {}
	~BusyScope()
	{
		if (entered)
			flag.leave();
	}
	BusyScope(const BusyScope &) = delete;
	BusyScope &operator=(const BusyScope &) = delete;
};

} /* namespace anni */
#endif

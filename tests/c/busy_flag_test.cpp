// Host-only test of anni_amd/csrc/busy_flag.h: at most one thread is ever inside, a thread that
// finds the section taken is turned away (it does not wait), and the flag is free again after
// every scope, also one left by an early return.
#include <atomic>
#include <cstdio>
#include <thread>
#include <vector>
#include "busy_flag.h"

static anni::BusyFlag flag;
static std::atomic<int> inside(0), worst(0);
static std::atomic<long> entered(0), refused(0);

static int section(bool leave_early)
{
	anni::BusyScope only(flag);

	if (!only.entered) {
		refused++;
		return -1;
	}
	const int now = ++inside;
	int w = worst.load();

	while (now > w && !worst.compare_exchange_weak(w, now))
		;
	entered++;
	if (leave_early) {
		--inside;
		return 1;
	}
	for (volatile int spin = 0; spin < 200; spin++)
		;
	--inside;
	return 0;
}

int main()
{
	std::vector<std::thread> pool;

	// alone: every call gets in, whatever way the one before it left
	for (int i = 0; i < 1000; i++)
		if (section(i % 3 == 0) < 0) {
			std::printf("FAIL refused with nobody inside at call %d\n", i);
			return 1;
		}
	// a second entry while the first is held is refused, and does not disturb the holder
	{
		anni::BusyScope first(flag);
		anni::BusyScope second(flag);

		if (!first.entered || second.entered) {
			std::printf("FAIL nested entry: first %d second %d\n", (int)first.entered, (int)second.entered);
			return 1;
		}
	}
	if (section(false) != 0) {
		std::printf("FAIL flag still held after the scopes ended\n");
		return 1;
	}
	entered = 0;
	refused = 0;
	for (int t = 0; t < 8; t++)
		pool.emplace_back([] {
			for (int i = 0; i < 200000; i++)
				(void)section(i % 7 == 0);
		});
	for (auto &th : pool)
		th.join();
	if (worst.load() != 1 || inside.load() != 0 || entered + refused != 8L * 200000 || entered == 0) {
		std::printf("FAIL worst %d inside %d entered %ld refused %ld\n", worst.load(), inside.load(),
		    entered.load(), refused.load());
		return 1;
	}
	std::printf("ok entered %ld refused %ld never more than one inside\n", entered.load(), refused.load());
	return 0;
}

/*
 * Arithmetic shared by the host-side scheduler (sched_host.cpp) and the GIN wire derivation
 * (gin_wire.cpp), which computes its schedule in place: one get_schedule() of the reference,
 * src/nccl_ofi_scheduler.cpp:47-133.
 */
#ifndef OFI_AMD_SCHED_HOST_HPP_
#define OFI_AMD_SCHED_HOST_HPP_

#include <cstdint>

namespace ofi_amd {

/* x / d, with a shift when d is a power of two (the defaults, 131072 and 128, are): this runs
 * once per message on the proxy thread, where 64-bit divisions are most of its cost */
inline uint64_t div_pow2_or_slow(uint64_t x, uint64_t d)
{
	return (d & (d - 1)) == 0 ? x >> __builtin_ctzll(d) : x / d;
}

/* x / k for the stripe counts that occur (1..4) */
inline uint64_t div_1_to_4(uint64_t x, uint32_t k)
{
	const uint64_t by3 = x / 3; /* a multiply by the compiler's reciprocal */
	const uint64_t sh = x >> (k >> 1); /* k = 1, 2, 4 -> shift 0, 1, 2 */
	return k == 3 ? by3 : sh;
}

/* (v + add) % R; the common cases (a counter already below R, add <= R) need no division */
inline uint32_t add_mod(uint32_t v, uint32_t add, uint32_t R)
{
	uint32_t s = v + add;
	if (s < R) {
		return s;
	}
	s -= R;
	return s < R ? s : s % R;
}

/* get_num_stripes, :47-64, after the cap to the rail count: the largest i in [2, n] that
 * divides R, else n itself (3 rails: a 2-stripe request stays 2).  [R - 1][n - 1]. */
constexpr uint8_t kStripeCount[4][4] = {
	{1, 1, 1, 1},
	{1, 2, 2, 2},
	{1, 2, 3, 3},
	{1, 2, 2, 4},
};

} // namespace ofi_amd

#endif

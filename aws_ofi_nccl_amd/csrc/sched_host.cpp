/*
 * The threshold scheduler for one message on the host (ofi_amd_sched_get_schedule): what the
 * reference's get_schedule() computes per call.  Plain C++: callers on the per-message path
 * (the send state machine, the GIN proxy) need no device for it.
 */
#include <cerrno>

#include "ofi_amd_hotpath.h"

namespace {

/* x / d, with a shift when d is a power of two (the defaults, 131072 and 128, are): this runs
 * once per message on the proxy thread, where three 64-bit divisions are most of its cost */
inline uint64_t div_by(uint64_t x, uint64_t d)
{
	return (d & (d - 1)) == 0 ? x >> __builtin_ctzll(d) : x / d;
}

/* NCCL_OFI_DIV_CEIL, include/nccl_ofi_math.h:23-26 */
inline uint64_t ceil_div(uint64_t x, uint64_t d)
{
	return x == 0 ? 0 : 1 + div_by(x - 1, d);
}

/* x / k for the stripe counts that occur (1..4) */
inline uint64_t div_small(uint64_t x, uint32_t k)
{
	switch (k) {
	case 1: return x;
	case 2: return x >> 1;
	case 4: return x >> 2;
	default: return x / k;
	}
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

} // namespace

extern "C" {

/* Host form: one get_schedule() call, src/nccl_ofi_scheduler.cpp:77-133. */
int ofi_amd_sched_get_schedule(ofi_amd_sched_state_t *st, uint64_t size, uint64_t align,
			       ofi_amd_xfer_info_t *xfers)
{
	if (!st || !xfers || st->num_rails < 1 || st->num_rails > OFI_AMD_MAX_NUM_RAILS ||
	    st->min_stripe_size == 0 || align == 0) {
		return -EINVAL;
	}
	const uint32_t R = (uint32_t)st->num_rails;

	if (size < st->max_small_msg_size) {
		xfers[0] = ofi_amd_xfer_info_t{(uint16_t)st->rr_small_counter, 0, 0, 0, size};
		st->rr_small_counter = add_mod(st->rr_small_counter, 1, R);
		return 1;
	}
	/* get_num_stripes, :47-64: the largest divisor of R not above ceil(size / min_stripe) */
	const uint64_t want = ceil_div(size, st->min_stripe_size);
	uint32_t n = (uint32_t)(want < R ? want : R);
	n = n > 1 ? n : 1;
	for (uint32_t i = n; i > 1; i--) {
		if (R % i == 0) {
			n = i;
			break;
		}
	}
	uint32_t rail = st->rr_counter;
	st->rr_counter = add_mod(st->rr_counter, n, R);
	const uint64_t per = size == 0 ? 0 : 1 + div_small(size - 1, n);
	const uint64_t max_stripe = ceil_div(per, align) * align;
	uint64_t left = size, offset = 0;
	for (uint32_t k = 0; k < n; k++) {
		const uint64_t stripe = left < max_stripe ? left : max_stripe;
		xfers[k] = ofi_amd_xfer_info_t{(uint16_t)rail, 0, 0, offset, stripe};
		offset += stripe;
		left -= stripe;
		rail = add_mod(rail, 1, R);
	}
	return (int)n;
}

} /* extern "C" */

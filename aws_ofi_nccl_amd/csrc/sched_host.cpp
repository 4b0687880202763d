/*
 * The threshold scheduler for one message on the host (ofi_amd_sched_get_schedule): what the
 * reference's get_schedule() computes per call.  Plain C++: callers on the per-message path
 * (the send state machine, the GIN proxy) need no device for it.
 */
#include <cerrno>

#include "ofi_amd_hotpath.h"

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
	auto ceil_div = [](uint64_t x, uint64_t y) -> uint64_t { return x == 0 ? 0 : 1 + (x - 1) / y; };

	if (size < st->max_small_msg_size) {
		xfers[0] = ofi_amd_xfer_info_t{(uint16_t)st->rr_small_counter, 0, 0, 0, size};
		st->rr_small_counter = (st->rr_small_counter + 1) % R;
		return 1;
	}
	uint64_t want = ceil_div(size, st->min_stripe_size);
	uint32_t n = (uint32_t)(want < R ? want : R);
	n = n > 1 ? n : 1;
	for (uint32_t i = n; i > 1; i--) {
		if (R % i == 0) {
			n = i;
			break;
		}
	}
	uint32_t rail = st->rr_counter;
	st->rr_counter = (st->rr_counter + n) % R;
	const uint64_t max_stripe = ceil_div(ceil_div(size, n), align) * align;
	uint64_t left = size, offset = 0;
	for (uint32_t k = 0; k < n; k++) {
		uint64_t stripe = left < max_stripe ? left : max_stripe;
		xfers[k] = ofi_amd_xfer_info_t{(uint16_t)rail, 0, 0, offset, stripe};
		offset += stripe;
		left -= stripe;
		rail = (rail + 1) % R;
	}
	return (int)n;
}

} /* extern "C" */

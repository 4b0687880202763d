/*
 * CPU oracle (test infrastructure): threshold scheduler.
 * Follows src/nccl_ofi_scheduler.cpp:47-133 and include/nccl_ofi_math.h:23-26.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

/* NCCL_OFI_DIV_CEIL, include/nccl_ofi_math.h:23-26: 0 for x == 0, no overflow near 2^64. */
static uint64_t div_ceil(uint64_t x, uint64_t y)
{
	return (x == 0) ? 0 : 1 + ((x - 1) / y);
}

void oracle_sched_init(oracle_sched_t *s, int num_rails, uint64_t min_stripe_size,
		       uint64_t max_small_msg_size)
{
	/* ctor, src/nccl_ofi_scheduler.cpp:203-210: both counters start at 0 */
	memset(s, 0, sizeof(*s));
	s->num_rails = num_rails;
	s->min_stripe_size = min_stripe_size;
	s->max_small_msg_size = max_small_msg_size;
}

/* get_num_stripes, src/nccl_ofi_scheduler.cpp:47-64 */
int oracle_sched_num_stripes(const oracle_sched_t *s, uint64_t size)
{
	uint64_t want = div_ceil(size, s->min_stripe_size);
	uint64_t rails = (uint64_t)s->num_rails;
	uint64_t capped = want < rails ? want : rails;
	int num_stripes = (int)(capped > 1 ? capped : 1);

	for (int i = num_stripes; i > 1; i--) {
		if ((s->num_rails % i) == 0) {
			num_stripes = i;
			break;
		}
	}
	return num_stripes;
}

/* set_schedule_by_threshold, src/nccl_ofi_scheduler.cpp:77-133 */
int oracle_sched_get_schedule(oracle_sched_t *s, uint64_t size, uint64_t align,
			      oracle_xfer_t *xfers)
{
	unsigned int rails = (unsigned int)s->num_rails;

	if (size < s->max_small_msg_size) {
		unsigned int rail = s->rr_small_counter;
		s->rr_small_counter = (s->rr_small_counter + 1) % rails;
		memset(&xfers[0], 0, sizeof(xfers[0]));
		xfers[0].rail_id = (uint16_t)rail;
		xfers[0].offset = 0;
		xfers[0].msg_size = size;
		return 1;
	}

	int num_stripes = oracle_sched_num_stripes(s, size);
	unsigned int rail = s->rr_counter;
	s->rr_counter = (s->rr_counter + (unsigned int)num_stripes) % rails;

	uint64_t left = size;
	uint64_t offset = 0;
	uint64_t max_stripe = div_ceil(div_ceil(size, (uint64_t)num_stripes), align) * align;

	for (int k = 0; k < num_stripes; k++) {
		uint64_t stripe = left < max_stripe ? left : max_stripe;
		memset(&xfers[k], 0, sizeof(xfers[k]));
		xfers[k].rail_id = (uint16_t)rail;
		xfers[k].offset = offset;
		xfers[k].msg_size = stripe;
		offset += stripe;
		left -= stripe;
		rail = (rail + 1) % rails;
	}
	return num_stripes;
}

void oracle_sched_batch(oracle_sched_t *s, const uint64_t *sizes, uint64_t n, uint64_t align,
			uint32_t *num_xfers, oracle_xfer_t *xfers)
{
	for (uint64_t i = 0; i < n; i++) {
		oracle_xfer_t *row = &xfers[i * ORACLE_MAX_RAILS];
		memset(row, 0, sizeof(oracle_xfer_t) * ORACLE_MAX_RAILS);
		num_xfers[i] = (uint32_t)oracle_sched_get_schedule(s, sizes[i], align, row);
	}
}

void oracle_sched_batch_alloc(oracle_sched_t *s, const uint64_t *sizes, uint64_t n,
			      uint64_t align, uint32_t *num_xfers, oracle_xfer_t *xfers)
{
	/* sizeof_schedule(): 16-byte header + one xfer_info per rail
	 * (include/nccl_ofi_scheduler.h:35-45) */
	size_t bytes = 16 + sizeof(oracle_xfer_t) * (size_t)s->num_rails;

	for (uint64_t i = 0; i < n; i++) {
		unsigned char *sched = (unsigned char *)malloc(bytes);
		oracle_xfer_t *tmp = (oracle_xfer_t *)(sched + 16);
		oracle_xfer_t *row = &xfers[i * ORACLE_MAX_RAILS];
		int k = oracle_sched_get_schedule(s, sizes[i], align, tmp);

		memset(row, 0, sizeof(oracle_xfer_t) * ORACLE_MAX_RAILS);
		memcpy(row, tmp, sizeof(oracle_xfer_t) * (size_t)k);
		num_xfers[i] = (uint32_t)k;
		free(sched);
	}
}

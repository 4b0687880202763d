/*
 * iputSignal's derivation for one descriptor as inline code, for the two places that run it:
 * ofi_amd_gin_iput_signal (csrc/gin_wire.cpp) and the proxy's drain loop (csrc/gin_proxy.cpp),
 * where it is inlined so that the communicator's state stays in registers from one descriptor
 * of a burst to the next.
 */
#ifndef OFI_AMD_GIN_DERIVE_HPP_
#define OFI_AMD_GIN_DERIVE_HPP_

#include <cerrno>
#include <cstring>

#include "ofi_amd_hotpath.h"
#include "sched_host.hpp"

namespace ofi_amd_gin {

/* include/rdma/gin/nccl_ofi_gin_types.h:55-113,209 */
constexpr uint32_t kImmCommShift = 1;
constexpr uint32_t kImmSeqShift = 11;
constexpr uint32_t kImmSeqMask = (1u << 13) - 1;
constexpr uint32_t kImmSegCntShift = 24;
constexpr uint32_t kImmAckReqShift = 28;
constexpr uint32_t kCursorMask = (1u << 14) - 1;   /* GIN_RX_CONSUMED_MASK */
constexpr uint32_t kCursorHalf = 1u << 13;         /* GIN_RX_CONSUMED_HALF */
constexpr uint32_t kAckInterval = 64;              /* GIN_ACK_INTERVAL */
constexpr uint32_t kReqsPerDoorbell = 16;          /* GIN_REQS_PER_DOORBELL */
constexpr uint32_t kAckReqThreshold = (kImmSeqMask + 1) / 2;
constexpr uint32_t kSignalInc = 1, kSignalAdd = 2; /* nccl/net.h:28-29 */
constexpr uint32_t kOptAggregate = 1;              /* nccl/rma_v15.h:19-21 */
constexpr uint64_t kStripeAlign = 128;             /* src/nccl_ofi_scheduler.cpp:168 */

inline uint32_t cursor_inc(uint32_t c) { return (c + 1) & kCursorMask; }
inline uint32_t cursor_delta(uint32_t a, uint32_t b) { return (a - b) & kCursorMask; }

/* GIN_IMM_SEG_DATA, include/rdma/gin/nccl_ofi_gin_types.h:76-79 */
inline uint32_t imm_word(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return (ack_req << kImmAckReqShift) | (nseg << kImmSegCntShift) | (seq << kImmSeqShift) |
	       (comm_id << kImmCommShift);
}

/* nccl_net_ofi_gin_msg_header_t, :128-145 */
inline uint64_t meta_header_word(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return ((uint64_t)(comm_id & 0x3ffu) << 2) | ((uint64_t)(seq & kImmSeqMask) << 12) |
	       ((uint64_t)(nseg & 0xfu) << 25) | ((uint64_t)(ack_req & 1u) << 29);
}

/* handle_ack_completion, src/rdma/gin/nccl_ofi_gin.cpp:1843-1869, with apply_rx_consumed,
 * include/rdma/gin/nccl_ofi_gin.h:535-543 */
inline void apply_ack(ofi_amd_gin_comm_t *c, uint32_t wire_rx_consumed)
{
	const uint32_t rx = wire_rx_consumed & kCursorMask;
	const uint32_t delta = cursor_delta(rx, c->tx_tail);
	if (delta > 0 && delta <= kCursorHalf) {
		c->tx_tail = rx;
	}
	if (c->has_pending_ack_request &&
	    cursor_delta(rx, c->last_ack_requested_seq) <= kCursorHalf) {
		c->has_pending_ack_request = 0;
	}
}

/*
 * iputSignal's derivation for one descriptor.  It runs once per descriptor on the proxy
 * thread, on operation sizes that are random from one descriptor to the next: whether the
 * message is small, how many stripes it has, whether it rides a pinned rail and whether its
 * doorbell is deferred are unpredictable branches if written as such, and a loop over the
 * stripes has an unpredictable trip count.  So the common case (a payload) is straight-line
 * code: the schedule is computed in place in closed form (every stripe but the last has the
 * full stripe length, so stripe k starts at k * max_stripe), all four write records are
 * produced every time and those beyond the stripe count are masked to zero, and the state
 * updates are selects.  Every field of *out is written exactly once.
 * POW2: the rail count is a power of two, both counters are below it and the minimum stripe
 * size is a power of two (the defaults: 4 rails, 128 KiB), so the modular steps are masks.
 */
template <bool POW2>
inline int derive(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
		  const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	const uint32_t sop = d->signal_op;
	const uint32_t head = c->tx_head;
	const uint32_t outstanding = cursor_delta(head, c->tx_tail);
	/* The handle indices come from a record that device code wrote: they are checked
	 * against the table before anything is looked up (a signal handle of 0xffff = none). */
	const bool bad_handle = (d->size > 0 && (d->src_mr >= n_mrs || d->dst_mr >= n_mrs)) ||
				(sop != 0 && d->sig_mr != 0xffff && d->sig_mr >= n_mrs);
	if (sop > kSignalAdd || bad_handle || outstanding >= kImmSeqMask + 1) {
		std::memset(out, 0, sizeof(*out));
		/* :580-584.  await_tx_window (:518-537) spins on progress; a pure derivation
		 * cannot, so a full window is handed back to the caller. */
		return (sop > kSignalAdd || bad_handle) ? -EINVAL : -EAGAIN;
	}
	if (!POW2) {
		/* a communicator edited by hand since comm_init: out-of-range rails are an error, not
		 * an index (the mask / shift path is only entered with all of this in range) */
		if (c->num_rails < 1 || c->num_rails > OFI_AMD_MAX_NUM_RAILS || c->next_rail_id >= c->num_rails ||
		    c->pinned_rail_id >= (int32_t)OFI_AMD_MAX_NUM_RAILS ||
		    (c->sched.num_rails >= 1 && c->pinned_rail_id >= c->sched.num_rails)) {
			std::memset(out, 0, sizeof(*out));
			return -EINVAL;
		}
	}
	const uint32_t seq = head & kImmSeqMask; /* :588 */
	const bool aggregate = (d->opt_flags & kOptAggregate) != 0;
	const bool has_signal = sop != 0;

	uint32_t ack_req = 0;
	if (outstanding >= kAckReqThreshold) { /* :611-627 */
		if (c->consecutive_puts_without_ack++ >= kAckInterval) {
			ack_req = 1;
			c->consecutive_puts_without_ack = 0;
			c->last_ack_requested_seq = head;
			c->has_pending_ack_request = 1;
		}
	}

	const int32_t pinned = c->pinned_rail_id;
	const bool batch_open = c->pinned_rail_run + 1 < kReqsPerDoorbell;
	const uint64_t size = d->size;
	bool defer;
	uint32_t nseg = has_signal ? 1u : 0u;
	uint32_t rail_id;

	if (size > 0) {
		ofi_amd_sched_state_t &st = c->sched;
		const uint32_t R = (uint32_t)st.num_rails;
		if (!POW2 && (R < 1 || R > OFI_AMD_MAX_NUM_RAILS || st.min_stripe_size == 0)) {
			std::memset(out, 0, sizeof(*out));
			return -ENOMEM; /* no schedule (:689-693) */
		}
		auto step = [R](uint32_t v, uint32_t add) -> uint32_t {
			return POW2 ? ((v + add) & (R - 1)) : ofi_amd::add_mod(v, add, R);
		};
		/* set_schedule_by_threshold, src/nccl_ofi_scheduler.cpp:77-133 */
		const bool small = size < st.max_small_msg_size;
		const uint64_t want = 1 + (POW2 ? (size - 1) >> __builtin_ctzll(st.min_stripe_size)
						: ofi_amd::div_pow2_or_slow(size - 1, st.min_stripe_size));
		const uint32_t capped = (uint32_t)(want < R ? want : R);
		const uint32_t n = small ? 1u : ofi_amd::kStripeCount[R - 1][capped - 1];
		/* counters at or beyond the rail count are taken modulo it, as the scheduler's own
		 * increment would leave them */
		const uint32_t rr_small = POW2 ? st.rr_small_counter : st.rr_small_counter % R;
		const uint32_t rr_big = POW2 ? st.rr_counter : st.rr_counter % R;
		const uint32_t first = small ? rr_small : rr_big;
		st.rr_small_counter = small ? step(rr_small, 1) : rr_small;
		st.rr_counter = small ? rr_big : step(rr_big, n);
		const uint64_t per = 1 + (POW2 ? (size - 1) >> (n >> 1) : ofi_amd::div_1_to_4(size - 1, n));
		const uint64_t aligned = (per + kStripeAlign - 1) & ~(kStripeAlign - 1);
		const uint64_t max_stripe = small ? size : aligned;

		const uint64_t src = mrs[d->src_mr].local_base + d->src_off;
		const ofi_amd_gin_mr_t &dst_mr = mrs[d->dst_mr];
		const uint64_t dest = dst_mr.remote_address_offset + d->dst_off;
		nseg += n;
		if (n == 1) {
			/* four ops in five: one stripe.  It rides the open pin so that the deferred
			 * doorbell is rung on that rail (:698-707). */
			rail_id = pinned >= 0 ? (uint32_t)pinned : first;
			defer = aggregate & batch_open;
			ofi_amd_gin_write_t &w = out->writes[0];
			w.src = src;
			w.len = size;
			w.dest = dest;
			w.key = dst_mr.key[rail_id];
			w.rail = rail_id;
			w.more = (uint32_t)(has_signal | defer);
			std::memset(&out->writes[1], 0, sizeof(out->writes[0]) * (OFI_AMD_MAX_NUM_RAILS - 1));
		} else {
			uint32_t rails[OFI_AMD_MAX_NUM_RAILS];
			rails[0] = first;
			rails[1] = step(first, 1);
			rails[2] = step(rails[1], 1);
			rails[3] = step(rails[2], 1);
			/* a striped op rings every rail it touches, so it is made to touch the pin
			 * (:708-726) */
			bool touches = false;
			for (uint32_t k = 0; k < OFI_AMD_MAX_NUM_RAILS; k++) {
				touches |= (k < n) & ((int32_t)rails[k] == pinned);
			}
			rails[0] = ((pinned >= 0) & !touches) ? (uint32_t)pinned : rails[0];
			defer = false;
			rail_id = rails[0];
			for (uint32_t k = 0; k < OFI_AMD_MAX_NUM_RAILS; k++) { /* :737-784 */
				const uint64_t live = (uint64_t)0 - (uint64_t)(k < n);
				const uint64_t offset = k * max_stripe;
				const uint64_t rest = size > offset ? size - offset : 0;
				const uint64_t stripe = rest < max_stripe ? rest : max_stripe;
				ofi_amd_gin_write_t &w = out->writes[k];
				w.src = (src + offset) & live;
				w.len = stripe & live;
				w.dest = (dest + offset) & live;
				w.key = dst_mr.key[rails[k]] & live;
				w.rail = rails[k] & (uint32_t)live;
				w.more = (k == 0 ? (uint32_t)has_signal : 0u);
			}
		}
		out->imm = imm_word(c->comm_id, seq, nseg, ack_req); /* :732 */
		out->num_writes = n;
	} else {
		/* signal only (:787-793); get_next_rail, nccl_ofi_gin_resources.h:363-368 */
		if (pinned >= 0) {
			rail_id = (uint32_t)pinned;
		} else {
			rail_id = c->next_rail_id;
			c->next_rail_id = (c->next_rail_id + 1) % c->num_rails;
		}
		defer = aggregate && batch_open;
		std::memset(out->writes, 0, sizeof(out->writes));
		out->imm = 0;
		out->num_writes = 0;
	}

	/* metadata message (:795-856); all-zero without a signal (63 ops in 64 as NCCL uses it:
	 * a branch that predicts well, unlike the ones above) */
	if (has_signal) {
		out->meta[0] = meta_header_word(c->comm_id, seq, nseg, ack_req);
		out->meta[1] = d->sig_mr != 0xffff ? mrs[d->sig_mr].remote_address : 0;
		out->meta[2] = d->signal_off;
		out->meta[3] = sop == kSignalInc ? 1 : d->signal_value;
		out->has_meta = 1;
		out->meta_rail = rail_id;
		out->meta_more = defer ? 1u : 0u;
	} else {
		std::memset(out->meta, 0, sizeof(out->meta));
		out->has_meta = 0;
		out->meta_rail = 0;
		out->meta_more = 0;
	}

	/* update_pin, :550-566 */
	c->pinned_rail_id = defer ? (int32_t)rail_id : -1;
	c->pinned_rail_run = defer ? c->pinned_rail_run + 1 : 0u;
	c->tx_head = cursor_inc(head); /* :860 */

	out->seq = seq;
	out->nseg = nseg;
	out->ack_req = ack_req;

	if (ack_req && c->ack_model == 1) {
		/* the standalone ACK for this op carries rx_consumed == tx_head */
		apply_ack(c, c->tx_head);
		c->has_pending_ack_request = 0;
	}
	return 0;
}

/* the mask / shift form of derive applies: power-of-two rail count and stripe size, both
 * counters below the rail count (derive keeps them there) */
inline bool derive_fast_path(const ofi_amd_gin_comm_t *c)
{
	/* The struct is the caller's: a rail count outside 1..4, a zero stripe size or a pin or
	 * rail cursor beyond the rail count (none of which comm_init or the derivation produce)
	 * would index the stripe and key tables out of range, so they never take this path. */
	const uint32_t R = (uint32_t)c->sched.num_rails;
	return R >= 1 && R <= OFI_AMD_MAX_NUM_RAILS && (R & (R - 1)) == 0 && c->sched.rr_small_counter < R &&
	       c->sched.rr_counter < R && c->sched.min_stripe_size != 0 &&
	       (c->sched.min_stripe_size & (c->sched.min_stripe_size - 1)) == 0 &&
	       c->pinned_rail_id < (int32_t)R && c->num_rails >= 1 && c->num_rails <= OFI_AMD_MAX_NUM_RAILS &&
	       c->next_rail_id < c->num_rails;
}

} // namespace ofi_amd_gin

#endif

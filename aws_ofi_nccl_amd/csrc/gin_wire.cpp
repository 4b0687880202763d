/*
 * What the GIN proxy derives from each descriptor -- the initiator part of
 * nccl_ofi_rdma_gin_put_comm::iputSignal, src/rdma/gin/nccl_ofi_gin.cpp:568-864
 * (sequence number, TX window, ACK-request hysteresis, stripes, rail pinning and
 * doorbell deferral, immediate data, 32-byte metadata message) -- and the encoders of the
 * GIN wire words.  The libfabric posts themselves (fi_writemsg / fi_sendmsg) are out of
 * scope: the derivation stops at their arguments.  Plain C++: no device needed.
 */
#include <cerrno>
#include <cstring>

#include "ofi_amd_hotpath.h"

namespace {

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

} // namespace

extern "C" {

/* GIN_IMM_SEG_DATA, include/rdma/gin/nccl_ofi_gin_types.h:76-79 */
uint32_t ofi_amd_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return (ack_req << kImmAckReqShift) | (nseg << kImmSegCntShift) | (seq << kImmSeqShift) |
	       (comm_id << kImmCommShift);
}

/* nccl_net_ofi_gin_msg_header_t, :128-145 */
uint64_t ofi_amd_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return ((uint64_t)(comm_id & 0x3ffu) << 2) | ((uint64_t)(seq & kImmSeqMask) << 12) |
	       ((uint64_t)(nseg & 0xfu) << 25) | ((uint64_t)(ack_req & 1u) << 29);
}

/* gin_ack_msg_t, :170-181 */
uint64_t ofi_amd_gin_ack_msg(uint32_t comm_id, uint32_t rx_consumed)
{
	return 1ull | ((uint64_t)(comm_id & 0x3ffu) << 2) | ((uint64_t)(rx_consumed & kCursorMask) << 12);
}

int ofi_amd_gin_comm_init(ofi_amd_gin_comm_t *c, uint32_t comm_id, uint32_t num_rails,
			  uint64_t min_stripe, uint64_t max_small, uint32_t ack_model)
{
	if (!c || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS || min_stripe == 0 ||
	    comm_id >= 1024 || ack_model > 1) {
		return -EINVAL;
	}
	std::memset(c, 0, sizeof(*c));
	c->sched.max_small_msg_size = max_small;
	c->sched.min_stripe_size = min_stripe;
	c->sched.num_rails = (int32_t)num_rails;
	c->comm_id = comm_id;
	c->num_rails = num_rails;
	c->pinned_rail_id = -1;
	c->ack_model = ack_model;
	return 0;
}

/* handle_ack_completion, src/rdma/gin/nccl_ofi_gin.cpp:1843-1869, with apply_rx_consumed,
 * include/rdma/gin/nccl_ofi_gin.h:535-543 */
void ofi_amd_gin_apply_ack(ofi_amd_gin_comm_t *c, uint32_t wire_rx_consumed)
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

int ofi_amd_gin_iput_signal(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs,
			    const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	const bool aggregate = (d->opt_flags & kOptAggregate) != 0;
	std::memset(out, 0, sizeof(*out));

	if (d->signal_op != 0 && d->signal_op != kSignalInc && d->signal_op != kSignalAdd) {
		return -EINVAL; /* :580-584 */
	}
	const uint32_t seq = c->tx_head & kImmSeqMask; /* :588 */

	/* await_tx_window (:518-537) spins on progress; a pure derivation cannot, so
	 * a full window is handed back to the caller. */
	const uint32_t outstanding = cursor_delta(c->tx_head, c->tx_tail);
	if (outstanding >= kImmSeqMask + 1) {
		return -EAGAIN;
	}

	const bool has_signal = d->signal_op != 0;
	uint32_t ack_req = 0;
	if (outstanding >= kAckReqThreshold) { /* :611-620 */
		if (c->consecutive_puts_without_ack++ >= kAckInterval) {
			ack_req = 1;
			c->consecutive_puts_without_ack = 0;
		}
	}
	if (ack_req) { /* :624-627 */
		c->last_ack_requested_seq = c->tx_head;
		c->has_pending_ack_request = 1;
	}

	bool defer = false;
	uint32_t nseg = has_signal ? 1u : 0u;
	uint32_t rail_id;

	if (d->size > 0) {
		const uint64_t src = mrs[d->src_mr].local_base + d->src_off;
		const ofi_amd_gin_mr_t &dst_mr = mrs[d->dst_mr];
		const uint64_t dest = dst_mr.remote_address_offset + d->dst_off;

		ofi_amd_xfer_info_t xfers[OFI_AMD_MAX_NUM_RAILS];
		const int n = ofi_amd_sched_get_schedule(&c->sched, d->size, kStripeAlign, xfers);
		if (n < 1) {
			return -ENOMEM;
		}
		const uint32_t num_xfers = (uint32_t)n;

		if (num_xfers == 1 && c->pinned_rail_id >= 0) {
			/* ride the open pin so the deferred doorbell is rung on that rail (:698-707) */
			xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
		} else if (num_xfers > 1 && c->pinned_rail_id >= 0) {
			/* a striped op rings every rail it touches; make it touch the pin (:708-726) */
			bool touches = false;
			for (uint32_t i = 0; i < num_xfers; i++) {
				touches |= xfers[i].rail_id == c->pinned_rail_id;
			}
			if (!touches) {
				xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
			}
		}
		defer = num_xfers == 1 && aggregate && (c->pinned_rail_run + 1 < kReqsPerDoorbell);

		nseg += num_xfers;
		out->imm = ofi_amd_gin_imm(c->comm_id, seq, nseg, ack_req); /* :732 */
		rail_id = xfers[0].rail_id;

		for (uint32_t k = 0; k < num_xfers; k++) { /* :737-784 */
			ofi_amd_gin_write_t &w = out->writes[k];
			w.rail = xfers[k].rail_id;
			w.src = src + xfers[k].offset;
			w.len = xfers[k].msg_size;
			w.dest = dest + xfers[k].offset;
			w.key = dst_mr.key[w.rail];
			w.more = ((has_signal && k == 0) || defer) ? 1u : 0u;
		}
		out->num_writes = num_xfers;
	} else {
		/* signal only (:787-793); get_next_rail, nccl_ofi_gin_resources.h:363-368 */
		if (c->pinned_rail_id >= 0) {
			rail_id = (uint32_t)c->pinned_rail_id;
		} else {
			rail_id = c->next_rail_id;
			c->next_rail_id = (c->next_rail_id + 1) % c->num_rails;
		}
		defer = aggregate && (c->pinned_rail_run + 1 < kReqsPerDoorbell);
	}

	if (has_signal) { /* :795-856 */
		out->has_meta = 1;
		out->meta[0] = ofi_amd_gin_meta_header(c->comm_id, seq, nseg, ack_req);
		out->meta[1] = d->sig_mr != 0xffff ? mrs[d->sig_mr].remote_address : 0;
		out->meta[2] = d->signal_off;
		out->meta[3] = d->signal_op == kSignalInc ? 1 : (d->signal_op == kSignalAdd ? d->signal_value : 0);
		out->meta_rail = rail_id;
		out->meta_more = defer ? 1u : 0u;
	}

	if (defer) { /* update_pin, :550-566 */
		c->pinned_rail_id = (int32_t)rail_id;
		c->pinned_rail_run++;
	} else {
		c->pinned_rail_id = -1;
		c->pinned_rail_run = 0;
	}
	c->tx_head = cursor_inc(c->tx_head); /* :860 */

	out->seq = seq;
	out->nseg = nseg;
	out->ack_req = ack_req;

	if (ack_req && c->ack_model == 1) {
		/* the standalone ACK for this op carries rx_consumed == tx_head */
		ofi_amd_gin_apply_ack(c, c->tx_head);
		c->has_pending_ack_request = 0;
	}
	return 0;
}

} /* extern "C" */

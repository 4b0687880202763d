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

#include "gin_derive.hpp"

namespace {

using namespace ofi_amd_gin;

/* kept out of line so that the common path below stays small */
__attribute__((noinline)) int derive_general(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs,
					     uint32_t n_mrs, const ofi_amd_gin_desc_t *d,
					     ofi_amd_gin_wire_t *out)
{
	return derive<false>(c, mrs, n_mrs, d, out);
}

} // namespace

extern "C" {

uint32_t ofi_amd_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return imm_word(comm_id, seq, nseg, ack_req);
}

uint64_t ofi_amd_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return meta_header_word(comm_id, seq, nseg, ack_req);
}

/* gin_ack_msg_t, include/rdma/gin/nccl_ofi_gin_types.h:170-181 */
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

void ofi_amd_gin_apply_ack(ofi_amd_gin_comm_t *c, uint32_t wire_rx_consumed)
{
	apply_ack(c, wire_rx_consumed);
}

int ofi_amd_gin_iput_signal(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
			    const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	if (!c || !mrs || !d || !out) {
		return -EINVAL;
	}
	return derive_fast_path(c) ? derive<true>(c, mrs, n_mrs, d, out) : derive_general(c, mrs, n_mrs, d, out);
}

/* nccl_ofi_rdma_gin_put_comm::iget, src/rdma/gin/nccl_ofi_gin.cpp:879-939: the schedule of the
 * size from the endpoint's scheduler (:899), and per stripe a read into
 * local input_address + localOff + offset from remote address_offset + remoteOff + offset with
 * the remote registration's key for the stripe's rail (:903-916).  No sequence number, no
 * window, no pin: gets are rare next to puts, so this is the plain loop. */
int ofi_amd_gin_iget(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
		     const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	if (!c || !mrs || !d || !out) {
		return -EINVAL;
	}
	std::memset(out, 0, sizeof(*out));
	if (d->kind != OFI_AMD_GIN_KIND_GET || d->src_mr >= n_mrs || d->dst_mr >= n_mrs) {
		return -EINVAL;
	}
	ofi_amd_xfer_info_t xfers[OFI_AMD_MAX_NUM_RAILS];
	const int n = ofi_amd_sched_get_schedule(&c->sched, d->size, kStripeAlign, xfers);
	if (n < 1 || n > OFI_AMD_MAX_NUM_RAILS) {
		return n < 0 ? n : -ENOMEM;
	}
	const ofi_amd_gin_mr_t &remote = mrs[d->src_mr];
	const uint64_t local = mrs[d->dst_mr].local_base + d->dst_off;
	const uint64_t from = remote.remote_address_offset + d->src_off;
	for (int k = 0; k < n; k++) {
		if (xfers[k].rail_id >= OFI_AMD_MAX_NUM_RAILS) {
			/* a round-robin counter edited beyond the rail count: an error, not a key index */
			std::memset(out, 0, sizeof(*out));
			return -EINVAL;
		}
	}
	for (int k = 0; k < n; k++) {
		ofi_amd_gin_write_t &r = out->writes[k];
		r.rail = xfers[k].rail_id;
		r.src = local + xfers[k].offset;
		r.len = xfers[k].msg_size;
		r.dest = from + xfers[k].offset;
		r.key = remote.key[r.rail];
		r.more = 0; /* "iget uses fi_read -- not part of the FI_MORE write-doorbell path" (:884) */
	}
	out->num_writes = (uint32_t)n;
	return 0;
}

int ofi_amd_gin_derive(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
		       const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	if (d && d->kind == OFI_AMD_GIN_KIND_GET) {
		return ofi_amd_gin_iget(c, mrs, n_mrs, d, out);
	}
	return ofi_amd_gin_iput_signal(c, mrs, n_mrs, d, out);
}

} /* extern "C" */

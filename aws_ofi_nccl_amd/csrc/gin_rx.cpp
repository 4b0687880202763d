/*
 * GIN receiver side on the host: what the proxy does with the completions its CQ
 * delivers -- reassembly per (peer, sequence number), strict in-order retire, greedy
 * folding of consecutive signals to one slot, standalone ACKs.  Follows
 * src/rdma/gin/nccl_ofi_gin.cpp:1016-1019, :1622-1790, :1792-1838, :1871-1924 of the
 * reference; the counter updates themselves run on the GPU (gin_signal.hip).
 *
 * The reference keeps outstanding ops in a hash map keyed (peer << 16 | seq).  The TX
 * window admits at most 8192 ops per peer, one per 13-bit sequence number, so a flat
 * table of 8192 slots per peer holds exactly the same set without hashing.
 */
#include <cerrno>
#include <cstring>
#include <new>
#include <vector>

#include "ofi_amd_hotpath.h"

namespace {

constexpr uint32_t kSeqMask = (1u << 13) - 1;    /* GIN_IMM_SEQ_MASK */
constexpr uint32_t kCursorMask = (1u << 14) - 1; /* GIN_RX_CONSUMED_MASK */

struct rx_req { /* 32 bytes: two to a cache line, walked in sequence order */
	uint8_t present = 0;
	uint8_t metadata_received = 0;
	uint8_t is_ack_requested = 0;
	uint8_t num_seg_completions = 0; /* at most 5: four writes and the metadata message */
	uint8_t total_segments = 0;
	uint8_t pad = 0;
	uint16_t meta_seq = 0;
	uint64_t base = 0, offset = 0, value = 0;
	bool complete() const { return present && num_seg_completions == total_segments; }
};
static_assert(sizeof(rx_req) == 32, "rx_req");

struct rx_peer {
	uint32_t comm_id = 0;
	uint32_t rx_consumed = 0;
	uint32_t next_delivered_seq = 0;
	std::vector<rx_req> reqs;
};

} // namespace

struct ofi_amd_gin_rx {
	std::vector<rx_peer> peers;
	std::vector<ofi_amd_gin_signal_work_t> work;
	std::vector<ofi_amd_gin_ack_t> acks;
};

namespace {

/* retire_completed_peer_iput_ops, :1622-1790 */
void retire(ofi_amd_gin_rx *rx, uint32_t peer)
{
	rx_peer &pc = rx->peers[peer];
	bool ack_requested = false;

	for (;;) {
		rx_req *req = &pc.reqs[pc.next_delivered_seq];
		if (!req->complete()) {
			break;
		}
		if (!req->metadata_received) {
			/* a put without signal: consume the sequence number, nothing to deliver */
			ack_requested |= req->is_ack_requested != 0;
			pc.rx_consumed = (pc.rx_consumed + 1) & kCursorMask;
			pc.next_delivered_seq = (pc.next_delivered_seq + 1) & kSeqMask;
			*req = rx_req();
			continue;
		}
		ofi_amd_gin_signal_work_t folded;
		std::memset(&folded, 0, sizeof(folded));
		folded.base = req->base;
		folded.offset = req->offset;
		folded.peer = peer;

		uint32_t cur_seq = pc.next_delivered_seq;
		rx_req *cur = req;
		for (;;) {
			folded.value += cur->value;
			folded.run_len++;
			ack_requested |= cur->is_ack_requested != 0;
			pc.rx_consumed = (pc.rx_consumed + 1) & kCursorMask;
			pc.next_delivered_seq = (pc.next_delivered_seq + 1) & kSeqMask;

			const uint32_t peek_seq = (cur_seq + 1) & kSeqMask;
			rx_req *peek = &pc.reqs[peek_seq];
			const bool extend = peek->complete() && peek->metadata_received &&
					    peek->base == folded.base && peek->offset == folded.offset;
			if (!extend) {
				break; /* cur is the run's last op */
			}
			*cur = rx_req();
			cur_seq = peek_seq;
			cur = peek;
		}
		folded.gate_seq = (uint16_t)cur->meta_seq;
		rx->work.push_back(folded);
		*cur = rx_req();
	}
	if (ack_requested) { /* maybe_send_ack, :1608-1620; send_ack, :267-315 */
		ofi_amd_gin_ack_t a;
		a.peer = peer;
		a.rx_consumed = pc.rx_consumed & kCursorMask;
		a.msg = ofi_amd_gin_ack_msg(pc.comm_id, pc.rx_consumed);
		rx->acks.push_back(a);
	}
}

template <typename T>
uint32_t take(std::vector<T> &q, T *out, uint32_t cap)
{
	const uint32_t n = q.size() < cap ? (uint32_t)q.size() : cap;
	if (n) {
		std::memcpy(out, q.data(), n * sizeof(T));
		q.erase(q.begin(), q.begin() + n);
	}
	return n;
}

} // namespace

extern "C" {

int ofi_amd_gin_rx_create(uint32_t n_peers, const uint32_t *peer_comm_ids, ofi_amd_gin_rx_t **out)
{
	if (!out || n_peers == 0 || n_peers > 65536) {
		return -EINVAL;
	}
	auto *rx = new (std::nothrow) ofi_amd_gin_rx();
	if (!rx) {
		return -ENOMEM;
	}
	try {
		rx->peers.resize(n_peers);
		for (uint32_t p = 0; p < n_peers; p++) {
			rx->peers[p].comm_id = peer_comm_ids ? peer_comm_ids[p] : p;
			rx->peers[p].reqs.resize(kSeqMask + 1);
		}
	} catch (...) {
		delete rx;
		return -ENOMEM;
	}
	*out = rx;
	return 0;
}

int ofi_amd_gin_rx_destroy(ofi_amd_gin_rx_t *rx)
{
	if (!rx) {
		return -EINVAL;
	}
	delete rx;
	return 0;
}

/* handle_signal_write_completion, :1871-1924 */
int ofi_amd_gin_rx_write_completion(ofi_amd_gin_rx_t *rx, uint32_t peer, uint32_t imm)
{
	if (!rx || peer >= rx->peers.size()) {
		return -EINVAL;
	}
	const uint32_t total = (imm >> 24) & 0xf; /* GIN_IMM_GET_SEG_CNT */
	const uint32_t seq = (imm >> 11) & kSeqMask;
	const bool ack = (imm >> 28) & 1;
	try {
		rx_req &req = rx->peers[peer].reqs[seq];
		if (!req.present) {
			req = rx_req();
			req.present = 1;
			req.num_seg_completions = 1;
			req.total_segments = (uint8_t)total;
			req.is_ack_requested = ack;
		} else {
			req.is_ack_requested |= (uint8_t)ack;
			req.num_seg_completions += 1;
		}
		if (req.num_seg_completions == req.total_segments) {
			req.meta_seq = (uint16_t)seq;
			retire(rx, peer);
		}
	} catch (...) {
		return -ENOMEM;
	}
	return 0;
}

/* handle_signal_metadata_completion, :1792-1838 */
int ofi_amd_gin_rx_metadata(ofi_amd_gin_rx_t *rx, uint32_t peer, const uint64_t meta[4])
{
	if (!rx || !meta || peer >= rx->peers.size() || (meta[0] & 3u) != 0) {
		return -EINVAL;
	}
	const uint32_t seq = (uint32_t)(meta[0] >> 12) & kSeqMask;
	const uint32_t total = (uint32_t)(meta[0] >> 25) & 0xf;
	const bool ack = (meta[0] >> 29) & 1;
	try {
		rx_req &req = rx->peers[peer].reqs[seq];
		if (!req.present) {
			req = rx_req();
			req.present = 1;
			req.num_seg_completions = 1;
			req.total_segments = (uint8_t)total;
			req.is_ack_requested = ack;
		} else {
			req.num_seg_completions += 1;
			req.is_ack_requested |= (uint8_t)ack;
		}
		req.metadata_received = 1;
		req.meta_seq = (uint16_t)seq;
		req.base = meta[1];
		req.offset = meta[2];
		req.value = meta[3];
		if (req.num_seg_completions == req.total_segments) {
			retire(rx, peer);
		}
	} catch (...) {
		return -ENOMEM;
	}
	return 0;
}

uint32_t ofi_amd_gin_rx_take_work(ofi_amd_gin_rx_t *rx, ofi_amd_gin_signal_work_t *out, uint32_t cap)
{
	return (rx && out) ? take(rx->work, out, cap) : 0;
}

uint32_t ofi_amd_gin_rx_take_acks(ofi_amd_gin_rx_t *rx, ofi_amd_gin_ack_t *out, uint32_t cap)
{
	return (rx && out) ? take(rx->acks, out, cap) : 0;
}

int ofi_amd_gin_rx_cursors(const ofi_amd_gin_rx_t *rx, uint32_t peer, uint32_t *rx_consumed,
			   uint32_t *next_seq)
{
	if (!rx || peer >= rx->peers.size() || !rx_consumed || !next_seq) {
		return -EINVAL;
	}
	*rx_consumed = rx->peers[peer].rx_consumed;
	*next_seq = rx->peers[peer].next_delivered_seq;
	return 0;
}

} /* extern "C" */

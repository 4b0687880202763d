/*
 * In-process loop-back of the send/receive path on one GPU (ofi_amd_sendrecv_loopback_run):
 * one send comm and one receive comm of this library, with this file standing where the
 * reference has two ranks and a libfabric provider (the isend/irecv/test loop of
 * tests/functional/nccl_message_transfer.cpp:19-56).  An eager send becomes a device copy of header
 * and payload into an rx buffer; the RDMA writes of a rendezvous become device copies stripe by
 * stripe; what the receiver decides to copy out of rx buffers goes through the batched eager
 * copy.  `inflight` messages are open at a time; each round is at most three launches (the wire's
 * copies, the eager copies, the flush read-back) and one wait on the flush slots.
 */
#include <cerrno>
#include <chrono>
#include <cstring>
#include <vector>

#include "host_util.hpp"
#include "ofi_amd_sendrecv.h"

namespace {

using ofi_amd::pinned_t;

constexpr uint32_t kPiece = 1u << 30;    /* a table entry's length is 32 bits: longer writes are cut */
constexpr uint32_t kRxStride = 8320;     /* 8192 + header room, rounded to the 128-byte rx alignment */
constexpr int64_t kEagerSendSize = 8192; /* OFI_NCCL_EAGER_MAX_SIZE default, src/nccl_ofi_rdma.cpp:6808 */

struct open_msg_t {
	uint64_t index = 0;
	int32_t send_req = -1;
	int32_t recv_req = -1;
	int32_t sub_idx = 0;
	uint32_t group_size = 1;
	ofi_amd_send_action_t action = {};
	bool sent = false;
};

uint64_t pieces_of(uint64_t bytes)
{
	return bytes == 0 ? 1 : (bytes + kPiece - 1) / kPiece;
}

} // namespace

extern "C" int ofi_amd_sendrecv_loopback_run(const uint64_t *src_addrs, const uint64_t *dst_addrs,
					     const uint64_t *sizes, const uint64_t *dst_sizes,
					     const int32_t *tags, uint64_t n_msgs, uint32_t inflight,
					     uint32_t num_rails, uint32_t group, void *rx_pool,
					     uint64_t rx_pool_bytes, uint32_t flags, void *stream,
					     ofi_amd_sendrecv_loopback_stats_t *stats)
{
	if (!src_addrs || !dst_addrs || !sizes || !dst_sizes || !rx_pool || !stats || inflight == 0 ||
	    inflight > OFI_AMD_MAX_REQUESTS || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS ||
	    group < 1 || group > OFI_AMD_WIRE_MAX_RECVS || rx_pool_bytes < (uint64_t)inflight * kRxStride) {
		return -EINVAL;
	}
	for (uint64_t i = 0; i < n_msgs; i++) {
		if (sizes[i] > 0xFFFFFFFFull || dst_sizes[i] > 0xFFFFFFFFull) {
			return -EMSGSIZE; /* the control message carries a 32-bit length */
		}
	}
	using clock = std::chrono::steady_clock;
	ofi_amd_sendrecv_loopback_stats_t st;
	std::memset(&st, 0, sizeof(st));

	/* table room for the fullest round */
	uint64_t cap_copy = 0;
	for (uint64_t lo = 0; lo < n_msgs; lo += inflight) {
		uint64_t need = 0;
		for (uint64_t i = lo; i < n_msgs && i < lo + inflight; i++) {
			need += pieces_of(sizes[i]) + OFI_AMD_WIRE_MAX_RAILS + 2;
		}
		cap_copy = need > cap_copy ? need : cap_copy;
	}
	if (cap_copy > (1ull << 30)) {
		return -EINVAL;
	}

	ofi_amd_send_comm_t *sc = nullptr;
	ofi_amd_recv_comm_t *rcv = nullptr;
	pinned_t t_src, t_dst, t_len, hdrs, e_rx, e_len, e_dst, e_cap, e_copied;
	std::vector<open_msg_t> open;
	std::vector<ofi_amd_eager_copy_item_t> items;
	int rc = ofi_amd_send_comm_create(1, num_rails, kEagerSendSize, 131072, 64, &sc);
	if (rc == 0) rc = ofi_amd_recv_comm_create(num_rails, &rcv);
	if (rc == 0) rc = t_src.alloc(sizeof(uint64_t) * cap_copy);
	if (rc == 0) rc = t_dst.alloc(sizeof(uint64_t) * cap_copy);
	if (rc == 0) rc = t_len.alloc(sizeof(uint32_t) * cap_copy);
	if (rc == 0) rc = hdrs.alloc(sizeof(ofi_amd_eager_hdr_t) * inflight);
	if (rc == 0) rc = e_rx.alloc(sizeof(uint64_t) * inflight);
	if (rc == 0) rc = e_len.alloc(sizeof(uint32_t) * inflight);
	if (rc == 0) rc = e_dst.alloc(sizeof(uint64_t) * inflight);
	if (rc == 0) rc = e_cap.alloc(sizeof(uint32_t) * inflight);
	if (rc == 0) rc = e_copied.alloc(sizeof(uint32_t) * inflight);
	/* the receiver's flush: a 64-byte sentinel buffer on the device, one 64-byte host slot per rail */
	pinned_t flush_slots;
	void *d_flush_buf = nullptr;
	if (rc == 0) rc = flush_slots.alloc(64 * OFI_AMD_WIRE_MAX_RAILS);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(d_flush_buf, OFI_AMD_RDMA_FLUSH_SENTINEL, stream);
	try {
		open.reserve(inflight);
		items.resize(inflight);
	} catch (...) {
		rc = rc ? rc : -ENOMEM;
	}
	auto release = [&]() {
		for (pinned_t *p : { &t_src, &t_dst, &t_len, &hdrs, &e_rx, &e_len, &e_dst, &e_cap, &e_copied }) {
			p->release();
		}
		flush_slots.release();
		if (d_flush_buf) (void)ofi_amd_gpu_mem_free(d_flush_buf);
		if (sc) (void)ofi_amd_send_comm_destroy(sc);
		if (rcv) (void)ofi_amd_recv_comm_destroy(rcv);
	};
	if (rc != 0) {
		release();
		return rc;
	}
	ofi_amd_ctrl_msg_t *mailbox = ofi_amd_send_comm_mailbox(sc);
	const bool receiver_first = (flags & 1u) != 0;
	const auto t0 = clock::now();

	for (uint64_t lo = 0; lo < n_msgs && rc == 0; lo += inflight) {
		const uint64_t hi = lo + inflight < n_msgs ? lo + inflight : n_msgs;
		open.clear();

		/* ---- both ranks post, one (grouped) receive at a time: the sender first unless told
		 * otherwise, so that whatever fits goes eager ahead of its control message; the rest
		 * waits for the receive.  Messages g .. g+group-1 share one receive request. ---- */
		for (uint64_t g = lo; g < hi && rc == 0; g += group) {
			const uint32_t gn = static_cast<uint32_t>(hi - g < group ? hi - g : group);
			const size_t first = open.size();
			int gtags[OFI_AMD_WIRE_MAX_RECVS];
			uint64_t keys[OFI_AMD_WIRE_MAX_RECVS * OFI_AMD_WIRE_MAX_RAILS];
			for (uint32_t k = 0; k < gn && rc == 0; k++) {
				open_msg_t m;
				m.index = g + k;
				gtags[k] = tags ? tags[g + k] : static_cast<int>(1 + k);
				for (uint32_t r = 0; r < num_rails; r++) {
					keys[k * num_rails + r] = g + k;
				}
				if (!receiver_first) {
					rc = ofi_amd_send_comm_send(sc, sizes[g + k], gtags[k], &m.action);
					m.sent = rc == 0 && m.action.kind != OFI_AMD_SEND_AGAIN;
					st.send_again += rc == 0 && !m.sent;
				}
				open.push_back(m);
			}
			int32_t recv_req = -1;
			if (rc == 0) {
				uint16_t seq = 0;
				rc = ofi_amd_recv_comm_recv(rcv, static_cast<int>(gn), &dst_addrs[g], &dst_sizes[g], gtags, keys, 0,
							    mailbox, &recv_req, &seq);
				/* the control message is in the sender's mailbox: its post is complete */
				if (rc == 0) rc = ofi_amd_recv_comm_ctrl_sent(rcv, recv_req);
			}
			for (uint32_t k = 0; k < gn && rc == 0; k++) {
				open_msg_t &m = open[first + k];
				m.recv_req = recv_req;
				m.sub_idx = static_cast<int32_t>(k);
				m.group_size = gn;
				if (!m.sent) {
					rc = ofi_amd_send_comm_send(sc, sizes[m.index], gtags[k], &m.action);
					if (rc == 0 && m.action.kind == OFI_AMD_SEND_AGAIN) {
						rc = -EPROTO; /* its control message is there: the send must go */
					}
					m.sent = rc == 0;
				}
				m.send_req = m.action.req;
			}
		}
		if (rc != 0) {
			break;
		}

		/* ---- the wire: one table of device copies for everything the sender handed out ---- */
		uint64_t *src = t_src.as<uint64_t>(), *dst = t_dst.as<uint64_t>();
		uint32_t *len = t_len.as<uint32_t>();
		uint32_t n_copy = 0, n_eager = 0, longest = OFI_AMD_EAGER_HEADER_SIZE;
		for (open_msg_t &m : open) {
			const ofi_amd_send_action_t &a = m.action;
			if (a.kind == OFI_AMD_SEND_EAGER) {
				const uint64_t slot = reinterpret_cast<uint64_t>(rx_pool) + (uint64_t)n_eager * kRxStride;
				hdrs.as<ofi_amd_eager_hdr_t>()[n_eager] = a.hdr;
				src[n_copy] = reinterpret_cast<uint64_t>(hdrs.dev) + n_eager * sizeof(ofi_amd_eager_hdr_t);
				dst[n_copy] = slot;
				len[n_copy++] = OFI_AMD_EAGER_HEADER_SIZE;
				if (a.size) {
					src[n_copy] = src_addrs[m.index];
					dst[n_copy] = slot + OFI_AMD_EAGER_HEADER_SIZE;
					len[n_copy++] = static_cast<uint32_t>(a.size);
					longest = a.size > longest ? static_cast<uint32_t>(a.size) : longest;
				}
				rc = ofi_amd_recv_comm_eager_arrival(rcv, a.msg_seq_num, &a.hdr, static_cast<uint32_t>(a.size),
								     n_eager);
				n_eager++;
				st.eager_messages++;
			} else {
				for (uint32_t k = 0; k < a.num_xfers && rc == 0; k++) {
					const ofi_amd_xfer_info_t &x = a.xfers[k];
					for (uint64_t off = 0; off < x.msg_size; off += kPiece) {
						const uint64_t n = x.msg_size - off < kPiece ? x.msg_size - off : kPiece;
						src[n_copy] = src_addrs[m.index] + x.offset + off;
						dst[n_copy] = a.remote_buff_offset + x.offset + off;
						len[n_copy++] = static_cast<uint32_t>(n);
						longest = n > longest ? static_cast<uint32_t>(n) : longest;
					}
					rc = ofi_amd_recv_comm_write_arrival(rcv, a.imm, x.msg_size);
					st.rdma_writes++;
				}
				st.write_messages++;
			}
			/* the sender's completions: the eager send, or every write of the schedule */
			for (uint32_t k = 0; k < (a.kind == OFI_AMD_SEND_EAGER ? 1u : a.num_xfers) && rc == 0; k++) {
				rc = ofi_amd_send_comm_completion(sc, m.send_req);
			}
			if (rc != 0) {
				break;
			}
		}
		if (rc == 0 && n_copy) {
			/* a write is one table entry whatever its length: the launch gives every 8 KiB of it
			 * a wavefront of its own */
			rc = ofi_amd_copy_table_pieces(t_src.dev_as<uint64_t>(), t_dst.dev_as<uint64_t>(),
						       t_len.dev_as<uint32_t>(), n_copy, longest, stream);
			st.launches++;
			st.copy_entries += n_copy;
		}

		/* ---- receiver: everything matched so far leaves the rx buffers in one launch ---- */
		uint32_t n_items = 0;
		if (rc == 0) {
			n_items = ofi_amd_recv_comm_take_copies(rcv, items.data(), inflight);
			if (n_items != n_eager) {
				rc = -EPROTO; /* every receive of the round is posted: every arrival must match */
			}
		}
		uint32_t n_ecopy = 0;
		for (uint32_t k = 0; k < n_items && rc == 0; k++) {
			if (!items[k].needs_copy) {
				continue;
			}
			e_rx.as<uint64_t>()[n_ecopy] = items[k].rx_cookie * kRxStride;
			e_len.as<uint32_t>()[n_ecopy] = items[k].recv_len;
			e_dst.as<uint64_t>()[n_ecopy] = items[k].dst;
			e_cap.as<uint32_t>()[n_ecopy] = static_cast<uint32_t>(items[k].dst_len);
			n_ecopy++;
		}
		if (rc == 0 && n_ecopy) {
			rc = ofi_amd_eager_copy_batch(rx_pool, e_rx.dev_as<uint64_t>(), e_len.dev_as<uint32_t>(), nullptr,
						      e_dst.dev_as<uint64_t>(), e_cap.dev_as<uint32_t>(), n_ecopy,
						      static_cast<uint32_t *>(e_copied.dev), nullptr, stream);
			st.launches++;
		}
		/* ---- receiver: flush, as NCCL asks for after receives into GPU memory.  The sentinel
		 * read-back is queued behind the round's launches, so its arrival in the host slots
		 * also says that they are done; a round that moved no byte needs no flush and just
		 * waits for the stream. ---- */
		if (rc == 0) {
			int any_bytes = 0;
			for (const open_msg_t &m : open) {
				any_bytes |= m.action.size != 0;
			}
			int32_t flush_req = -1;
			rc = ofi_amd_recv_comm_flush(rcv, 1, &any_bytes, &flush_req);
			if (rc == 0 && flush_req >= 0) {
				std::memset(flush_slots.host, 0, 64 * OFI_AMD_WIRE_MAX_RAILS);
				rc = ofi_amd_flush_post(d_flush_buf, flush_slots.dev, num_rails, stream);
				st.launches++;
				const auto w0 = clock::now();
				for (int done = 0; rc == 0 && !done;) {
					rc = ofi_amd_recv_comm_flush_test(rcv, flush_req, flush_slots.host, num_rails,
									  OFI_AMD_RDMA_FLUSH_SENTINEL, &done);
					if (!done && std::chrono::duration<double>(clock::now() - w0).count() > 20.0) {
						rc = -ETIMEDOUT;
					}
				}
				st.flushes++;
			} else if (rc == 0) {
				rc = ofi_amd_gpu_stream_synchronize(stream);
			}
		}
		for (uint32_t k = 0, j = 0; k < n_items && rc == 0; k++) {
			if (!items[k].needs_copy) {
				continue;
			}
			const uint32_t want = items[k].recv_len < items[k].dst_len ? items[k].recv_len
										    : static_cast<uint32_t>(items[k].dst_len);
			if (e_copied.as<uint32_t>()[j++] != want) {
				rc = -EIO;
				break;
			}
			rc = ofi_amd_recv_comm_copy_done(rcv, items[k].req, items[k].sub_idx);
		}

		/* ---- both ranks test their requests: all of the round must be complete ---- */
		uint64_t group_moved = 0;
		for (open_msg_t &m : open) {
			if (rc != 0) {
				break;
			}
			int done = 0;
			int rsizes[OFI_AMD_WIRE_MAX_RECVS] = {};
			uint64_t ssize = 0;
			rc = ofi_amd_send_comm_test(sc, m.send_req, &done, &ssize);
			if (rc == 0 && !done) rc = -EPROTO;
			if (rc == 0 && m.sub_idx == static_cast<int32_t>(m.group_size) - 1) {
				/* the group's last message: the receive request is complete with it */
				rc = ofi_amd_recv_comm_test(rcv, m.recv_req, &done, rsizes);
				if (rc == 0 && !done) rc = -EPROTO;
			}
			const uint64_t moved = sizes[m.index] < dst_sizes[m.index] ? sizes[m.index] : dst_sizes[m.index];
			if (rc == 0 && ssize != moved) rc = -EIO;
			group_moved += moved;
			if (m.sub_idx == static_cast<int32_t>(m.group_size) - 1) {
				/* the receiver reports, per sub-receive, the bytes that landed in it */
				uint64_t reported = 0;
				for (uint32_t j = 0; j < m.group_size; j++) {
					reported += static_cast<uint64_t>(static_cast<uint32_t>(rsizes[j]));
				}
				if (rc == 0 && reported != group_moved) rc = -EIO;
				group_moved = 0;
			}
			st.payload_bytes += moved;
			st.messages++;
		}
		st.rounds++;
	}
	st.seconds = std::chrono::duration<double>(clock::now() - t0).count();
	if (rc != 0) {
		/* a round that was given up may have launches in flight that read the tables freed below */
		(void)ofi_amd_gpu_stream_synchronize(stream);
	}
	release();
	*stats = st;
	return rc;
}

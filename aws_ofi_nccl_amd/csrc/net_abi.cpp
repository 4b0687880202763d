/*
 * The data-path members of ncclNet_vN_t (3rd-party/nccl/cuda/include/nccl/net_v12.h:110-119:
 * isend, irecv, iflush, test) as free functions over this library's send and receive state
 * machines (sendrecv_proto.cpp) and copy kernels, for the two ends of a link inside one
 * process on one GPU.  The wrappers they stand for: nccl_net_ofi_isend / _irecv / _iflush /
 * _test, src/nccl_ofi_api.cpp:440-567, and the versioned shims of
 * src/nccl_ofi_interface_nvidia.cpp:502-555.
 *
 * The "network" is a pipeline of launch groups on the caller's stream.  A group holds the
 * device copies of what the sending end handed out since the last launch (an eager send:
 * header and payload into an rx buffer; a rendezvous write: one table entry per rail stripe)
 * and the eager copies of what the receiving end has matched (rx buffer -> user buffer), and
 * ends in a sentinel read-back into a pinned word; the flushes asked for since the last launch
 * ride on that read-back.  When the sentinel of a group is seen, its
 * transfers are reported to the state machines in the order they were posted: the arrivals to
 * the receiving end, the completions to the sending end.  Every entry point makes progress
 * (polls the sentinels), the way the reference's drain the completion queue; test and iflush
 * also launch the group being filled, so a run of posts followed by polling is one group.
 */
#include <cerrno>
#include <cstring>
#include <new>
#include <vector>

#include "host_util.hpp"
#include "nccl_translate.hpp"
#include "ofi_amd_hotpath.h"
#include "ofi_amd_net_abi.h"

namespace {

constexpr uint32_t kRxStride = 8320;    /* 8192 + header room, rounded to the 128-byte rx alignment */
constexpr uint32_t kGroups = 8;         /* launch groups in flight, at most */
constexpr uint32_t kGroupsKeptBusy = 2; /* in flight before posts start gathering instead of leaving at once */
constexpr uint32_t kGroupEntries = 512; /* table entries of a group's wire copies */
constexpr uint32_t kGroupEager = 256;   /* eager copies of a group */
constexpr uint32_t kMagic = 0x4e455451; /* marks a live request */
constexpr uint32_t kMaxRxBuffers = 256; /* the receiving end queues at most 256 eager arrivals (ofi_amd_recv_comm_eager_arrival) */

using ofi_amd::pinned_t;

enum req_kind_t : uint8_t { kSend = 1, kRecv = 2, kFlush = 3 };

/* What a request pointer handed to NCCL points to. */
struct net_req_t {
	uint32_t magic = 0;
	uint8_t kind = 0;
	uint8_t n = 0; /* receives of the request */
	int32_t id = -1;
	ofi_amd_net_link *link = nullptr;
};

/* One transfer of a group, as the state machines will hear of it. */
struct landing_t {
	uint8_t eager;
	int32_t send_req;
	uint32_t rx_slot;      /* eager */
	uint16_t msg_seq_num;  /* eager */
	ofi_amd_eager_hdr_t hdr;
	uint32_t imm;          /* write */
	uint64_t len;          /* eager: payload bytes; write: this stripe's bytes */
};

struct group_t {
	pinned_t src, dst, len;                        /* wire copies */
	pinned_t hdrs;                                 /* eager headers on their way into rx buffers */
	pinned_t e_rx, e_len, e_dst, e_cap, e_copied;  /* eager copies */
	pinned_t done;                                 /* the sentinel lands here */
	uint32_t n_copy = 0, n_hdr = 0, n_eager = 0, max_len = 0;
	std::vector<landing_t> landings;
	std::vector<ofi_amd_eager_copy_item_t> items;
	std::vector<int32_t> flushes; /* flush requests that ride on this group's sentinel read-back */
	bool launched = false;
	int alloc()
	{
		int rc = src.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = dst.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = len.alloc(sizeof(uint32_t) * kGroupEntries);
		if (rc == 0) rc = hdrs.alloc(sizeof(ofi_amd_eager_hdr_t) * kGroupEntries);
		if (rc == 0) rc = e_rx.alloc(sizeof(uint64_t) * kGroupEager);
		if (rc == 0) rc = e_len.alloc(sizeof(uint32_t) * kGroupEager);
		if (rc == 0) rc = e_dst.alloc(sizeof(uint64_t) * kGroupEager);
		if (rc == 0) rc = e_cap.alloc(sizeof(uint32_t) * kGroupEager);
		if (rc == 0) rc = e_copied.alloc(sizeof(uint32_t) * kGroupEager);
		if (rc == 0) rc = done.alloc(64);
		return rc;
	}
	void release()
	{
		for (pinned_t *p : { &src, &dst, &len, &hdrs, &e_rx, &e_len, &e_dst, &e_cap, &e_copied, &done }) {
			p->release();
		}
	}
	/* a transfer without bytes (a zero-length write) still waits for its group's sentinel */
	bool empty() const { return n_copy == 0 && n_eager == 0 && landings.empty() && flushes.empty(); }
	void reset()
	{
		n_copy = n_hdr = n_eager = max_len = 0;
		landings.clear();
		items.clear();
		flushes.clear();
		launched = false;
	}
};

} // namespace

struct ofi_amd_net_link {
	uint32_t num_rails = 0;
	int64_t eager_max_size = 0;
	void *stream = nullptr;
	ofi_amd_send_comm_t *sc = nullptr;
	ofi_amd_recv_comm_t *rcv = nullptr;
	void *rx_pool = nullptr;
	std::vector<uint32_t> rx_free;
	void *d_flush_buf = nullptr;
	std::vector<uint64_t> flush_slots; /* per flush request: one 64-byte slot per rail */
	group_t groups[kGroups];
	uint32_t head = 0, cur = 0; /* positions: head = oldest launched group, cur = the one being filled */
	std::vector<net_req_t> send_reqs, recv_reqs, flush_reqs;
	ofi_amd_net_link_stats_t st = {};
	/* the two ends are tagged pointers into this object, so that a send comm handed to irecv
	 * is refused */
	struct end_t {
		uint32_t magic;
		ofi_amd_net_link *link;
	} send_end = { 0x53454e44, this }, recv_end = { 0x52454356, this };

	group_t &filling() { return groups[cur % kGroups]; }
	bool can_launch() const { return cur - head < kGroups - 1; }

	/* the sentinel of the oldest launched groups: report what they carried */
	int reap()
	{
		while (head != cur) {
			group_t &g = groups[head % kGroups];
			if (!g.launched || ofi_amd_flush_test(g.done.host, 1, OFI_AMD_RDMA_FLUSH_SENTINEL) != 1) {
				break;
			}
			for (const landing_t &l : g.landings) {
				int rc;
				if (l.eager) {
					rc = ofi_amd_recv_comm_eager_arrival(rcv, l.msg_seq_num, &l.hdr, (uint32_t)l.len, l.rx_slot);
				} else {
					rc = ofi_amd_recv_comm_write_arrival(rcv, l.imm, l.len);
				}
				if (rc == 0) {
					rc = ofi_amd_send_comm_completion(sc, l.send_req);
				}
				if (rc != 0) {
					return rc;
				}
			}
			for (uint32_t k = 0; k < g.n_eager; k++) {
				const ofi_amd_eager_copy_item_t &it = g.items[k];
				const uint32_t want = it.recv_len < it.dst_len ? it.recv_len : (uint32_t)it.dst_len;
				if (g.e_copied.as<uint32_t>()[k] != want) {
					return -EIO;
				}
				const int rc = ofi_amd_recv_comm_copy_done(rcv, it.req, it.sub_idx);
				if (rc != 0) {
					return rc;
				}
				rx_free.push_back((uint32_t)it.rx_cookie);
				st.eager_copies++;
			}
			/* the group's sentinel read-back was queued behind everything launched before these
			 * flushes were asked for: it is their read-back too (one operation flushes all requests
			 * at once, as the reference's flush does for the buffers of one call) */
			for (int32_t id : g.flushes) {
				for (uint32_t rail = 0; rail < num_rails; rail++) {
					__atomic_store_n(&flush_slots[((size_t)id * OFI_AMD_WIRE_MAX_RAILS + rail) * 8],
							 (uint64_t)OFI_AMD_RDMA_FLUSH_SENTINEL, __ATOMIC_RELEASE);
				}
			}
			g.reset();
			head++;
		}
		return 0;
	}

	/* what the receiving end has matched since the last call joins the group being filled */
	int gather_eager_copies()
	{
		for (;;) {
			group_t &g = filling();
			if (g.n_eager == kGroupEager) {
				return 0; /* the rest waits for the next group */
			}
			ofi_amd_eager_copy_item_t it;
			if (ofi_amd_recv_comm_take_copies(rcv, &it, 1) == 0) {
				return 0;
			}
			if (!it.needs_copy) {
				rx_free.push_back((uint32_t)it.rx_cookie); /* a zero-length message: nothing to move */
				continue;
			}
			const uint32_t k = g.n_eager++;
			g.items.push_back(it);
			g.e_rx.as<uint64_t>()[k] = it.rx_cookie * kRxStride;
			g.e_len.as<uint32_t>()[k] = it.recv_len;
			g.e_dst.as<uint64_t>()[k] = it.dst;
			g.e_cap.as<uint32_t>()[k] = (uint32_t)it.dst_len;
		}
	}

	/* While two groups are in flight, what is posted keeps gathering in the group being filled
	 * instead of leaving as a group of its own: the pipeline stays busy, and the size of a group
	 * follows the time a launch takes (small messages, many to a group; large ones, few).
	 * `now`: launch regardless, as long as a group slot is free (the caller is out of room). */
	int launch(bool now = false)
	{
		group_t &g = filling();
		if (g.empty() || !can_launch() || (!now && cur - head >= kGroupsKeptBusy)) {
			return 0;
		}
		int rc = 0;
		if (g.n_copy) {
			/* a launch holds at most 2^31 - 1 wavefronts, one per 8 KiB of the longest entry */
			const uint64_t per_entry = ((uint64_t)g.max_len + 8191u) / 8192u;
			const uint64_t most = per_entry ? 0x7fff0000ull / per_entry : g.n_copy;
			const uint32_t part = most < 1 ? 1u : (most < g.n_copy ? (uint32_t)most : g.n_copy);
			for (uint32_t at = 0; at < g.n_copy && rc == 0; at += part) {
				const uint32_t cnt = g.n_copy - at < part ? g.n_copy - at : part;
				rc = ofi_amd_copy_table_pieces(g.src.dev_as<uint64_t>() + at, g.dst.dev_as<uint64_t>() + at,
							       g.len.dev_as<uint32_t>() + at, cnt, g.max_len, stream);
				st.launches++;
			}
			st.copy_entries += g.n_copy;
		}
		if (rc == 0 && g.n_eager) {
			rc = ofi_amd_eager_copy_batch(rx_pool, g.e_rx.dev_as<uint64_t>(), g.e_len.dev_as<uint32_t>(), nullptr,
						      g.e_dst.dev_as<uint64_t>(), g.e_cap.dev_as<uint32_t>(), g.n_eager,
						      static_cast<uint32_t *>(g.e_copied.dev), nullptr, stream);
			st.launches++;
		}
		if (rc == 0) {
			__atomic_store_n(g.done.as<uint64_t>(), 0ull, __ATOMIC_RELEASE);
			rc = ofi_amd_flush_post(d_flush_buf, g.done.dev, 1, stream);
			st.launches++;
		}
		if (rc != 0) {
			return rc;
		}
		g.launched = true;
		cur++;
		return 0;
	}

	/* Posting calls (isend, irecv) only look at what has completed; the calls that wait for
	 * something (test, iflush) also launch what has been posted since the last launch, so a run
	 * of posts followed by polling -- NCCL's pattern -- travels as one launch group. */
	int progress(bool launch_pending)
	{
		st.progress_calls++;
		int rc = reap();
		if (rc == 0) rc = gather_eager_copies();
		if (rc == 0 && launch_pending) rc = launch();
		return rc;
	}
};

namespace {

ofi_amd_net_link *link_of(void *comm, uint32_t magic)
{
	ofi_amd_net_link::end_t *e = static_cast<ofi_amd_net_link::end_t *>(comm);
	return (e && e->magic == magic && e->link) ? e->link : nullptr;
}

net_req_t *take_req(std::vector<net_req_t> &pool, uint8_t kind, int32_t id, uint8_t n, ofi_amd_net_link *link)
{
	if (id < 0 || (size_t)id >= pool.size() || pool[(size_t)id].magic == kMagic) {
		return nullptr;
	}
	net_req_t &q = pool[(size_t)id];
	q.magic = kMagic;
	q.kind = kind;
	q.n = n;
	q.id = id;
	q.link = link;
	return &q;
}

int isend_impl(void *sendComm, void *data, size_t size, int tag, void **request)
{
	if (request) {
		*request = nullptr;
	}
	ofi_amd_net_link *l = link_of(sendComm, 0x53454e44);
	if (!l || !request) {
		return -EINVAL;
	}
	l->st.isend_calls++;
	int rc = l->progress(false);
	if (rc != 0) {
		return rc;
	}
	/* room for whatever the state machine decides: an rx buffer if the message may go eager, a
	 * header and a payload entry or one entry per rail */
	group_t *g = &l->filling();
	const bool may_go_eager = ofi_amd_eager_fits(size, l->eager_max_size) != 0;
	if (g->n_copy + OFI_AMD_WIRE_MAX_RAILS + 2 > kGroupEntries || (may_go_eager && l->rx_free.empty())) {
		rc = l->launch(true);
		g = &l->filling();
		if (rc != 0) {
			return rc;
		}
		if (g->n_copy + OFI_AMD_WIRE_MAX_RAILS + 2 > kGroupEntries || (may_go_eager && l->rx_free.empty())) {
			l->st.isend_again++;
			return 0; /* call again */
		}
	}
	ofi_amd_send_action_t a;
	rc = ofi_amd_send_comm_send(l->sc, size, tag, &a);
	if (rc != 0) {
		return rc;
	}
	if (a.kind == OFI_AMD_SEND_AGAIN) {
		l->st.isend_again++;
		return 0;
	}
	const uint64_t from = reinterpret_cast<uintptr_t>(data);
	if (a.kind == OFI_AMD_SEND_EAGER) {
		const uint32_t slot = l->rx_free.back();
		l->rx_free.pop_back();
		const uint64_t rx = reinterpret_cast<uintptr_t>(l->rx_pool) + (uint64_t)slot * kRxStride;
		g->hdrs.as<ofi_amd_eager_hdr_t>()[g->n_hdr] = a.hdr;
		g->src.as<uint64_t>()[g->n_copy] =
			reinterpret_cast<uintptr_t>(g->hdrs.dev) + g->n_hdr * sizeof(ofi_amd_eager_hdr_t);
		g->dst.as<uint64_t>()[g->n_copy] = rx;
		g->len.as<uint32_t>()[g->n_copy++] = OFI_AMD_EAGER_HEADER_SIZE;
		g->n_hdr++;
		g->max_len = g->max_len < OFI_AMD_EAGER_HEADER_SIZE ? OFI_AMD_EAGER_HEADER_SIZE : g->max_len;
		if (a.size) {
			g->src.as<uint64_t>()[g->n_copy] = from;
			g->dst.as<uint64_t>()[g->n_copy] = rx + OFI_AMD_EAGER_HEADER_SIZE;
			g->len.as<uint32_t>()[g->n_copy++] = (uint32_t)a.size;
			g->max_len = g->max_len < (uint32_t)a.size ? (uint32_t)a.size : g->max_len;
		}
		landing_t ld;
		std::memset(&ld, 0, sizeof(ld));
		ld.eager = 1;
		ld.send_req = a.req;
		ld.rx_slot = slot;
		ld.msg_seq_num = a.msg_seq_num;
		ld.hdr = a.hdr;
		ld.len = a.size;
		g->landings.push_back(ld);
		l->st.eager_sends++;
	} else {
		if (a.num_xfers == 0) {
			return -EPROTO; /* a write message always has a schedule, if only of one empty stripe */
		}
		for (uint32_t k = 0; k < a.num_xfers; k++) {
			const ofi_amd_xfer_info_t &x = a.xfers[k];
			if (x.msg_size > 0xffffffffull) {
				return -EMSGSIZE;
			}
			if (x.msg_size) {
				g->src.as<uint64_t>()[g->n_copy] = from + x.offset;
				g->dst.as<uint64_t>()[g->n_copy] = a.remote_buff_offset + x.offset;
				g->len.as<uint32_t>()[g->n_copy++] = (uint32_t)x.msg_size;
				g->max_len = g->max_len < (uint32_t)x.msg_size ? (uint32_t)x.msg_size : g->max_len;
			}
			landing_t ld;
			std::memset(&ld, 0, sizeof(ld));
			ld.send_req = a.req;
			ld.imm = a.imm;
			ld.len = x.msg_size;
			g->landings.push_back(ld);
			l->st.rdma_writes++;
		}
		l->st.write_sends++;
	}
	l->st.payload_bytes += a.size;
	net_req_t *q = take_req(l->send_reqs, kSend, a.req, 1, l);
	if (!q) {
		return -EPROTO;
	}
	*request = q;
	return 0;
}

int irecv_impl(void *recvComm, int n, void **data, const size_t *sizes, int *tags, void **mhandles, void **request)
{
	ofi_amd_net_link *l = link_of(recvComm, 0x52454356);
	if (!l) {
		return -EINVAL;
	}
	*request = nullptr;
	l->st.irecv_calls++;
	int rc = l->progress(false);
	if (rc != 0) {
		return rc;
	}
	uint64_t dsts[OFI_AMD_WIRE_MAX_RECVS], lens[OFI_AMD_WIRE_MAX_RECVS];
	uint64_t keys[OFI_AMD_WIRE_MAX_RECVS * OFI_AMD_WIRE_MAX_RAILS];
	for (int i = 0; i < n; i++) {
		if (sizes[i] > 0xffffffffull) {
			return -EINVAL; /* the control message carries a 32-bit length */
		}
		dsts[i] = reinterpret_cast<uintptr_t>(data[i]);
		lens[i] = sizes[i];
		for (uint32_t r = 0; r < l->num_rails; r++) {
			keys[(uint32_t)i * l->num_rails + r] = reinterpret_cast<uintptr_t>(mhandles[i]);
		}
	}
	int32_t id = -1;
	uint16_t seq = 0;
	/* the control message is written straight into the sending end's mailbox: its post is
	 * complete when recv returns */
	rc = ofi_amd_recv_comm_recv(l->rcv, n, dsts, lens, tags, keys, 0, ofi_amd_send_comm_mailbox(l->sc), &id, &seq);
	if (rc == 0) rc = ofi_amd_recv_comm_ctrl_sent(l->rcv, id);
	if (rc != 0) {
		return rc;
	}
	net_req_t *q = take_req(l->recv_reqs, kRecv, id, (uint8_t)n, l);
	if (!q) {
		return -EPROTO;
	}
	*request = q;
	return 0;
}

} // namespace

extern "C" {

int ofi_amd_net_link_create(uint32_t num_rails, int64_t eager_max_size, uint64_t min_stripe_size,
			    uint64_t max_small_msg_size, uint32_t rx_buffers, void *stream,
			    ofi_amd_net_link_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS || rx_buffers > kMaxRxBuffers ||
	    eager_max_size > 8192) {
		return -EINVAL; /* an rx buffer holds 8 + 8192 bytes */
	}
	*out = nullptr;
	int rc = ofi_amd_gpu_init();
	if (rc != 0) {
		return rc;
	}
	ofi_amd_net_link *l = new (std::nothrow) ofi_amd_net_link;
	if (!l) {
		return -ENOMEM;
	}
	const uint32_t n_rx = rx_buffers ? rx_buffers : 256;
	try {
		l->send_reqs.resize(OFI_AMD_MAX_SEND_REQUESTS);
		l->recv_reqs.resize(OFI_AMD_MAX_REQUESTS);
		l->flush_reqs.resize(OFI_AMD_MAX_REQUESTS);
		l->flush_slots.assign((size_t)OFI_AMD_MAX_REQUESTS * OFI_AMD_WIRE_MAX_RAILS * 8, 0);
		for (group_t &g : l->groups) {
			g.flushes.reserve(OFI_AMD_MAX_REQUESTS);
		}
		for (uint32_t k = n_rx; k > 0; k--) {
			l->rx_free.push_back(k - 1);
		}
		for (group_t &g : l->groups) {
			g.landings.reserve(kGroupEntries);
			g.items.reserve(kGroupEager);
		}
	} catch (...) {
		delete l;
		return -ENOMEM;
	}
	l->num_rails = num_rails;
	l->eager_max_size = eager_max_size;
	l->stream = stream;
	rc = ofi_amd_send_comm_create(1, num_rails, eager_max_size, min_stripe_size ? min_stripe_size : 131072,
				      max_small_msg_size ? max_small_msg_size : 64, &l->sc);
	if (rc == 0) rc = ofi_amd_recv_comm_create(num_rails, &l->rcv);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&l->rx_pool, (size_t)n_rx * kRxStride);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&l->d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(l->d_flush_buf, OFI_AMD_RDMA_FLUSH_SENTINEL, stream);
	for (uint32_t k = 0; k < kGroups && rc == 0; k++) {
		rc = l->groups[k].alloc();
	}
	if (rc != 0) {
		(void)ofi_amd_net_link_destroy(l);
		return rc;
	}
	*out = l;
	return 0;
}

int ofi_amd_net_link_destroy(ofi_amd_net_link_t *l)
{
	if (!l) {
		return -EINVAL;
	}
	/* launches in flight read the pinned tables and write the rx pool */
	const int rc = l->rx_pool ? ofi_amd_gpu_stream_synchronize(l->stream) : 0;
	for (group_t &g : l->groups) {
		g.release();
	}
	if (l->rx_pool) (void)ofi_amd_gpu_mem_free(l->rx_pool);
	if (l->d_flush_buf) (void)ofi_amd_gpu_mem_free(l->d_flush_buf);
	if (l->sc) (void)ofi_amd_send_comm_destroy(l->sc);
	if (l->rcv) (void)ofi_amd_recv_comm_destroy(l->rcv);
	for (auto *pool : { &l->send_reqs, &l->recv_reqs, &l->flush_reqs }) {
		for (net_req_t &q : *pool) {
			q.magic = 0;
		}
	}
	l->send_end.magic = l->recv_end.magic = 0;
	delete l;
	return rc;
}

void *ofi_amd_net_link_send_comm(ofi_amd_net_link_t *l)
{
	return l ? &l->send_end : nullptr;
}

void *ofi_amd_net_link_recv_comm(ofi_amd_net_link_t *l)
{
	return l ? &l->recv_end : nullptr;
}

int ofi_amd_net_link_stats(const ofi_amd_net_link_t *l, ofi_amd_net_link_stats_t *out)
{
	if (!l || !out) {
		return -EINVAL;
	}
	*out = l->st;
	return 0;
}

int ofi_amd_net_link_state(const ofi_amd_net_link_t *l, ofi_amd_send_state_t *send, ofi_amd_recv_state_t *recv)
{
	if (!l || !send || !recv) {
		return -EINVAL;
	}
	ofi_amd_send_comm_state(l->sc, send);
	ofi_amd_recv_comm_state(l->rcv, recv);
	return 0;
}

ncclResult_t ofi_amd_net_isend(void *sendComm, void *data, size_t size, int tag, void *mhandle, void *phandle,
			       void **request)
{
	(void)mhandle;
	(void)phandle; /* "TODO: Add support for network profiling events via pHandles", isend_v10 */
	return ofi_amd::nccl_result_of(isend_impl(sendComm, data, size, tag, request));
}

ncclResult_t ofi_amd_net_irecv(void *recvComm, int n, void **data, size_t *sizes, int *tags, void **mhandles,
			       void **phandles, void **request)
{
	(void)phandles;
	/* the checks of nccl_net_ofi_irecv, src/nccl_ofi_api.cpp:474-510, in its order */
	if (!recvComm || !data || !sizes || !tags || !mhandles || !request) {
		return ncclInvalidArgument;
	}
	if (n <= 0 || n > OFI_AMD_WIRE_MAX_RECVS) {
		return ncclInvalidArgument;
	}
	return ofi_amd::nccl_result_of(irecv_impl(recvComm, n, data, sizes, tags, mhandles, request));
}

ncclResult_t ofi_amd_net_iflush(void *recvComm, int n, void **data, int *sizes, void **mhandles, void **request)
{
	(void)data;
	ofi_amd_net_link *l = link_of(recvComm, 0x52454356);
	/* the checks of nccl_net_ofi_iflush, :538-563 */
	if (!l || n > OFI_AMD_WIRE_MAX_RECVS || !mhandles || !request) {
		return ncclInternalError;
	}
	*request = nullptr;
	if (n < 1 || !sizes) {
		return ncclInternalError;
	}
	int rc = l->progress(true);
	if (rc != 0) {
		return ofi_amd::nccl_result_of(rc);
	}
	int32_t id = -1;
	rc = ofi_amd_recv_comm_flush(l->rcv, n, sizes, &id);
	if (rc != 0 || id < 0) {
		return ofi_amd::nccl_result_of(rc); /* nothing to flush: a NULL request */
	}
	net_req_t *q = take_req(l->flush_reqs, kFlush, id, 0, l);
	if (!q) {
		return ncclSystemError;
	}
	/* the flush rides on the sentinel read-back of the next launch group, which goes behind
	 * everything launched so far; what the receives it covers wrote has been launched, or their
	 * requests would not have completed */
	std::memset(&l->flush_slots[(size_t)id * OFI_AMD_WIRE_MAX_RAILS * 8], 0, OFI_AMD_WIRE_MAX_RAILS * 64);
	l->filling().flushes.push_back(id);
	l->st.flushes++;
	*request = q;
	return ncclSuccess;
}

ncclResult_t ofi_amd_net_test(void *request, int *done, int *sizes)
{
	net_req_t *q = static_cast<net_req_t *>(request);
	if (!q || !done || q->magic != kMagic || !q->link) {
		return ncclInternalError;
	}
	*done = 0;
	ofi_amd_net_link *l = q->link;
	int rc = l->progress(true);
	if (rc != 0) {
		return ofi_amd::nccl_result_of(rc);
	}
	if (q->kind == kSend) {
		uint64_t size = 0;
		rc = ofi_amd_send_comm_test(l->sc, q->id, done, &size);
		if (rc == 0 && *done && sizes) {
			sizes[0] = (int)size;
		}
	} else if (q->kind == kRecv) {
		int got[OFI_AMD_WIRE_MAX_RECVS] = {};
		rc = ofi_amd_recv_comm_test(l->rcv, q->id, done, got);
		if (rc == 0 && *done && sizes) {
			for (uint32_t i = 0; i < q->n; i++) {
				sizes[i] = got[i];
			}
		}
	} else {
		const uint64_t *slots = &l->flush_slots[(size_t)q->id * OFI_AMD_WIRE_MAX_RAILS * 8];
		rc = ofi_amd_recv_comm_flush_test(l->rcv, q->id, slots, l->num_rails, OFI_AMD_RDMA_FLUSH_SENTINEL, done);
	}
	if (rc == 0 && *done) {
		q->magic = 0; /* back in the pool */
	}
	return ofi_amd::nccl_result_of(rc);
}

ncclResult_t ofi_amd_net_isend_v5(void *sendComm, void *data, int size, int tag, void *mhandle, void **request)
{
	return ofi_amd_net_isend(sendComm, data, static_cast<size_t>(size), tag, mhandle, nullptr, request);
}

ncclResult_t ofi_amd_net_irecv_v5(void *recvComm, int n, void **data, int *sizes, int *tags, void **mhandles,
				  void **request)
{
	/* irecv_v5, src/nccl_ofi_interface_nvidia.cpp:524-533 */
	size_t casted[OFI_AMD_WIRE_MAX_RECVS] = { 0 };
	for (int i = 0; sizes && i < n && i < OFI_AMD_WIRE_MAX_RECVS; i++) {
		casted[i] = static_cast<size_t>(sizes[i]);
	}
	return ofi_amd_net_irecv(recvComm, n, data, sizes ? casted : nullptr, tags, mhandles, nullptr, request);
}

ncclResult_t ofi_amd_net_isend_v9(void *sendComm, void *data, size_t size, int tag, void *mhandle, void **request)
{
	return ofi_amd_net_isend(sendComm, data, size, tag, mhandle, nullptr, request);
}

ncclResult_t ofi_amd_net_irecv_v9(void *recvComm, int n, void **data, size_t *sizes, int *tags, void **mhandles,
				  void **request)
{
	return ofi_amd_net_irecv(recvComm, n, data, sizes, tags, mhandles, nullptr, request);
}

} /* extern "C" */

/*
 * The data-path members of ncclNet_vN_t (3rd-party/nccl/cuda/include/nccl/net_v12.h:110-119:
 * isend, irecv, iflush, test) as free functions over this library's send and receive state
 * machines (sendrecv_proto.cpp), a fabric behind three callbacks (ofi_amd_net_fabric_ops_t) and,
 * on the receiving end, the batched eager copy.  The wrappers they stand for:
 * nccl_net_ofi_isend / _irecv / _iflush / _test, src/nccl_ofi_api.cpp:440-567, and the versioned
 * shims of src/nccl_ofi_interface_nvidia.cpp:502-555.
 *
 * A sending end turns what the state machine decides into posts (one eager send, or one write
 * per rail stripe), keeps the posts the fabric refuses in a queue that its progress retries in
 * order, and feeds the completions back.  A receiving end posts control messages and flush
 * reads, hears of eager arrivals and remote writes, and empties matched rx buffers into the
 * posted receives with ofi_amd_eager_copy_batch: the copies of a progress call are one launch,
 * ended by a sentinel read-back, and when the sentinel is seen the copies are reported and the
 * rx buffers handed back to the fabric.  Every entry point progresses its end the way the
 * reference's drain the completion queue: test() always, the posting calls when something of
 * theirs is still queued.
 */
#include <cerrno>
#include <cstring>
#include <deque>
#include <new>
#include <vector>

#include "host_util.hpp"
#include "nccl_translate.hpp"
#include "ofi_amd_hotpath.h"
#include "ofi_amd_net_abi.h"

namespace {

using ofi_amd::pinned_t;

constexpr uint32_t kCopyGroups = 4;      /* eager-copy launches in flight, at most */
constexpr uint32_t kCopyLaunchesKeptBusy = 2;
constexpr uint32_t kCopyGroupItems = 256;
constexpr uint32_t kMagic = 0x4e455451;  /* marks a live request */
constexpr uint32_t kSendMagic = 0x53454e44, kRecvMagic = 0x52454356;
constexpr uint32_t kCqBatch = 16;
/* completion contexts: the kind of post in the top bits, the state machine's request below */
constexpr uint32_t kCtxSend = 1u << 28, kCtxCtrl = 2u << 28, kCtxFlush = 3u << 28, kCtxIdMask = (1u << 28) - 1;

enum req_kind_t : uint8_t { kSend = 1, kRecv = 2, kFlush = 3 };

/* What a request pointer handed to NCCL points to. */
struct net_req_t {
	uint32_t magic = 0;
	uint8_t kind = 0;
	uint8_t n = 0; /* receives of the request */
	int32_t id = -1;
	void *comm = nullptr;
};

net_req_t *take_req(std::vector<net_req_t> &pool, uint8_t kind, int32_t id, uint8_t n, void *comm)
{
	if (id < 0 || (size_t)id >= pool.size() || pool[(size_t)id].magic == kMagic) {
		return nullptr;
	}
	net_req_t &q = pool[(size_t)id];
	q.magic = kMagic;
	q.kind = kind;
	q.n = n;
	q.id = id;
	q.comm = comm;
	return &q;
}

struct comm_base_t {
	uint32_t magic = 0;
	uint32_t num_rails = 0;
	ofi_amd_net_fabric_ops_t ops = {};
	std::deque<ofi_amd_net_post_t> pending; /* posts the fabric refused, oldest first */
	uint64_t refused = 0, progress_calls = 0;

	/* one attempt now, or behind what is already waiting: posts leave in the order they were made
	 * (post_with_pending_retry, src/nccl_ofi_rdma.cpp:1375-1387) */
	int post(const ofi_amd_net_post_t &p)
	{
		if (pending.empty()) {
			const int rc = ops.post(ops.end, &p);
			if (rc != -EAGAIN) {
				return rc;
			}
			refused++;
		}
		try {
			pending.push_back(p);
		} catch (...) {
			return -ENOMEM;
		}
		return 0;
	}

	/* process_pending_reqs, :1421-1460: in order, up to the first post still refused */
	int retry_pending()
	{
		while (!pending.empty()) {
			const int rc = ops.post(ops.end, &pending.front());
			if (rc == -EAGAIN) {
				return 0;
			}
			if (rc != 0) {
				return rc;
			}
			pending.pop_front();
		}
		return 0;
	}
};

struct send_end_t : comm_base_t {
	ofi_amd_send_comm_t *sc = nullptr;
	std::vector<net_req_t> reqs;
	uint64_t isend_calls = 0, isend_again = 0, eager_sends = 0, write_sends = 0, rdma_writes = 0, payload_bytes = 0;

	int progress()
	{
		progress_calls++;
		ofi_amd_net_cqe_t cqe[kCqBatch];
		for (;;) {
			const int n = ops.cq_read(ops.end, cqe, kCqBatch);
			if (n < 0) {
				return n;
			}
			for (int i = 0; i < n; i++) {
				if (cqe[i].kind != OFI_AMD_NET_CQ_POSTED || (cqe[i].context & ~kCtxIdMask) != kCtxSend) {
					return -EPROTO; /* nothing else is addressed to a sending end */
				}
				const int rc = ofi_amd_send_comm_completion(sc, (int32_t)(cqe[i].context & kCtxIdMask));
				if (rc != 0) {
					return rc;
				}
			}
			if (n < (int)kCqBatch) {
				break;
			}
		}
		return retry_pending();
	}
};

struct copy_group_t {
	pinned_t rx, len, dst, cap, copied, done;
	uint32_t n = 0;
	std::vector<ofi_amd_eager_copy_item_t> items;
	int alloc()
	{
		int rc = rx.alloc(sizeof(uint64_t) * kCopyGroupItems);
		if (rc == 0) rc = len.alloc(sizeof(uint32_t) * kCopyGroupItems);
		if (rc == 0) rc = dst.alloc(sizeof(uint64_t) * kCopyGroupItems);
		if (rc == 0) rc = cap.alloc(sizeof(uint32_t) * kCopyGroupItems);
		if (rc == 0) rc = copied.alloc(sizeof(uint32_t) * kCopyGroupItems);
		if (rc == 0) rc = done.alloc(64);
		return rc;
	}
	void release()
	{
		for (pinned_t *p : { &rx, &len, &dst, &cap, &copied, &done }) {
			p->release();
		}
	}
};

struct recv_end_t : comm_base_t {
	ofi_amd_recv_comm_t *rcv = nullptr;
	const void *rx_pool = nullptr;
	void *stream = nullptr;
	void *d_flush_buf = nullptr; /* what a flush reads, and what the copy launches read back */
	pinned_t flush_slots;        /* per flush request: one 64-byte slot per rail */
	std::vector<ofi_amd_ctrl_msg_t> staging; /* control messages on their way to the peer's mailbox */
	copy_group_t groups[kCopyGroups];
	uint32_t head = 0, cur = 0;
	std::vector<net_req_t> recv_reqs, flush_reqs;
	uint64_t irecv_calls = 0, flushes = 0, launches = 0, eager_copies = 0;

	/* copy launches whose sentinel has arrived: the receives hear of their bytes, the rx buffers
	 * go back to the fabric */
	int reap_copies()
	{
		while (head != cur) {
			copy_group_t &g = groups[head % kCopyGroups];
			if (ofi_amd_flush_test(g.done.host, 1, OFI_AMD_RDMA_FLUSH_SENTINEL) != 1) {
				break;
			}
			for (uint32_t k = 0; k < g.n; k++) {
				const ofi_amd_eager_copy_item_t &it = g.items[k];
				const uint32_t want = it.recv_len < it.dst_len ? it.recv_len : (uint32_t)it.dst_len;
				if (g.copied.as<uint32_t>()[k] != want) {
					return -EIO;
				}
				int rc = ofi_amd_recv_comm_copy_done(rcv, it.req, it.sub_idx);
				if (rc == 0) rc = ops.repost_rx(ops.end, it.rx_cookie);
				if (rc != 0) {
					return rc;
				}
				eager_copies++;
			}
			g.n = 0;
			g.items.clear();
			head++;
		}
		return 0;
	}

	/* everything matched since the last call leaves its rx buffer in one launch; while two
	 * launches are in flight the matches keep gathering in the state machine's queue instead
	 * of leaving a few at a time */
	int launch_copies()
	{
		while (cur - head < kCopyLaunchesKeptBusy) {
			copy_group_t &g = groups[cur % kCopyGroups];
			while (g.n < kCopyGroupItems) {
				ofi_amd_eager_copy_item_t it;
				if (ofi_amd_recv_comm_take_copies(rcv, &it, 1) == 0) {
					break;
				}
				if (!it.needs_copy) { /* a zero-length message: nothing to move */
					const int rc = ops.repost_rx(ops.end, it.rx_cookie);
					if (rc != 0) {
						return rc;
					}
					continue;
				}
				const uint32_t k = g.n++;
				g.items.push_back(it);
				g.rx.as<uint64_t>()[k] = it.rx_cookie;
				g.len.as<uint32_t>()[k] = it.recv_len;
				g.dst.as<uint64_t>()[k] = it.dst;
				g.cap.as<uint32_t>()[k] = (uint32_t)it.dst_len;
			}
			if (g.n == 0) {
				return 0;
			}
			int rc = ofi_amd_eager_copy_batch(rx_pool, g.rx.dev_as<uint64_t>(), g.len.dev_as<uint32_t>(), nullptr,
							  g.dst.dev_as<uint64_t>(), g.cap.dev_as<uint32_t>(), g.n,
							  static_cast<uint32_t *>(g.copied.dev), nullptr, stream);
			if (rc == 0) {
				__atomic_store_n(g.done.as<uint64_t>(), 0ull, __ATOMIC_RELEASE);
				rc = ofi_amd_flush_post(d_flush_buf, g.done.dev, 1, stream);
			}
			if (rc != 0) {
				return rc;
			}
			launches += 2;
			cur++;
			if (g.n < kCopyGroupItems) {
				return 0;
			}
		}
		return 0;
	}

	int progress()
	{
		progress_calls++;
		ofi_amd_net_cqe_t cqe[kCqBatch];
		for (;;) {
			const int n = ops.cq_read(ops.end, cqe, kCqBatch);
			if (n < 0) {
				return n;
			}
			for (int i = 0; i < n; i++) {
				const ofi_amd_net_cqe_t &c = cqe[i];
				int rc = 0;
				if (c.kind == OFI_AMD_NET_CQ_EAGER) {
					uint32_t comm_id, seq, recv_idx, nseg;
					ofi_amd_rdma_imm_decode(c.imm, &comm_id, &seq, &recv_idx, &nseg);
					rc = ofi_amd_recv_comm_eager_arrival(rcv, (uint16_t)seq, &c.hdr, (uint32_t)c.len, c.rx_cookie);
				} else if (c.kind == OFI_AMD_NET_CQ_WRITE) {
					rc = ofi_amd_recv_comm_write_arrival(rcv, c.imm, c.len);
				} else if (c.kind == OFI_AMD_NET_CQ_POSTED && (c.context & ~kCtxIdMask) == kCtxCtrl) {
					rc = ofi_amd_recv_comm_ctrl_sent(rcv, (int32_t)(c.context & kCtxIdMask));
				} else if (c.kind == OFI_AMD_NET_CQ_POSTED && (c.context & ~kCtxIdMask) == kCtxFlush) {
					rc = 0; /* the slots say when a flush is done, not its reads' completions */
				} else {
					rc = -EPROTO;
				}
				if (rc != 0) {
					return rc;
				}
			}
			if (n < (int)kCqBatch) {
				break;
			}
		}
		int rc = retry_pending();
		if (rc == 0) rc = reap_copies();
		if (rc == 0) rc = launch_copies();
		return rc;
	}
};

send_end_t *send_end_of(void *comm)
{
	send_end_t *s = static_cast<send_end_t *>(comm);
	return (s && s->magic == kSendMagic) ? s : nullptr;
}

recv_end_t *recv_end_of(void *comm)
{
	recv_end_t *r = static_cast<recv_end_t *>(comm);
	return (r && r->magic == kRecvMagic) ? r : nullptr;
}

int isend_impl(void *sendComm, void *data, size_t size, int tag, void **request)
{
	if (request) {
		*request = nullptr;
	}
	send_end_t *s = send_end_of(sendComm);
	if (!s || !request || (!data && size)) {
		return -EINVAL; /* bytes from address 0 would be a fault on the device, not an error code */
	}
	s->isend_calls++;
	/* process_cq_if_pending (src/nccl_ofi_rdma.cpp:3523-3545, called at :5682-5692): the queue is
	 * looked at when posts of this end are still waiting, and while they still are afterwards the
	 * network is busy: "Return NULL to NCCL" */
	if (!s->pending.empty()) {
		const int rc = s->progress();
		if (rc != 0) {
			return rc;
		}
		if (!s->pending.empty()) {
			s->isend_again++;
			return 0;
		}
	}
	ofi_amd_send_action_t a;
	int rc = ofi_amd_send_comm_send(s->sc, size, tag, &a);
	if (rc != 0) {
		return rc;
	}
	if (a.kind == OFI_AMD_SEND_AGAIN) {
		s->isend_again++;
		/* no control message for it yet, and it cannot go eager: look at the fabric before the
		 * caller asks again */
		return s->progress();
	}
	net_req_t *q = take_req(s->reqs, kSend, a.req, 1, s);
	if (!q) {
		return -EPROTO;
	}
	ofi_amd_net_post_t p;
	std::memset(&p, 0, sizeof(p));
	p.context = kCtxSend | (uint32_t)a.req;
	p.imm = a.imm;
	const uint64_t from = reinterpret_cast<uintptr_t>(data);
	if (a.kind == OFI_AMD_SEND_EAGER) {
		p.kind = OFI_AMD_NET_POST_EAGER;
		p.rail = a.num_xfers ? a.xfers[0].rail_id : 0;
		p.src = from;
		p.len = a.size;
		p.hdr = a.hdr;
		rc = s->post(p);
		s->eager_sends++;
	} else {
		if (a.num_xfers == 0) {
			rc = -EPROTO; /* a write message always has a schedule, if only of one empty stripe */
		}
		p.kind = OFI_AMD_NET_POST_WRITE;
		for (uint32_t k = 0; k < a.num_xfers && rc == 0; k++) {
			const ofi_amd_xfer_info_t &x = a.xfers[k];
			p.rail = x.rail_id;
			p.src = from + x.offset;
			p.len = x.msg_size;
			p.dest = a.remote_buff_offset + x.offset;
			p.key = a.mr_key[x.rail_id < OFI_AMD_WIRE_MAX_RAILS ? x.rail_id : 0];
			rc = s->post(p);
			s->rdma_writes++;
		}
		s->write_sends++;
	}
	if (rc != 0) {
		q->magic = 0;
		return rc;
	}
	s->payload_bytes += a.size;
	*request = q;
	return 0;
}

int irecv_impl(void *recvComm, int n, void **data, const size_t *sizes, int *tags, void **mhandles, void **request)
{
	recv_end_t *r = recv_end_of(recvComm);
	if (!r) {
		return -EINVAL;
	}
	*request = nullptr;
	r->irecv_calls++;
	if (!r->pending.empty()) { /* as in isend: :3595-3605 */
		const int rc = r->progress();
		if (rc != 0) {
			return rc;
		}
		if (!r->pending.empty()) {
			return 0; /* network busy: a NULL request */
		}
	}
	uint64_t dsts[OFI_AMD_WIRE_MAX_RECVS], lens[OFI_AMD_WIRE_MAX_RECVS];
	uint64_t keys[OFI_AMD_WIRE_MAX_RECVS * OFI_AMD_WIRE_MAX_RAILS];
	for (int i = 0; i < n; i++) {
		if (sizes[i] > 0xffffffffull || (!data[i] && sizes[i])) {
			return -EINVAL; /* the control message carries a 32-bit length; no receive into address 0 */
		}
		dsts[i] = reinterpret_cast<uintptr_t>(data[i]);
		lens[i] = sizes[i];
		for (uint32_t k = 0; k < r->num_rails; k++) {
			keys[(uint32_t)i * r->num_rails + k] = reinterpret_cast<uintptr_t>(mhandles[i]);
		}
	}
	int32_t id = -1;
	uint16_t seq = 0;
	/* the control message is built in the staging copy of the mailbox and written to the peer's
	 * slot of the same number (rdma_recv_req::post, src/nccl_ofi_rdma.cpp:2566-2615) */
	int rc = ofi_amd_recv_comm_recv(r->rcv, n, dsts, lens, tags, keys, 0, r->staging.data(), &id, &seq);
	if (rc != 0) {
		return rc;
	}
	net_req_t *q = take_req(r->recv_reqs, kRecv, id, (uint8_t)n, r);
	if (!q) {
		return -EPROTO;
	}
	const uint32_t slot = ofi_amd_ctrl_mailbox_slot(seq);
	ofi_amd_net_post_t p;
	std::memset(&p, 0, sizeof(p));
	p.kind = OFI_AMD_NET_POST_CTRL;
	p.context = kCtxCtrl | (uint32_t)id;
	p.src = reinterpret_cast<uintptr_t>(&r->staging[slot]);
	p.len = (uint64_t)n * sizeof(ofi_amd_ctrl_entry_t);
	p.dest = (uint64_t)slot * sizeof(ofi_amd_ctrl_msg_t);
	rc = r->post(p);
	if (rc != 0) {
		q->magic = 0;
		return rc;
	}
	*request = q;
	return 0;
}

} // namespace

/* the in-process link: a fabric and the two comms over it */
struct ofi_amd_net_link {
	ofi_amd_netfab_t *fab = nullptr;
	void *send_comm = nullptr, *recv_comm = nullptr;
};

extern "C" {

int ofi_amd_net_send_comm_create(uint32_t num_rails, int64_t eager_max_size, uint64_t min_stripe_size,
				 uint64_t max_small_msg_size, const ofi_amd_net_fabric_ops_t *fabric, void **sendComm)
{
	if (!sendComm || !fabric || !fabric->post || !fabric->cq_read || num_rails < 1 ||
	    num_rails > OFI_AMD_WIRE_MAX_RAILS || eager_max_size > 8192) {
		return -EINVAL; /* an rx buffer holds 8 + 8184 bytes */
	}
	*sendComm = nullptr;
	send_end_t *s = new (std::nothrow) send_end_t;
	if (!s) {
		return -ENOMEM;
	}
	try {
		s->reqs.resize(OFI_AMD_MAX_SEND_REQUESTS);
	} catch (...) {
		delete s;
		return -ENOMEM;
	}
	const int rc = ofi_amd_send_comm_create(1, num_rails, eager_max_size, min_stripe_size ? min_stripe_size : 131072,
						max_small_msg_size ? max_small_msg_size : 64, &s->sc);
	if (rc != 0) {
		delete s;
		return rc;
	}
	s->num_rails = num_rails;
	s->ops = *fabric;
	s->magic = kSendMagic;
	*sendComm = s;
	return 0;
}

void *ofi_amd_net_send_comm_mailbox(void *sendComm)
{
	send_end_t *s = send_end_of(sendComm);
	return s ? ofi_amd_send_comm_mailbox(s->sc) : nullptr;
}

int ofi_amd_net_recv_comm_create(uint32_t num_rails, const ofi_amd_net_fabric_ops_t *fabric, const void *rx_pool_base,
				 void *stream, void **recvComm)
{
	if (!recvComm || !fabric || !fabric->post || !fabric->cq_read || !fabric->repost_rx || !rx_pool_base ||
	    num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS) {
		return -EINVAL;
	}
	*recvComm = nullptr;
	int rc = ofi_amd_gpu_init();
	if (rc != 0) {
		return rc;
	}
	recv_end_t *r = new (std::nothrow) recv_end_t;
	if (!r) {
		return -ENOMEM;
	}
	try {
		r->recv_reqs.resize(OFI_AMD_MAX_REQUESTS);
		r->flush_reqs.resize(OFI_AMD_MAX_REQUESTS);
		r->staging.resize(OFI_AMD_CTRL_MAILBOX_SIZE);
		std::memset(r->staging.data(), 0, r->staging.size() * sizeof(ofi_amd_ctrl_msg_t));
		for (copy_group_t &g : r->groups) {
			g.items.reserve(kCopyGroupItems);
		}
	} catch (...) {
		delete r;
		return -ENOMEM;
	}
	r->num_rails = num_rails;
	r->ops = *fabric;
	r->rx_pool = rx_pool_base;
	r->stream = stream;
	r->magic = kRecvMagic;
	rc = ofi_amd_recv_comm_create(num_rails, &r->rcv);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&r->d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(r->d_flush_buf, OFI_AMD_RDMA_FLUSH_SENTINEL, stream);
	if (rc == 0) rc = r->flush_slots.alloc((size_t)OFI_AMD_MAX_REQUESTS * OFI_AMD_WIRE_MAX_RAILS * 64);
	for (uint32_t k = 0; k < kCopyGroups && rc == 0; k++) {
		rc = r->groups[k].alloc();
	}
	if (rc != 0) {
		(void)ofi_amd_net_comm_destroy(r);
		return rc;
	}
	*recvComm = r;
	return 0;
}

int ofi_amd_net_comm_destroy(void *comm)
{
	if (send_end_t *s = send_end_of(comm)) {
		for (net_req_t &q : s->reqs) {
			q.magic = 0;
		}
		if (s->sc) (void)ofi_amd_send_comm_destroy(s->sc);
		s->magic = 0;
		delete s;
		return 0;
	}
	recv_end_t *r = recv_end_of(comm);
	if (!r) {
		return -EINVAL;
	}
	/* copy launches in flight read the pinned tables */
	const int rc = r->d_flush_buf ? ofi_amd_gpu_stream_synchronize(r->stream) : 0;
	for (copy_group_t &g : r->groups) {
		g.release();
	}
	r->flush_slots.release();
	if (r->d_flush_buf) (void)ofi_amd_gpu_mem_free(r->d_flush_buf);
	if (r->rcv) (void)ofi_amd_recv_comm_destroy(r->rcv);
	for (auto *pool : { &r->recv_reqs, &r->flush_reqs }) {
		for (net_req_t &q : *pool) {
			q.magic = 0;
		}
	}
	r->magic = 0;
	delete r;
	return rc;
}

int ofi_amd_net_link_create(uint32_t num_rails, int64_t eager_max_size, uint64_t min_stripe_size,
			    uint64_t max_small_msg_size, uint32_t rx_buffers, void *stream,
			    ofi_amd_net_link_t **out)
{
	if (!out) {
		return -EINVAL;
	}
	*out = nullptr;
	if (eager_max_size > 8192) {
		return -EINVAL;
	}
	ofi_amd_net_link *l = new (std::nothrow) ofi_amd_net_link;
	if (!l) {
		return -ENOMEM;
	}
	ofi_amd_net_fabric_ops_t send_ops, recv_ops;
	int rc = ofi_amd_netfab_create(num_rails, rx_buffers, stream, &l->fab);
	if (rc == 0) rc = ofi_amd_netfab_ops(l->fab, &send_ops, &recv_ops);
	if (rc == 0) {
		rc = ofi_amd_net_send_comm_create(num_rails, eager_max_size, min_stripe_size, max_small_msg_size, &send_ops,
						  &l->send_comm);
	}
	if (rc == 0) {
		rc = ofi_amd_net_recv_comm_create(num_rails, &recv_ops, ofi_amd_netfab_rx_pool(l->fab), stream, &l->recv_comm);
	}
	if (rc == 0) rc = ofi_amd_netfab_connect(l->fab, ofi_amd_net_send_comm_mailbox(l->send_comm));
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
	int rc = 0;
	if (l->recv_comm) rc = ofi_amd_net_comm_destroy(l->recv_comm);
	if (l->send_comm) (void)ofi_amd_net_comm_destroy(l->send_comm);
	if (l->fab) {
		const int e = ofi_amd_netfab_destroy(l->fab); /* waits for the wire's launches */
		rc = rc ? rc : e;
	}
	delete l;
	return rc;
}

void *ofi_amd_net_link_send_comm(ofi_amd_net_link_t *l)
{
	return l ? l->send_comm : nullptr;
}

void *ofi_amd_net_link_recv_comm(ofi_amd_net_link_t *l)
{
	return l ? l->recv_comm : nullptr;
}

int ofi_amd_net_link_stats(const ofi_amd_net_link_t *l, ofi_amd_net_link_stats_t *out)
{
	if (!l || !out) {
		return -EINVAL;
	}
	const send_end_t *s = send_end_of(l->send_comm);
	const recv_end_t *r = recv_end_of(l->recv_comm);
	if (!s || !r) {
		return -EINVAL;
	}
	std::memset(out, 0, sizeof(*out));
	out->isend_calls = s->isend_calls;
	out->isend_again = s->isend_again;
	out->eager_sends = s->eager_sends;
	out->write_sends = s->write_sends;
	out->rdma_writes = s->rdma_writes;
	out->payload_bytes = s->payload_bytes;
	out->irecv_calls = r->irecv_calls;
	out->flushes = r->flushes;
	out->eager_copies = r->eager_copies;
	out->progress_calls = s->progress_calls + r->progress_calls;
	out->posts_refused = s->refused + r->refused;
	uint64_t wire_launches = 0;
	(void)ofi_amd_netfab_counts(l->fab, &wire_launches, &out->copy_entries);
	out->launches = wire_launches + r->launches;
	return 0;
}

int ofi_amd_net_link_state(const ofi_amd_net_link_t *l, ofi_amd_send_state_t *send, ofi_amd_recv_state_t *recv)
{
	if (!l || !send || !recv) {
		return -EINVAL;
	}
	const send_end_t *s = send_end_of(l->send_comm);
	const recv_end_t *r = recv_end_of(l->recv_comm);
	if (!s || !r) {
		return -EINVAL;
	}
	ofi_amd_send_comm_state(s->sc, send);
	ofi_amd_recv_comm_state(r->rcv, recv);
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
	recv_end_t *r = recv_end_of(recvComm);
	/* the checks of nccl_net_ofi_iflush, :538-563 */
	if (!r || n > OFI_AMD_WIRE_MAX_RECVS || !mhandles || !request) {
		return ncclInternalError;
	}
	*request = nullptr;
	if (n < 1 || !sizes) {
		return ncclInternalError;
	}
	/* process_cq_if_pending, src/nccl_ofi_rdma.cpp:4431-4439; a flush asked for while the network
	 * is busy joins the queue behind what is waiting (:4480-4495), which post() does */
	int rc = r->pending.empty() ? 0 : r->progress();
	if (rc != 0) {
		return ofi_amd::nccl_result_of(rc);
	}
	int32_t id = -1;
	rc = ofi_amd_recv_comm_flush(r->rcv, n, sizes, &id);
	if (rc != 0 || id < 0) {
		return ofi_amd::nccl_result_of(rc); /* nothing to flush: a NULL request */
	}
	net_req_t *q = take_req(r->flush_reqs, kFlush, id, 0, r);
	if (!q) {
		return ncclSystemError;
	}
	/* one read of the flush buffer per rail into the request's host slots (rdma_flush_req::post,
	 * :2664-2713); the slots, not the reads' completions, say when it is done */
	uint8_t *slots = r->flush_slots.as<uint8_t>() + (size_t)id * OFI_AMD_WIRE_MAX_RAILS * 64;
	std::memset(slots, 0, OFI_AMD_WIRE_MAX_RAILS * 64);
	ofi_amd_net_post_t p;
	std::memset(&p, 0, sizeof(p));
	p.kind = OFI_AMD_NET_POST_FLUSH;
	p.context = kCtxFlush | (uint32_t)id;
	p.len = 64;
	p.dest = reinterpret_cast<uintptr_t>(r->d_flush_buf);
	for (uint32_t rail = 0; rail < r->num_rails && rc == 0; rail++) {
		p.rail = rail;
		p.src = reinterpret_cast<uintptr_t>(slots + rail * 64);
		rc = r->post(p);
	}
	if (rc != 0) {
		q->magic = 0;
		return ofi_amd::nccl_result_of(rc);
	}
	r->flushes++;
	*request = q;
	return ncclSuccess;
}

ncclResult_t ofi_amd_net_test(void *request, int *done, int *sizes)
{
	net_req_t *q = static_cast<net_req_t *>(request);
	if (!q || !done || q->magic != kMagic || !q->comm) {
		return ncclInternalError;
	}
	*done = 0;
	int rc;
	if (q->kind == kSend) {
		send_end_t *s = static_cast<send_end_t *>(q->comm);
		rc = s->progress();
		uint64_t size = 0;
		if (rc == 0) rc = ofi_amd_send_comm_test(s->sc, q->id, done, &size);
		if (rc == 0 && *done && sizes) {
			sizes[0] = (int)size;
		}
	} else {
		recv_end_t *r = static_cast<recv_end_t *>(q->comm);
		rc = r->progress();
		if (rc == 0 && q->kind == kRecv) {
			int got[OFI_AMD_WIRE_MAX_RECVS] = {};
			rc = ofi_amd_recv_comm_test(r->rcv, q->id, done, got);
			if (rc == 0 && *done && sizes) {
				for (uint32_t i = 0; i < q->n; i++) {
					sizes[i] = got[i];
				}
			}
		} else if (rc == 0) {
			const uint8_t *slots = r->flush_slots.as<uint8_t>() + (size_t)q->id * OFI_AMD_WIRE_MAX_RAILS * 64;
			rc = ofi_amd_recv_comm_flush_test(r->rcv, q->id, slots, r->num_rails, OFI_AMD_RDMA_FLUSH_SENTINEL, done);
		}
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

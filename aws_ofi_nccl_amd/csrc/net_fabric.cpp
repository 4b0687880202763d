/*
 * The fabric of an in-process send/receive link (ofi_amd_netfab_*): what libfabric, the NIC and
 * the wire are to the reference's two ranks, for two comms inside one process on one GPU.
 *
 * A post becomes entries of a device copy table: an eager send is the 8-byte header (staged in
 * pinned memory) and the payload into an rx buffer, a write one entry; a flush read rides on
 * the sentinel read-back of a group (the same 64 bytes of the flush buffer, read once for all
 * the flushes waiting).  A control message is copied into the sending
 * end's mailbox at once.  Posts gather in a launch group; a group leaves on the stream as one
 * ofi_amd_copy_table_pieces launch and a sentinel read-back, and when the sentinel is seen its
 * completions are put on the two ends' queues in posting order: for an eager send the arrival
 * on the receiving end and the completion on the sending end, and so on.
 */
#include <cerrno>
#include <cstring>
#include <deque>
#include <new>
#include <vector>

#include "host_util.hpp"
#include "ofi_amd_hotpath.h"
#include "ofi_amd_net_abi.h"

namespace {

using ofi_amd::pinned_t;

constexpr uint32_t kRxStride = 8320;    /* 8192 + header room, rounded to the 128-byte rx alignment */
constexpr uint32_t kMaxRxBuffers = 256; /* the receiving end queues at most 256 eager arrivals */
constexpr uint32_t kGroups = 8;         /* launch groups in flight, at most */
constexpr uint32_t kGroupsKeptBusy = 2; /* in flight before posts start gathering instead of leaving at once */
constexpr uint32_t kGroupEntries = 512; /* table entries of a group */

struct landed_t {
	bool to_recv_end; /* which queue the entry goes to */
	ofi_amd_net_cqe_t cqe;
};

/* A flush read that rides on a group's sentinel read-back instead of being a read of its own. */
struct rider_t {
	uint64_t host_slot;
	uint32_t context;
};

struct group_t {
	pinned_t src, dst, len, hdrs, done;
	uint32_t n_copy = 0, n_hdr = 0, max_len = 0;
	std::vector<landed_t> landings;
	std::vector<rider_t> riders;
	int alloc()
	{
		int rc = src.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = dst.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = len.alloc(sizeof(uint32_t) * kGroupEntries);
		if (rc == 0) rc = hdrs.alloc(sizeof(ofi_amd_eager_hdr_t) * kGroupEntries);
		if (rc == 0) rc = done.alloc(64);
		return rc;
	}
	void release()
	{
		for (pinned_t *p : { &src, &dst, &len, &hdrs, &done }) {
			p->release();
		}
	}
	/* a transfer without bytes (a zero-length write) still waits for its group's sentinel */
	bool empty() const { return n_copy == 0 && landings.empty() && riders.empty(); }
	/* every post adds at most two landings; a zero-length write adds them without a table entry */
	bool room(uint32_t entries) const
	{
		return n_copy + entries <= kGroupEntries && landings.size() + 2 <= 2 * kGroupEntries;
	}
	void add(uint64_t from, uint64_t to, uint64_t bytes)
	{
		src.as<uint64_t>()[n_copy] = from;
		dst.as<uint64_t>()[n_copy] = to;
		len.as<uint32_t>()[n_copy++] = (uint32_t)bytes;
		max_len = max_len < (uint32_t)bytes ? (uint32_t)bytes : max_len;
	}
	void reset()
	{
		n_copy = n_hdr = max_len = 0;
		landings.clear();
		riders.clear();
	}
};

} // namespace

struct ofi_amd_netfab {
	/* an end is a tagged pointer into this object: the callbacks get it as `end` */
	struct end_t {
		ofi_amd_netfab *fab;
		bool recv_end;
		std::deque<ofi_amd_net_cqe_t> cq;
	} send_end = { this, false, {} }, recv_end = { this, true, {} };
	uint32_t num_rails = 0;
	void *stream = nullptr;
	void *rx_pool = nullptr;
	std::vector<uint32_t> rx_free;
	uint32_t n_rx = 0;
	bool rx_is_free[kMaxRxBuffers] = {}; /* a buffer handed back twice would take two messages at once */
	void *d_flush_buf = nullptr; /* the sentinel the groups read back */
	uint8_t *mailbox = nullptr;  /* the sending end's, 256 slots of 512 bytes */
	group_t groups[kGroups];
	uint32_t head = 0, cur = 0; /* positions: head = oldest launched group, cur = the one being filled */
	uint64_t n_launches = 0, n_entries = 0;

	group_t &filling() { return groups[cur % kGroups]; }

	void landed(bool to_recv_end, uint32_t kind, uint32_t context, uint32_t imm, uint64_t len, uint64_t rx_cookie,
		    const ofi_amd_eager_hdr_t *hdr)
	{
		landed_t l;
		std::memset(&l, 0, sizeof(l));
		l.to_recv_end = to_recv_end;
		l.cqe.kind = kind;
		l.cqe.context = context;
		l.cqe.imm = imm;
		l.cqe.len = len;
		l.cqe.rx_cookie = rx_cookie;
		if (hdr) {
			l.cqe.hdr = *hdr;
		}
		filling().landings.push_back(l);
	}

	int post(end_t *e, const ofi_amd_net_post_t *p)
	{
		if (!p || p->rail >= num_rails || p->len > 0xffffffffull) {
			return -EINVAL;
		}
		group_t &g = filling();
		switch (p->kind) {
		case OFI_AMD_NET_POST_EAGER: {
			if (e->recv_end || p->len > kRxStride - OFI_AMD_EAGER_HEADER_SIZE || (p->len && p->src == 0)) {
				return -EINVAL;
			}
			if (rx_free.empty() || !g.room(2)) {
				return -EAGAIN; /* no rx buffer posted at the receiving end, or no room in the table */
			}
			const uint32_t slot = rx_free.back();
			rx_free.pop_back();
			rx_is_free[slot] = false;
			const uint64_t rx = reinterpret_cast<uintptr_t>(rx_pool) + (uint64_t)slot * kRxStride;
			g.hdrs.as<ofi_amd_eager_hdr_t>()[g.n_hdr] = p->hdr;
			g.add(reinterpret_cast<uintptr_t>(g.hdrs.dev) + g.n_hdr * sizeof(ofi_amd_eager_hdr_t), rx,
			      OFI_AMD_EAGER_HEADER_SIZE);
			g.n_hdr++;
			if (p->len) {
				g.add(p->src, rx + OFI_AMD_EAGER_HEADER_SIZE, p->len);
			}
			landed(true, OFI_AMD_NET_CQ_EAGER, 0, p->imm, p->len, (uint64_t)slot * kRxStride, &p->hdr);
			landed(false, OFI_AMD_NET_CQ_POSTED, p->context, 0, 0, 0, nullptr);
			return 0;
		}
		case OFI_AMD_NET_POST_WRITE:
			if (e->recv_end || (p->len && (p->src == 0 || p->dest == 0))) {
				return -EINVAL; /* a copy from or to address 0 would be a fault on the device */
			}
			if (!g.room(1)) {
				return -EAGAIN;
			}
			if (p->len) {
				g.add(p->src, p->dest, p->len);
			}
			landed(true, OFI_AMD_NET_CQ_WRITE, 0, p->imm, p->len, 0, nullptr);
			landed(false, OFI_AMD_NET_CQ_POSTED, p->context, 0, 0, 0, nullptr);
			return 0;
		case OFI_AMD_NET_POST_CTRL: {
			constexpr uint64_t kMailboxBytes = 256u * sizeof(ofi_amd_ctrl_msg_t);
			if (!e->recv_end || !mailbox || p->src == 0 || p->dest > kMailboxBytes || p->len > kMailboxBytes - p->dest) {
				return -EINVAL;
			}
			/* entry 0's sequence number is the ready mark: it goes in last */
			const uint8_t *from = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p->src));
			const size_t mark = offsetof(ofi_amd_ctrl_entry_t, msg_seq_num);
			if (p->len > mark + sizeof(uint16_t)) {
				std::memcpy(mailbox + p->dest + mark + sizeof(uint16_t), from + mark + sizeof(uint16_t),
					    p->len - mark - sizeof(uint16_t));
			}
			std::memcpy(mailbox + p->dest, from, p->len < mark ? p->len : mark);
			if (p->len >= mark + sizeof(uint16_t)) {
				uint16_t seq;
				std::memcpy(&seq, from + mark, sizeof(seq));
				__atomic_store_n(reinterpret_cast<uint16_t *>(mailbox + p->dest + mark), seq, __ATOMIC_RELEASE);
			}
			ofi_amd_net_cqe_t c;
			std::memset(&c, 0, sizeof(c));
			c.kind = OFI_AMD_NET_CQ_POSTED;
			c.context = p->context;
			e->cq.push_back(c);
			return 0;
		}
		case OFI_AMD_NET_POST_FLUSH: {
			if (!e->recv_end || p->len != 64 || p->src == 0) {
				return -EINVAL;
			}
			/* A flush is asked for after receives have completed, and a receive completes here
			 * only once the sentinel behind its copies has been seen: every write the flush has to
			 * be ordered behind has landed.  Its read of the flush buffer therefore rides on a
			 * read-back that is on its way anyway -- that of the newest group in flight -- and
			 * only with nothing in flight on that of the group being filled. */
			group_t &carrier = head != cur ? groups[(cur - 1) % kGroups] : g;
			carrier.riders.push_back(rider_t{ p->src, p->context });
			return 0;
		}
		default:
			return -EINVAL;
		}
	}

	void reap()
	{
		while (head != cur) {
			group_t &g = groups[head % kGroups];
			if (ofi_amd_flush_test(g.done.host, 1, OFI_AMD_RDMA_FLUSH_SENTINEL) != 1) {
				break;
			}
			for (const landed_t &l : g.landings) {
				(l.to_recv_end ? recv_end : send_end).cq.push_back(l.cqe);
			}
			/* what the group's read-back read from the flush buffer is what its riders read */
			const uint64_t word = __atomic_load_n(g.done.as<uint64_t>(), __ATOMIC_ACQUIRE);
			for (const rider_t &r : g.riders) {
				__atomic_store_n(reinterpret_cast<uint64_t *>(static_cast<uintptr_t>(r.host_slot)), word, __ATOMIC_RELEASE);
				ofi_amd_net_cqe_t c;
				std::memset(&c, 0, sizeof(c));
				c.kind = OFI_AMD_NET_CQ_POSTED;
				c.context = r.context;
				recv_end.cq.push_back(c);
			}
			g.reset();
			head++;
		}
	}

	/* `now`: the caller has polled and found nothing */
	int launch(bool now)
	{
		group_t &g = filling();
		if (g.empty() || cur - head >= kGroups - 1) {
			return 0;
		}
		const bool full = !g.room(OFI_AMD_WIRE_MAX_RAILS + 2);
		if (!full && (!now || cur - head >= kGroupsKeptBusy)) {
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
				n_launches++;
			}
			n_entries += g.n_copy;
		}
		if (rc == 0) {
			__atomic_store_n(g.done.as<uint64_t>(), 0ull, __ATOMIC_RELEASE);
			rc = ofi_amd_flush_post(d_flush_buf, g.done.dev, 1, stream);
			n_launches++;
		}
		if (rc == 0) {
			cur++;
		}
		return rc;
	}

	int cq_read(end_t *e, ofi_amd_net_cqe_t *out, uint32_t max)
	{
		if (!out) {
			return -EINVAL;
		}
		reap();
		const int rc = launch(e->cq.empty());
		if (rc != 0) {
			return rc;
		}
		uint32_t n = 0;
		while (n < max && !e->cq.empty()) {
			out[n++] = e->cq.front();
			e->cq.pop_front();
		}
		return (int)n;
	}

	static int post_cb(void *end, const ofi_amd_net_post_t *p)
	{
		end_t *e = static_cast<end_t *>(end);
		return e->fab->post(e, p);
	}
	static int cq_read_cb(void *end, ofi_amd_net_cqe_t *out, uint32_t max)
	{
		end_t *e = static_cast<end_t *>(end);
		return e->fab->cq_read(e, out, max);
	}
	static int repost_rx_cb(void *end, uint64_t rx_cookie)
	{
		end_t *e = static_cast<end_t *>(end);
		ofi_amd_netfab *f = e->fab;
		if (!e->recv_end || rx_cookie % kRxStride != 0 || rx_cookie / kRxStride >= f->n_rx ||
		    f->rx_is_free[rx_cookie / kRxStride]) {
			return -EINVAL;
		}
		f->rx_is_free[rx_cookie / kRxStride] = true;
		f->rx_free.push_back((uint32_t)(rx_cookie / kRxStride)); /* within the capacity reserved at creation */
		return 0;
	}
};

extern "C" {

int ofi_amd_netfab_create(uint32_t num_rails, uint32_t rx_buffers, void *stream, ofi_amd_netfab_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS || rx_buffers > kMaxRxBuffers) {
		return -EINVAL;
	}
	*out = nullptr;
	int rc = ofi_amd_gpu_init();
	if (rc != 0) {
		return rc;
	}
	ofi_amd_netfab *f = new (std::nothrow) ofi_amd_netfab;
	if (!f) {
		return -ENOMEM;
	}
	const uint32_t n_rx = rx_buffers ? rx_buffers : kMaxRxBuffers;
	try {
		f->rx_free.reserve(n_rx);
		for (uint32_t k = n_rx; k > 0; k--) {
			f->rx_free.push_back(k - 1);
			f->rx_is_free[k - 1] = true;
		}
		f->n_rx = n_rx;
		for (group_t &g : f->groups) {
			g.landings.reserve(2 * kGroupEntries);
			g.riders.reserve(OFI_AMD_MAX_REQUESTS * OFI_AMD_WIRE_MAX_RAILS);
		}
	} catch (...) {
		delete f;
		return -ENOMEM;
	}
	f->num_rails = num_rails;
	f->stream = stream;
	rc = ofi_amd_gpu_mem_alloc(&f->rx_pool, (size_t)n_rx * kRxStride);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&f->d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(f->d_flush_buf, OFI_AMD_RDMA_FLUSH_SENTINEL, stream);
	for (uint32_t k = 0; k < kGroups && rc == 0; k++) {
		rc = f->groups[k].alloc();
	}
	if (rc != 0) {
		(void)ofi_amd_netfab_destroy(f);
		return rc;
	}
	*out = f;
	return 0;
}

int ofi_amd_netfab_destroy(ofi_amd_netfab_t *f)
{
	if (!f) {
		return -EINVAL;
	}
	/* launches in flight read the pinned tables and write the rx pool */
	const int rc = f->rx_pool ? ofi_amd_gpu_stream_synchronize(f->stream) : 0;
	for (group_t &g : f->groups) {
		g.release();
	}
	if (f->rx_pool) (void)ofi_amd_gpu_mem_free(f->rx_pool);
	if (f->d_flush_buf) (void)ofi_amd_gpu_mem_free(f->d_flush_buf);
	delete f;
	return rc;
}

int ofi_amd_netfab_ops(ofi_amd_netfab_t *f, ofi_amd_net_fabric_ops_t *send_end, ofi_amd_net_fabric_ops_t *recv_end)
{
	if (!f || !send_end || !recv_end) {
		return -EINVAL;
	}
	send_end->post = recv_end->post = &ofi_amd_netfab::post_cb;
	send_end->cq_read = recv_end->cq_read = &ofi_amd_netfab::cq_read_cb;
	send_end->repost_rx = recv_end->repost_rx = &ofi_amd_netfab::repost_rx_cb;
	send_end->end = &f->send_end;
	recv_end->end = &f->recv_end;
	return 0;
}

const void *ofi_amd_netfab_rx_pool(const ofi_amd_netfab_t *f)
{
	return f ? f->rx_pool : nullptr;
}

int ofi_amd_netfab_connect(ofi_amd_netfab_t *f, void *send_comm_mailbox)
{
	if (!f || !send_comm_mailbox) {
		return -EINVAL;
	}
	f->mailbox = static_cast<uint8_t *>(send_comm_mailbox);
	return 0;
}

int ofi_amd_netfab_counts(const ofi_amd_netfab_t *f, uint64_t *launches, uint64_t *copy_entries)
{
	if (!f || !launches || !copy_entries) {
		return -EINVAL;
	}
	*launches = f->n_launches;
	*copy_entries = f->n_entries;
	return 0;
}

} /* extern "C" */

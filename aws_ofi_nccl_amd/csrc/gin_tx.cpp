/*
 * The GIN initiator below the wire derivation: what nccl_ofi_rdma_gin_put_comm::iputSignal does
 * with the records it has derived (src/rdma/gin/nccl_ofi_gin.cpp:737-864), send_ack (:267-315),
 * the request pool (include/rdma/gin/nccl_ofi_gin_resources.h:318-348), the pending list
 * (:353-356) and nccl_ofi_gin_resources::progress -- a bounded drain of every rail's completion
 * queue, then a retry of the queued requests (src/rdma/gin/nccl_ofi_gin_resources.cpp:89-166,
 * 574-599).  The fabric is two callbacks; plain C++, no device needed.
 *
 * Also here: the in-process fabric of the loop-back runs (bounded send queue per rail,
 * doorbells, a completion queue per rail).
 */
#include <cerrno>
#include <cstring>
#include <deque>
#include <new>
#include <vector>

#include "host_util.hpp"
#include "ofi_amd_hotpath.h"

namespace {

constexpr int32_t kNoParent = -1;
constexpr uint32_t kMetaSlot = OFI_AMD_MAX_NUM_RAILS; /* reqs_pending[MAX_NUM_RAILS]: the metadata send */

enum : uint8_t { kFree = 0, kOperation = 1, kSub = 2, kFlush = 3 };

/* One pool entry: the umbrella request of an operation (nccl_ofi_rdma_gin_iputsignal_req) or
 * one post (write / metadata send / ACK send request). */
struct alignas(64) request_t { /* two cache lines to an entry, none shared with a neighbour */
	uint8_t use = kFree;
	uint8_t slot = 0;            /* sub: which reqs_pending flag of the parent it clears */
	int32_t parent = kNoParent;  /* sub: the operation, or kNoParent (ACKs, given-up operations) */
	uint32_t pending_mask = 0;   /* operation: bit per outstanding post */
	const volatile uint64_t *flush_slots = nullptr; /* flush: one 64-byte slot per rail in host memory */
	uint64_t sentinel = 0;       /* flush: what a slot holds once its read has landed */
	ofi_amd_gin_post_t post;     /* sub */
};

} // namespace

struct ofi_amd_gin_tx {
	uint32_t num_rails = 0, cq_read_count = 0, cq_max_iter = 0;
	ofi_amd_gin_fabric_ops_t ops = {};
	std::vector<request_t> pool;
	std::vector<uint32_t> free_list; /* used as a stack: the entry freed last is handed out first */
	std::deque<uint32_t> pending;    /* requests the fabric refused, oldest first */
	std::vector<uint32_t> cq_buf;
	ofi_amd_gin_tx_stats_t st = {};

	bool alloc(uint32_t *idx)
	{
		if (free_list.empty()) {
			return false;
		}
		*idx = free_list.back();
		free_list.pop_back();
		request_t &r = pool[*idx]; /* what a user does not set itself starts clean; `post` is always set whole */
		r.slot = 0;
		r.parent = kNoParent;
		r.pending_mask = 0;
		st.requests++;
		if (st.requests > st.requests_max) {
			st.requests_max = st.requests;
		}
		return true;
	}

	void release(uint32_t idx)
	{
		pool[idx].use = kFree; /* the rest is rewritten by whoever takes the entry next */
		free_list.push_back(idx);
		st.requests--;
	}

	/* One attempt.  The request's FI_MORE is dropped after it whatever the outcome: a retried
	 * post rings its own doorbell (nccl_net_ofi_gin_write_req_t::post,
	 * src/rdma/gin/nccl_ofi_gin_reqs.cpp:262-263; metadata send :310-311). */
	int post_once(uint32_t idx)
	{
		request_t &r = pool[idx];
		const int rc = ops.post(ops.fabric, &r.post);
		r.post.more = 0;
		if (rc == 0 && r.post.kind == OFI_AMD_GIN_POST_ACK) {
			st.outstanding_acks++; /* nccl_net_ofi_gin_sendack_req_t::post, :187-189 */
		}
		return rc;
	}

	void queue_pending(uint32_t idx)
	{
		pending.push_back(idx); /* add_pending_req */
		st.refused++;
		st.pending = (uint32_t)pending.size();
		if (st.pending > st.pending_max) {
			st.pending_max = st.pending;
		}
	}

	/* handle_cq_entry of the three request kinds (nccl_ofi_gin_reqs.cpp:164-172, 271-284,
	 * 319-331): clear the parent's flag, return the request to the pool */
	int complete(uint32_t ctx)
	{
		if (ctx >= pool.size() || pool[ctx].use != kSub) {
			return -EINVAL; /* "Invalid request context provided" */
		}
		request_t &r = pool[ctx];
		if (r.post.kind == OFI_AMD_GIN_POST_ACK) {
			st.outstanding_acks--;
		}
		if (r.parent != kNoParent) {
			pool[(uint32_t)r.parent].pending_mask &= ~(1u << r.slot);
		}
		release(ctx);
		st.completions++;
		return 0;
	}

	/* gin_process_cq_rail, nccl_ofi_gin_resources.cpp:89-150 */
	int process_cq_rail(uint32_t rail)
	{
		uint32_t iter = 0;
		do {
			++iter;
			const int rc = ops.cq_read(ops.fabric, rail, cq_buf.data(), cq_read_count);
			if (rc > 0) {
				for (int k = 0; k < rc; k++) {
					const int e = complete(cq_buf[(size_t)k]);
					if (e != 0) {
						return e;
					}
				}
			} else if (rc == 0 || rc == -EAGAIN) {
				break; /* no completions to process */
			} else {
				return rc;
			}
		} while (iter < cq_max_iter);
		return 0;
	}

	/* retry_pending_reqs, :584-599: in order, stop at the first request still refused */
	int retry_pending()
	{
		while (!pending.empty()) {
			const uint32_t idx = pending.front();
			st.retries++;
			const int rc = post_once(idx);
			if (rc == 0) {
				pending.pop_front();
				st.retried_ok++;
				st.pending = (uint32_t)pending.size();
			} else if (rc == -EAGAIN) {
				return 0;
			} else {
				return rc;
			}
		}
		return 0;
	}
};

extern "C" {

int ofi_amd_gin_tx_create(uint32_t num_rails, uint32_t cq_read_count, uint32_t cq_process_max_iter,
			  uint32_t max_requests, const ofi_amd_gin_fabric_ops_t *ops, ofi_amd_gin_tx_t **out)
{
	if (!out || !ops || !ops->post || !ops->cq_read || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS ||
	    cq_read_count == 0 || cq_read_count > 4096 || cq_process_max_iter == 0 || max_requests == 0 ||
	    max_requests > (1u << 24)) {
		return -EINVAL;
	}
	ofi_amd_gin_tx *tx = new (std::nothrow) ofi_amd_gin_tx;
	if (!tx) {
		return -ENOMEM;
	}
	try {
		tx->pool.resize(max_requests);
		tx->free_list.reserve(max_requests);
		for (uint32_t i = max_requests; i > 0; i--) {
			tx->free_list.push_back(i - 1); /* entry 0 is handed out first */
		}
		tx->cq_buf.resize(cq_read_count);
	} catch (...) {
		delete tx;
		return -ENOMEM;
	}
	tx->num_rails = num_rails;
	tx->cq_read_count = cq_read_count;
	tx->cq_max_iter = cq_process_max_iter;
	tx->ops = *ops;
	*out = tx;
	return 0;
}

int ofi_amd_gin_tx_destroy(ofi_amd_gin_tx_t *tx)
{
	if (!tx) {
		return -EINVAL;
	}
	delete tx;
	return 0;
}

/* The posts of one operation: its writes (or, for a get, its reads) in stripe order, then its
 * metadata message. */
static int post_operation(ofi_amd_gin_tx_t *tx, uint32_t peer, const ofi_amd_gin_wire_t *wire,
			  uint32_t transfer_kind, int32_t *request)
{
	*request = -1;
	const uint32_t need = 1 + wire->num_writes + (wire->has_meta ? 1u : 0u);
	if (tx->free_list.size() < need) {
		return -ENOMEM; /* get_req_from_pool throws; here nothing has been posted yet */
	}
	for (uint32_t k = 0; k < wire->num_writes; k++) {
		if (wire->writes[k].rail >= tx->num_rails) {
			return -EINVAL;
		}
	}
	if (wire->has_meta && wire->meta_rail >= tx->num_rails) {
		return -EINVAL;
	}

	uint32_t op = 0;
	(void)tx->alloc(&op);
	tx->pool[op].use = kOperation;
	uint32_t subs[OFI_AMD_MAX_NUM_RAILS + 1];
	uint32_t n_subs = 0;

	/* a post failed for good: the umbrella goes back to the pool and the posts already made
	 * lose their way back to it (clear_write_reqs_pending_back_pointers, :746-758;
	 * clear_read_reqs_pending_back_pointers, :869-877).  The failed request goes back too; the
	 * reference's iget leaves its failed read request out of the pool (:925-931), which is not
	 * repeated here. */
	auto give_up = [&](uint32_t failed) {
		for (uint32_t k = 0; k < n_subs; k++) {
			if (subs[k] != failed) {
				tx->pool[subs[k]].parent = kNoParent;
			}
		}
		tx->release(failed);
		tx->release(op);
	};

	for (uint32_t k = 0; k < wire->num_writes; k++) { /* :737-784, :901-932 */
		const ofi_amd_gin_write_t &w = wire->writes[k];
		uint32_t idx = 0;
		(void)tx->alloc(&idx);
		request_t &r = tx->pool[idx];
		r.use = kSub;
		r.slot = (uint8_t)k;
		r.parent = (int32_t)op;
		r.post = ofi_amd_gin_post_t{transfer_kind, w.rail, w.more, idx, peer, wire->imm,
					    w.src, w.len, w.dest, w.key, {0, 0, 0, 0}};
		tx->pool[op].pending_mask |= 1u << k;
		subs[n_subs++] = idx;
		const int rc = tx->post_once(idx);
		if (rc == -EAGAIN) {
			tx->queue_pending(idx); /* SQ full: queue for retry (FI_MORE dropped on retry) */
			continue;
		}
		if (rc != 0) {
			give_up(idx);
			return rc;
		}
		tx->st.posts++;
	}
	if (wire->has_meta) { /* :795-856 */
		uint32_t idx = 0;
		(void)tx->alloc(&idx);
		request_t &r = tx->pool[idx];
		r.use = kSub;
		r.slot = (uint8_t)kMetaSlot;
		r.parent = (int32_t)op;
		r.post = ofi_amd_gin_post_t{OFI_AMD_GIN_POST_META, wire->meta_rail, wire->meta_more, idx, peer, 0,
					    0, 32, 0, 0,
					    {wire->meta[0], wire->meta[1], wire->meta[2], wire->meta[3]}};
		tx->pool[op].pending_mask |= 1u << kMetaSlot;
		subs[n_subs++] = idx;
		const int rc = tx->post_once(idx);
		if (rc == -EAGAIN) {
			tx->queue_pending(idx);
		} else if (rc != 0) {
			give_up(idx);
			return rc;
		} else {
			tx->st.posts++;
		}
	}
	*request = (int32_t)op;
	return 0;
}

int ofi_amd_gin_tx_iput_signal(ofi_amd_gin_tx_t *tx, uint32_t peer, const ofi_amd_gin_wire_t *wire,
			       int32_t *request)
{
	if (!tx || !wire || !request || wire->num_writes > OFI_AMD_MAX_NUM_RAILS) {
		return -EINVAL;
	}
	return post_operation(tx, peer, wire, OFI_AMD_GIN_POST_WRITE, request);
}

int ofi_amd_gin_tx_iget(ofi_amd_gin_tx_t *tx, uint32_t peer, const ofi_amd_gin_wire_t *wire,
			int32_t *request)
{
	/* a get's record: reads only, nothing for the target (ofi_amd_gin_iget) */
	if (!tx || !wire || !request || wire->num_writes < 1 || wire->num_writes > OFI_AMD_MAX_NUM_RAILS ||
	    wire->has_meta || wire->nseg != 0 || wire->imm != 0) {
		return -EINVAL;
	}
	return post_operation(tx, peer, wire, OFI_AMD_GIN_POST_READ, request);
}

/* nccl_ofi_rdma_gin_put_comm::iflush, src/rdma/gin/nccl_ofi_gin.cpp:941-1003: clear the host
 * slots, take the umbrella request, post one 64-byte read per rail from the device flush buffer
 * into the rail's slot.  The reads carry no way back to the umbrella ("No pending_flag --
 * completion detected via sentinel polling"); their own completions only return them to the pool. */
int ofi_amd_gin_tx_iflush(ofi_amd_gin_tx_t *tx, void *host_slots, uint64_t device_flush_buffer,
			  uint64_t sentinel, int32_t *request)
{
	if (!tx || !host_slots || !request || (reinterpret_cast<uintptr_t>(host_slots) & 7u) != 0) {
		return -EINVAL;
	}
	*request = -1;
	if (tx->free_list.size() < 1 + tx->num_rails) {
		return -ENOMEM;
	}
	volatile uint64_t *slots = static_cast<volatile uint64_t *>(host_slots);
	for (uint32_t rail = 0; rail < tx->num_rails; rail++) {
		slots[rail * 8] = 0; /* :957-962 */
	}
	uint32_t op = 0;
	(void)tx->alloc(&op);
	tx->pool[op].use = kFlush;
	tx->pool[op].flush_slots = slots;
	tx->pool[op].sentinel = sentinel;
	for (uint32_t rail = 0; rail < tx->num_rails; rail++) { /* :967-996 */
		uint32_t idx = 0;
		(void)tx->alloc(&idx);
		request_t &r = tx->pool[idx];
		r.use = kSub;
		r.parent = kNoParent;
		r.post = ofi_amd_gin_post_t{OFI_AMD_GIN_POST_READ, rail, 0, idx, OFI_AMD_GIN_PEER_SELF, 0,
					    reinterpret_cast<uintptr_t>(host_slots) + 64u * rail, 64, device_flush_buffer,
					    0, {0, 0, 0, 0}};
		const int rc = tx->post_once(idx);
		if (rc == -EAGAIN) {
			tx->queue_pending(idx);
		} else if (rc != 0) {
			/* the umbrella goes back (:990-993); the reads already posted complete on their own */
			tx->release(idx);
			tx->release(op);
			return rc;
		} else {
			tx->st.posts++;
		}
	}
	*request = (int32_t)op;
	return 0;
}

int ofi_amd_gin_tx_send_ack(ofi_amd_gin_tx_t *tx, uint32_t peer, uint64_t ack_msg)
{
	if (!tx) {
		return -EINVAL;
	}
	uint32_t idx = 0;
	if (!tx->alloc(&idx)) {
		return -ENOMEM;
	}
	request_t &r = tx->pool[idx];
	r.use = kSub;
	r.parent = kNoParent;
	/* "For now, always send acks on rail 0" (:270-272) */
	r.post = ofi_amd_gin_post_t{OFI_AMD_GIN_POST_ACK, 0, 0, idx, peer, 0, 0, 8, 0, 0, {ack_msg, 0, 0, 0}};
	const int rc = tx->post_once(idx);
	if (rc == -EAGAIN) {
		tx->queue_pending(idx);
		return 0;
	}
	if (rc != 0) {
		tx->release(idx);
		return rc;
	}
	tx->st.posts++;
	return 0;
}

int ofi_amd_gin_tx_progress(ofi_amd_gin_tx_t *tx)
{
	if (!tx) {
		return -EINVAL;
	}
	for (uint32_t rail = 0; rail < tx->num_rails; rail++) { /* process_cq, :152-166 */
		const int rc = tx->process_cq_rail(rail);
		if (rc != 0) {
			return rc;
		}
	}
	return tx->retry_pending();
}

int ofi_amd_gin_tx_test(ofi_amd_gin_tx_t *tx, int32_t request, int *done)
{
	if (!tx || !done || request < 0 || (size_t)request >= tx->pool.size() ||
	    (tx->pool[(uint32_t)request].use != kOperation && tx->pool[(uint32_t)request].use != kFlush)) {
		return -EINVAL;
	}
	*done = 0;
	if (tx->pool[(uint32_t)request].use == kFlush) {
		/* nccl_ofi_gin_iflush_req::test, src/rdma/gin/nccl_ofi_gin_reqs.cpp:373-394: the sentinel in
		 * every rail's slot, not the completion queue, says that the reads have landed */
		const request_t &f = tx->pool[(uint32_t)request];
		for (uint32_t rail = 0; rail < tx->num_rails; rail++) {
			if (__atomic_load_n(const_cast<const uint64_t *>(&f.flush_slots[rail * 8]), __ATOMIC_ACQUIRE) !=
			    f.sentinel) {
				return 0;
			}
		}
		*done = 1;
		tx->release((uint32_t)request);
		return 0;
	}
	if (tx->pool[(uint32_t)request].pending_mask == 0) {
		*done = 1;
		tx->release((uint32_t)request);
	}
	return 0;
}

int ofi_amd_gin_tx_stats(const ofi_amd_gin_tx_t *tx, ofi_amd_gin_tx_stats_t *out)
{
	if (!tx || !out) {
		return -EINVAL;
	}
	*out = tx->st;
	return 0;
}

} /* extern "C" */

/* ---------------------------------------------------------------- the in-process fabric ---- */

using ofi_amd::ring_t;

struct ofi_amd_loopfab {
	struct rail_t {
		ring_t<ofi_amd_gin_post_t> sq; /* posted, completion not read yet: at most sq_depth */
		uint32_t transmitted = 0;      /* of which the doorbell has rung for */
		uint32_t taken = 0;            /* of which handed to the wire */
		uint32_t readable = 0;         /* of which the completion can be read */
	};
	uint32_t num_rails = 0, sq_depth = 0;
	std::vector<rail_t> rails;
	ring_t<uint8_t> rung; /* rails in the order their doorbells rang, one entry per transmitted post:
			       * at most num_rails * sq_depth */

	static int post(void *self, const ofi_amd_gin_post_t *p)
	{
		ofi_amd_loopfab *f = static_cast<ofi_amd_loopfab *>(self);
		if (!p || p->rail >= f->num_rails) {
			return -EINVAL;
		}
		rail_t &r = f->rails[p->rail];
		if (r.sq.size() >= f->sq_depth) {
			return -EAGAIN;
		}
		r.sq.push(*p);
		/* a provider never leaves a full queue unsubmitted */
		if (!p->more || r.sq.size() >= f->sq_depth) {
			while (r.transmitted < r.sq.size()) {
				f->rung.push((uint8_t)p->rail);
				r.transmitted++;
			}
		}
		return 0;
	}

	static int cq_read(void *self, uint32_t rail, uint32_t *contexts, uint32_t max)
	{
		ofi_amd_loopfab *f = static_cast<ofi_amd_loopfab *>(self);
		if (rail >= f->num_rails || !contexts) {
			return -EINVAL;
		}
		rail_t &r = f->rails[rail];
		uint32_t n = 0;
		while (n < max && r.readable > 0) {
			contexts[n++] = r.sq.at(0).context;
			r.sq.pop(); /* the send-queue entry is free again */
			r.readable--;
			r.taken--;
			r.transmitted--;
		}
		return (int)n;
	}
};

extern "C" {

int ofi_amd_loopfab_create(uint32_t num_rails, uint32_t sq_depth, ofi_amd_loopfab_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS || sq_depth == 0) {
		return -EINVAL;
	}
	ofi_amd_loopfab *f = new (std::nothrow) ofi_amd_loopfab;
	if (!f) {
		return -ENOMEM;
	}
	if (sq_depth > (1u << 20)) {
		delete f;
		return -EINVAL;
	}
	try {
		f->rails.resize(num_rails);
		for (auto &r : f->rails) {
			r.sq.reset(sq_depth);
		}
		f->rung.reset(num_rails * sq_depth);
	} catch (...) {
		delete f;
		return -ENOMEM;
	}
	f->num_rails = num_rails;
	f->sq_depth = sq_depth;
	*out = f;
	return 0;
}

int ofi_amd_loopfab_destroy(ofi_amd_loopfab_t *f)
{
	if (!f) {
		return -EINVAL;
	}
	delete f;
	return 0;
}

int ofi_amd_loopfab_ops(ofi_amd_loopfab_t *f, ofi_amd_gin_fabric_ops_t *ops)
{
	if (!f || !ops) {
		return -EINVAL;
	}
	ops->post = &ofi_amd_loopfab::post;
	ops->cq_read = &ofi_amd_loopfab::cq_read;
	ops->fabric = f;
	return 0;
}

int ofi_amd_loopfab_ring_all(ofi_amd_loopfab_t *f)
{
	if (!f) {
		return -EINVAL;
	}
	for (uint32_t rail = 0; rail < f->num_rails; rail++) {
		ofi_amd_loopfab::rail_t &r = f->rails[rail];
		while (r.transmitted < r.sq.size()) {
			f->rung.push((uint8_t)rail);
			r.transmitted++;
		}
	}
	return 0;
}

uint32_t ofi_amd_loopfab_take_transmitted(ofi_amd_loopfab_t *f, ofi_amd_gin_post_t *out, uint32_t cap)
{
	if (!f || !out) {
		return 0;
	}
	uint32_t n = 0;
	while (n < cap && !f->rung.empty()) {
		ofi_amd_loopfab::rail_t &r = f->rails[f->rung.at(0)];
		f->rung.pop();
		out[n++] = r.sq.at(r.taken);
		r.taken++;
		r.readable++; /* executed on the spot by the caller: the completion is there */
	}
	return n;
}

const ofi_amd_gin_post_t *ofi_amd_loopfab_next_transmitted(ofi_amd_loopfab_t *f)
{
	if (!f || f->rung.empty()) {
		return nullptr;
	}
	ofi_amd_loopfab::rail_t &r = f->rails[f->rung.at(0)];
	f->rung.pop();
	const ofi_amd_gin_post_t *p = &r.sq.at(r.taken);
	r.taken++;
	r.readable++;
	return p;
}

} /* extern "C" */

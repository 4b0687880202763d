/*
 * TEST INFRASTRUCTURE (CPU oracle).  Restates, below the point where iputSignal has derived its
 * wire record, what the reference does with it:
 *   - the post loop of nccl_ofi_rdma_gin_put_comm::iputSignal, src/rdma/gin/nccl_ofi_gin.cpp:
 *     737-784 (one write request per stripe, -FI_EAGAIN -> add_pending_req and carry on),
 *     795-856 (the metadata send, same rule), send_ack :267-315 (rail 0, same rule);
 *   - the request pool, include/rdma/gin/nccl_ofi_gin_resources.h:318-348 (one freelist for
 *     every request type; the entry freed last is allocated next) and add_pending_req :353-356;
 *   - nccl_ofi_gin_resources::progress and retry_pending_reqs,
 *     src/rdma/gin/nccl_ofi_gin_resources.cpp:574-599, with gin_process_cq_rail :89-150 and
 *     process_cq :152-166;
 *   - the completion handlers and test() of src/rdma/gin/nccl_ofi_gin_reqs.cpp:164-172,
 *     196-238, 241-331 (FI_MORE is dropped after the first post attempt, :262-263, :310-311).
 * libfabric is two callbacks here, as in the product, so that a test can hold both to one
 * scripted fabric.
 *
 * Pinned by: post / retry / completion orders worked out by hand for scripted fabrics
 * (tests/test_gin_tx.py).  The reference has no test of this path and it does not build here.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

enum { REQ_FREE = 0, REQ_OP = 1, REQ_POST = 2, REQ_FLUSH = 3 };

typedef struct {
	int use;
	int parent;          /* REQ_POST: index of its REQ_OP, or -1 */
	int flag;            /* REQ_POST: which reqs_pending[] flag of the parent it owns */
	int reqs_pending[ORACLE_MAX_RAILS + 1]; /* REQ_OP: nccl_ofi_rdma_gin_iputsignal_req */
	const volatile uint64_t *host_buff;     /* REQ_FLUSH: nccl_ofi_gin_iflush_req */
	uint64_t sentinel;
	oracle_gin_post_t post;
} oreq_t;

struct oracle_gin_tx {
	uint32_t num_rails, cq_read_count, cq_process_max_iter, max_requests;
	oracle_gin_fabric_ops_t ops;
	oreq_t *reqs;
	uint32_t *freelist; /* stack */
	uint32_t n_free;
	uint32_t *pending;  /* FIFO as a ring of max_requests entries */
	uint32_t pend_head, pend_count;
	oracle_gin_tx_stats_t st;
};

oracle_gin_tx_t *oracle_gin_tx_create(uint32_t num_rails, uint32_t cq_read_count,
				      uint32_t cq_process_max_iter, uint32_t max_requests,
				      const oracle_gin_fabric_ops_t *ops)
{
	oracle_gin_tx_t *tx = (oracle_gin_tx_t *)calloc(1, sizeof(*tx));
	if (!tx) {
		return NULL;
	}
	tx->num_rails = num_rails;
	tx->cq_read_count = cq_read_count;
	tx->cq_process_max_iter = cq_process_max_iter;
	tx->max_requests = max_requests;
	tx->ops = *ops;
	tx->reqs = (oreq_t *)calloc(max_requests, sizeof(oreq_t));
	tx->freelist = (uint32_t *)calloc(max_requests, sizeof(uint32_t));
	tx->pending = (uint32_t *)calloc(max_requests, sizeof(uint32_t));
	if (!tx->reqs || !tx->freelist || !tx->pending) {
		oracle_gin_tx_destroy(tx);
		return NULL;
	}
	for (uint32_t i = 0; i < max_requests; i++) {
		tx->freelist[i] = max_requests - 1 - i; /* top of the stack: entry 0 */
	}
	tx->n_free = max_requests;
	return tx;
}

void oracle_gin_tx_destroy(oracle_gin_tx_t *tx)
{
	if (tx) {
		free(tx->reqs);
		free(tx->freelist);
		free(tx->pending);
		free(tx);
	}
}

static int req_alloc(oracle_gin_tx_t *tx)
{
	if (tx->n_free == 0) {
		return -1;
	}
	uint32_t idx = tx->freelist[--tx->n_free];
	memset(&tx->reqs[idx], 0, sizeof(oreq_t));
	tx->st.requests++;
	if (tx->st.requests > tx->st.requests_max) {
		tx->st.requests_max = tx->st.requests;
	}
	return (int)idx;
}

static void req_free(oracle_gin_tx_t *tx, int idx)
{
	tx->reqs[idx].use = REQ_FREE;
	tx->freelist[tx->n_free++] = (uint32_t)idx;
	tx->st.requests--;
}

/* nccl_net_ofi_gin_write_req_t::post / metadata_send_req_t::post / sendack_req_t::post */
static int req_post(oracle_gin_tx_t *tx, int idx)
{
	oreq_t *r = &tx->reqs[idx];
	int rc = tx->ops.post(tx->ops.fabric, &r->post);
	r->post.more = 0; /* flags &= ~FI_MORE */
	if (rc == 0 && r->post.kind == ORACLE_GIN_POST_ACK) {
		tx->st.outstanding_acks++;
	}
	return rc;
}

static void add_pending_req(oracle_gin_tx_t *tx, int idx)
{
	tx->pending[(tx->pend_head + tx->pend_count) % tx->max_requests] = (uint32_t)idx;
	tx->pend_count++;
	tx->st.refused++;
	tx->st.pending = tx->pend_count;
	if (tx->st.pending > tx->st.pending_max) {
		tx->st.pending_max = tx->st.pending;
	}
}

int oracle_gin_tx_iput_signal(oracle_gin_tx_t *tx, uint32_t peer, const oracle_gin_wire_t *wire,
			      int32_t *request)
{
	*request = -1;
	uint32_t need = 1 + wire->num_writes + (wire->has_meta ? 1 : 0);
	if (tx->n_free < need) {
		return -12;
	}
	int op = req_alloc(tx);
	tx->reqs[op].use = REQ_OP;
	int posted[ORACLE_MAX_RAILS + 1];
	int n_posted = 0;

	for (uint32_t rail_it = 0; rail_it < wire->num_writes; rail_it++) {
		const oracle_gin_write_t *w = &wire->writes[rail_it];
		int wr = req_alloc(tx);
		oreq_t *r = &tx->reqs[wr];
		r->use = REQ_POST;
		r->parent = op;
		r->flag = (int)rail_it;
		r->post.kind = ORACLE_GIN_POST_WRITE;
		r->post.rail = w->rail;
		r->post.more = w->more;
		r->post.context = (uint32_t)wr;
		r->post.peer = peer;
		r->post.imm = wire->imm;
		r->post.src = w->src;
		r->post.len = w->len;
		r->post.dest = w->dest;
		r->post.key = w->key;
		tx->reqs[op].reqs_pending[rail_it] = 1;
		posted[n_posted++] = wr;
		int ret = req_post(tx, wr);
		if (ret != 0) {
			if (ret == -11) {
				add_pending_req(tx, wr);
				continue;
			}
			for (int k = 0; k < n_posted - 1; k++) {
				tx->reqs[posted[k]].parent = -1;
			}
			req_free(tx, wr);
			req_free(tx, op);
			return ret;
		}
		tx->st.posts++;
	}
	if (wire->has_meta) {
		int sr = req_alloc(tx);
		oreq_t *r = &tx->reqs[sr];
		r->use = REQ_POST;
		r->parent = op;
		r->flag = ORACLE_MAX_RAILS;
		r->post.kind = ORACLE_GIN_POST_META;
		r->post.rail = wire->meta_rail;
		r->post.more = wire->meta_more;
		r->post.context = (uint32_t)sr;
		r->post.peer = peer;
		r->post.len = 32;
		memcpy(r->post.msg, wire->meta, sizeof(r->post.msg));
		tx->reqs[op].reqs_pending[ORACLE_MAX_RAILS] = 1;
		int ret = req_post(tx, sr);
		if (ret == -11) {
			add_pending_req(tx, sr);
		} else if (ret != 0) {
			for (int k = 0; k < n_posted; k++) {
				tx->reqs[posted[k]].parent = -1;
			}
			req_free(tx, sr);
			req_free(tx, op);
			return ret;
		} else {
			tx->st.posts++;
		}
	}
	*request = op;
	return 0;
}

/* nccl_ofi_rdma_gin_put_comm::iget below its schedule, src/rdma/gin/nccl_ofi_gin.cpp:895-938:
 * an umbrella request, one read request per stripe with a back pointer to the umbrella's
 * flag (:918-920), -FI_EAGAIN -> add_pending_req (:923-924), any other failure gives the
 * operation up (:925-931).  The reference leaves the failed read request out of the pool on
 * that path; it is returned here, as the product does. */
int oracle_gin_tx_iget(oracle_gin_tx_t *tx, uint32_t peer, const oracle_gin_wire_t *wire,
		       int32_t *request)
{
	*request = -1;
	if (tx->n_free < 1 + wire->num_writes) {
		return -12;
	}
	int op = req_alloc(tx);
	tx->reqs[op].use = REQ_OP;
	int posted[ORACLE_MAX_RAILS];
	int n_posted = 0;
	for (uint32_t i = 0; i < wire->num_writes; i++) {
		const oracle_gin_write_t *w = &wire->writes[i];
		int rd = req_alloc(tx);
		oreq_t *r = &tx->reqs[rd];
		r->use = REQ_POST;
		r->parent = op;
		r->flag = (int)i;
		r->post.kind = ORACLE_GIN_POST_READ;
		r->post.rail = w->rail;
		r->post.more = 0;
		r->post.context = (uint32_t)rd;
		r->post.peer = peer;
		r->post.src = w->src;   /* local_buf */
		r->post.len = w->len;
		r->post.dest = w->dest; /* remote_offset */
		r->post.key = w->key;
		tx->reqs[op].reqs_pending[i] = 1;
		posted[n_posted++] = rd;
		int ret = req_post(tx, rd);
		if (ret == -11) {
			add_pending_req(tx, rd);
		} else if (ret != 0) {
			for (int k = 0; k < n_posted - 1; k++) {
				tx->reqs[posted[k]].parent = -1;
			}
			req_free(tx, rd);
			req_free(tx, op);
			return ret;
		} else {
			tx->st.posts++;
		}
	}
	*request = op;
	return 0;
}

/* nccl_ofi_rdma_gin_put_comm::iflush, src/rdma/gin/nccl_ofi_gin.cpp:941-1003 */
int oracle_gin_tx_iflush(oracle_gin_tx_t *tx, void *host_slots, uint64_t device_flush_buffer,
			 uint64_t sentinel, int32_t *request)
{
	*request = -1;
	if (tx->n_free < 1 + tx->num_rails) {
		return -12;
	}
	volatile uint64_t *host = (volatile uint64_t *)host_slots;
	for (uint32_t rail_id = 0; rail_id < tx->num_rails; rail_id++) { /* :957-962 */
		host[rail_id * 8] = 0;
	}
	int fr = req_alloc(tx); /* :964-965 */
	tx->reqs[fr].use = REQ_FLUSH;
	tx->reqs[fr].host_buff = host;
	tx->reqs[fr].sentinel = sentinel;
	for (uint32_t rail_id = 0; rail_id < tx->num_rails; rail_id++) { /* :967-996 */
		int rd = req_alloc(tx);
		oreq_t *r = &tx->reqs[rd];
		r->use = REQ_POST;
		r->parent = -1; /* pending_flag = nullptr */
		r->post.kind = ORACLE_GIN_POST_READ;
		r->post.rail = rail_id;
		r->post.context = (uint32_t)rd;
		r->post.peer = 0xffffffffu; /* own rank's address: loop-back */
		r->post.src = (uint64_t)(uintptr_t)host_slots + 64u * rail_id;
		r->post.len = 64;
		r->post.dest = device_flush_buffer;
		int ret = req_post(tx, rd);
		if (ret == -11) {
			add_pending_req(tx, rd);
		} else if (ret != 0) {
			req_free(tx, rd); /* the reference leaves it out of the pool; see oracle_gin_tx_iget */
			req_free(tx, fr);
			return ret;
		} else {
			tx->st.posts++;
		}
	}
	*request = fr;
	return 0;
}

int oracle_gin_tx_send_ack(oracle_gin_tx_t *tx, uint32_t peer, uint64_t ack_msg)
{
	int ar = req_alloc(tx);
	if (ar < 0) {
		return -12;
	}
	oreq_t *r = &tx->reqs[ar];
	r->use = REQ_POST;
	r->parent = -1;
	r->post.kind = ORACLE_GIN_POST_ACK;
	r->post.rail = 0;
	r->post.context = (uint32_t)ar;
	r->post.peer = peer;
	r->post.len = 8;
	r->post.msg[0] = ack_msg;
	int ret = req_post(tx, ar);
	if (ret == -11) {
		add_pending_req(tx, ar);
		return 0;
	}
	if (ret != 0) {
		req_free(tx, ar);
		return ret;
	}
	tx->st.posts++;
	return 0;
}

static int handle_cq_entry(oracle_gin_tx_t *tx, uint32_t ctx)
{
	if (ctx >= tx->max_requests || tx->reqs[ctx].use != REQ_POST) {
		return -22;
	}
	oreq_t *r = &tx->reqs[ctx];
	if (r->post.kind == ORACLE_GIN_POST_ACK) {
		tx->st.outstanding_acks--;
	}
	if (r->parent >= 0) {
		tx->reqs[r->parent].reqs_pending[r->flag] = 0; /* *pending_flag = false */
	}
	req_free(tx, (int)ctx);
	tx->st.completions++;
	return 0;
}

int oracle_gin_tx_progress(oracle_gin_tx_t *tx)
{
	uint32_t *cqe = (uint32_t *)calloc(tx->cq_read_count, sizeof(uint32_t));
	if (!cqe) {
		return -12;
	}
	int ret = 0;
	for (uint32_t rail_id = 0; rail_id < tx->num_rails && ret == 0; rail_id++) {
		uint32_t iter = 0;
		do {
			++iter;
			int rc = tx->ops.cq_read(tx->ops.fabric, rail_id, cqe, tx->cq_read_count);
			if (rc > 0) {
				for (int i = 0; i < rc && ret == 0; i++) {
					ret = handle_cq_entry(tx, cqe[i]);
				}
				if (ret != 0) {
					break;
				}
			} else if (rc == 0 || rc == -11) {
				break;
			} else {
				ret = rc;
				break;
			}
		} while (iter < tx->cq_process_max_iter);
	}
	free(cqe);
	if (ret != 0) {
		return ret;
	}
	/* retry_pending_reqs */
	while (tx->pend_count > 0) {
		int idx = (int)tx->pending[tx->pend_head];
		tx->st.retries++;
		ret = req_post(tx, idx);
		if (ret == 0) {
			tx->pend_head = (tx->pend_head + 1) % tx->max_requests;
			tx->pend_count--;
			tx->st.retried_ok++;
			tx->st.pending = tx->pend_count;
		} else if (ret == -11) {
			return 0;
		} else {
			return ret;
		}
	}
	return 0;
}

int oracle_gin_tx_test(oracle_gin_tx_t *tx, int32_t request, int *done)
{
	*done = 0;
	if (request < 0 || (uint32_t)request >= tx->max_requests ||
	    (tx->reqs[request].use != REQ_OP && tx->reqs[request].use != REQ_FLUSH)) {
		return -22;
	}
	if (tx->reqs[request].use == REQ_FLUSH) {
		/* nccl_ofi_gin_iflush_req::test, src/rdma/gin/nccl_ofi_gin_reqs.cpp:373-394 */
		for (uint32_t rail_id = 0; rail_id < tx->num_rails; rail_id++) {
			if (tx->reqs[request].host_buff[rail_id * 8] != tx->reqs[request].sentinel) {
				return 0;
			}
		}
		*done = 1;
		req_free(tx, request);
		return 0;
	}
	for (int i = 0; i <= ORACLE_MAX_RAILS; i++) {
		if (tx->reqs[request].reqs_pending[i]) {
			return 0;
		}
	}
	*done = 1;
	req_free(tx, request);
	return 0;
}

void oracle_gin_tx_stats(const oracle_gin_tx_t *tx, oracle_gin_tx_stats_t *out)
{
	*out = tx->st;
}

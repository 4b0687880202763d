/*
 * CPU oracle (test infrastructure): GIN put / put-signal.
 *
 * Wire encoders follow include/rdma/gin/nccl_ofi_gin_types.h:39-181; the
 * initiator state machine follows nccl_ofi_rdma_gin_put_comm::iputSignal,
 * src/rdma/gin/nccl_ofi_gin.cpp:518-566 (window, pin) and :568-864.
 */
#include <string.h>

#include "oracle.h"

/* include/rdma/gin/nccl_ofi_gin_types.h:55-79 */
#define IMM_TYPE_BITS 1
#define IMM_COMM_BITS 10
#define IMM_SEQ_BITS 13
#define IMM_COMM_SHIFT IMM_TYPE_BITS
#define IMM_SEQ_SHIFT (IMM_COMM_SHIFT + IMM_COMM_BITS)
#define IMM_SEQ_MASK ((1u << IMM_SEQ_BITS) - 1)
#define IMM_SEG_CNT_BITS 4
#define IMM_SEG_CNT_SHIFT (IMM_SEQ_SHIFT + IMM_SEQ_BITS)
#define IMM_ACK_REQ_SHIFT (IMM_SEG_CNT_SHIFT + IMM_SEG_CNT_BITS)
/* :90-92 */
#define RX_CONSUMED_BITS (IMM_SEQ_BITS + 1)
#define RX_CONSUMED_MASK ((1u << RX_CONSUMED_BITS) - 1)
/* :102, :107, :209 */
#define ACK_INTERVAL 64u
#define REQS_PER_DOORBELL 16u
#define ACK_REQ_THRESHOLD ((IMM_SEQ_MASK + 1) / 2)
/* nccl/net.h:28-29 */
#define SIGNAL_OP_INC 1u
#define SIGNAL_OP_ADD 2u
/* nccl/rma_v15.h:19-21 */
#define OPT_AGGREGATE 1u

/* GIN_IMM_SEG_DATA, :76-79; bit 0 stays 0 */
uint32_t oracle_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return (ack_req << IMM_ACK_REQ_SHIFT) | (nseg << IMM_SEG_CNT_SHIFT) |
	       (seq << IMM_SEQ_SHIFT) | (comm_id << IMM_COMM_SHIFT);
}

/* nccl_net_ofi_gin_msg_header_t, :128-145: little-endian bit-fields from the LSB:
 * msg_type:2 (=0 metadata), remote_comm_id:10, seq_num:13, seq_seg_cnt:4, ack_req:1 */
uint64_t oracle_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	uint64_t h = 0;
	h |= (uint64_t)(comm_id & 0x3ffu) << 2;
	h |= (uint64_t)(seq & 0x1fffu) << 12;
	h |= (uint64_t)(nseg & 0xfu) << 25;
	h |= (uint64_t)(ack_req & 1u) << 29;
	return h;
}

/* gin_ack_msg_t, :170-181: msg_type:2 (=1 ack), ack_comm_id:10, rx_consumed:14 */
uint64_t oracle_gin_ack_msg(uint32_t comm_id, uint32_t rx_consumed)
{
	uint64_t h = 1;
	h |= (uint64_t)(comm_id & 0x3ffu) << 2;
	h |= (uint64_t)(rx_consumed & RX_CONSUMED_MASK) << 12;
	return h;
}

/* ---- synthetic op stream (defined by this project, not by the reference) ---- */

static uint64_t mix64(uint64_t z)
{
	z ^= z >> 30;
	z *= 0xBF58476D1CE4E5B9ull;
	z ^= z >> 27;
	z *= 0x94D049BB133111EBull;
	z ^= z >> 31;
	return z;
}

static uint64_t rnd(uint64_t seed, uint32_t ctx, uint64_t i, uint32_t j)
{
	uint64_t ctr = ((((uint64_t)ctx << 40) + i) * 4u) + j + 1u;
	return mix64(seed + 0x9E3779B97F4A7C15ull * ctr);
}

void oracle_gin_gen_desc(uint64_t seed, uint32_t context, uint64_t i, uint32_t peer_rank,
			 uint32_t signal_every, uint32_t signal_op, uint32_t aggregate_mask,
			 oracle_gin_desc_t *out)
{
	const uint64_t span = (1ull << 30) - (1ull << 20);
	uint64_t r0 = rnd(seed, context, i, 0);
	uint64_t r1 = rnd(seed, context, i, 1);
	uint64_t r2 = rnd(seed, context, i, 2);
	uint32_t e = 3u + (uint32_t)((r0 & 0xffu) % 17u); /* octave 2^3 .. 2^19 */

	memset(out, 0, sizeof(*out));
	out->size = (1ull << e) | ((r0 >> 8) & ((1ull << e) - 1));
	out->src_off = ((r1 & 0xffffffffull) % span) & ~7ull;
	out->dst_off = ((r1 >> 32) % span) & ~7ull;
	out->rank = peer_rank;
	out->opt_flags = (uint32_t)(r2 & aggregate_mask);
	out->context = context;
	out->src_mr = 0;
	out->dst_mr = 1;
	if (signal_every != 0 && (i % signal_every) == signal_every - 1) {
		out->signal_op = signal_op;
		out->signal_off = 8ull * ((i / signal_every) % 512u);
		out->signal_value = (signal_op == SIGNAL_OP_ADD) ? (((r2 >> 8) & 0xffffu) + 1u) : 0;
		out->sig_mr = 2;
		out->kind = 2;
	} else {
		out->sig_mr = 0xffff;
		out->kind = 1;
	}
}

/* ---- initiator state machine ---- */

void oracle_gin_comm_init(oracle_gin_comm_t *c, uint32_t comm_id, uint32_t num_rails,
			  uint64_t min_stripe, uint64_t max_small, uint32_t ack_model)
{
	memset(c, 0, sizeof(*c));
	oracle_sched_init(&c->sched, (int)num_rails, min_stripe, max_small);
	c->comm_id = comm_id;
	c->num_rails = num_rails;
	c->pinned_rail_id = -1; /* no pin open */
	c->ack_model = ack_model;
}

/* gin_cursor_inc / gin_cursor_delta, include/rdma/gin/nccl_ofi_gin.h:155-163 */
static uint32_t cursor_inc(uint32_t c) { return (c + 1) & RX_CONSUMED_MASK; }
static uint32_t cursor_delta(uint32_t a, uint32_t b) { return (a - b) & RX_CONSUMED_MASK; }

int oracle_gin_iput_signal(oracle_gin_comm_t *c, const oracle_gin_mr_t *mrs,
			   const oracle_gin_desc_t *d, oracle_gin_wire_t *out)
{
	const int aggregate = (d->opt_flags & OPT_AGGREGATE) != 0; /* :576 */
	memset(out, 0, sizeof(*out));

	/* :580-584 */
	if (d->signal_op != 0 && d->signal_op != SIGNAL_OP_INC && d->signal_op != SIGNAL_OP_ADD) {
		return -22;
	}

	uint32_t seq = c->tx_head & IMM_SEQ_MASK; /* :588 */
	uint32_t rail_id;

	/* await_tx_window, :518-537: blocks while outstanding >= 8192.  Nothing
	 * can unblock it in this single-threaded model. */
	if (cursor_delta(c->tx_head, c->tx_tail) >= IMM_SEQ_MASK + 1) {
		return -11;
	}

	/* ack-request hysteresis, :607-620 */
	int has_signal = d->signal_op != 0;
	uint32_t ack_req = 0;
	uint32_t outstanding = cursor_delta(c->tx_head, c->tx_tail);
	if (outstanding >= ACK_REQ_THRESHOLD) {
		if (c->consecutive_puts_without_ack++ >= ACK_INTERVAL) {
			ack_req = 1;
			c->consecutive_puts_without_ack = 0;
		}
	}
	if (ack_req) { /* :624-627 */
		c->last_ack_requested_seq = c->tx_head;
		c->has_pending_ack_request = 1;
	}

	int defer = 0;
	uint32_t nseg = has_signal ? 1u : 0u; /* :653-658 */

	if (d->size > 0) {
		uint64_t src = mrs[d->src_mr].local_base + d->src_off;            /* :682 */
		const oracle_gin_mr_t *dst_mr = &mrs[d->dst_mr];
		uint64_t dest = dst_mr->remote_address_offset + d->dst_off;       /* :685 */
		oracle_xfer_t xfers[ORACLE_MAX_RAILS];
		uint32_t num_xfers =
			(uint32_t)oracle_sched_get_schedule(&c->sched, d->size, 128, xfers); /* :688-696 */

		if (num_xfers == 1 && c->pinned_rail_id >= 0) {                    /* :698-707 */
			xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
		} else if (num_xfers > 1 && c->pinned_rail_id >= 0) {            /* :708-726 */
			int touches = 0;
			for (uint32_t i = 0; i < num_xfers; i++) {
				if (xfers[i].rail_id == c->pinned_rail_id) {
					touches = 1;
					break;
				}
			}
			if (!touches) {
				xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
			}
		}
		defer = (num_xfers == 1) && aggregate &&
			(c->pinned_rail_run + 1 < REQS_PER_DOORBELL);             /* :727-728 */

		nseg += num_xfers;                                                 /* :730 */
		out->imm = oracle_gin_imm(c->comm_id, seq, nseg, ack_req);        /* :732 */
		rail_id = xfers[0].rail_id;                                        /* :735 */

		for (uint32_t k = 0; k < num_xfers; k++) {                        /* :737-784 */
			oracle_gin_write_t *w = &out->writes[k];
			w->rail = xfers[k].rail_id;
			w->src = src + xfers[k].offset;
			w->len = xfers[k].msg_size;
			w->dest = dest + xfers[k].offset;
			w->key = dst_mr->key[w->rail];
			w->more = ((has_signal && k == 0) || defer) ? 1u : 0u;     /* :747-749 */
		}
		out->num_writes = num_xfers;
	} else {
		/* signal only, :787-793; get_next_rail, nccl_ofi_gin_resources.h:363-368 */
		if (c->pinned_rail_id >= 0) {
			rail_id = (uint32_t)c->pinned_rail_id;
		} else {
			rail_id = c->next_rail_id;
			c->next_rail_id = (c->next_rail_id + 1) % c->num_rails;
		}
		defer = aggregate && (c->pinned_rail_run + 1 < REQS_PER_DOORBELL);
	}

	if (has_signal) { /* :795-856 */
		out->has_meta = 1;
		out->meta[0] = oracle_gin_meta_header(c->comm_id, seq, nseg, ack_req);
		out->meta[1] = (d->sig_mr != 0xffff) ? mrs[d->sig_mr].remote_address : 0; /* :815-816 */
		out->meta[2] = d->signal_off;
		if (d->signal_op == SIGNAL_OP_INC) {
			out->meta[3] = 1;
		} else if (d->signal_op == SIGNAL_OP_ADD) {
			out->meta[3] = d->signal_value;
		} else {
			out->meta[3] = 0;
		}
		out->meta_rail = rail_id;
		out->meta_more = defer ? 1u : 0u; /* :829-834 */
	}

	/* update_pin, :550-566 */
	if (defer) {
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

	/* Deterministic ACK model 1: the receiver's standalone ACK for this op
	 * carries rx_consumed == the new tx_head and is applied at once
	 * (apply_rx_consumed, include/rdma/gin/nccl_ofi_gin.h:535-543). */
	if (ack_req && c->ack_model == 1) {
		uint32_t delta = cursor_delta(c->tx_head, c->tx_tail);
		if (delta > 0 && delta <= (RX_CONSUMED_MASK + 1) / 2) {
			c->tx_tail = c->tx_head;
		}
		c->has_pending_ack_request = 0;
	}
	return 0;
}

/* nccl_ofi_rdma_gin_put_comm::iget, src/rdma/gin/nccl_ofi_gin.cpp:879-939, down to the
 * arguments of its reads.  Descriptor fields: src_off / src_mr = remoteOff / remoteMhandle,
 * dst_off / dst_mr = localOff / localMhandle. */
int oracle_gin_iget(oracle_gin_comm_t *c, const oracle_gin_mr_t *mrs, const oracle_gin_desc_t *d,
		    oracle_gin_wire_t *out)
{
	memset(out, 0, sizeof(*out));
	const oracle_gin_mr_t *remote_mr = &mrs[d->src_mr];
	const oracle_gin_mr_t *local_mr = &mrs[d->dst_mr];
	oracle_xfer_t xfers[ORACLE_MAX_RAILS];
	/* :899, the endpoint's scheduler: the one the puts use */
	uint32_t num_xfers = (uint32_t)oracle_sched_get_schedule(&c->sched, d->size, 128, xfers);
	for (uint32_t i = 0; i < num_xfers; i++) { /* :903-932 */
		oracle_gin_write_t *r = &out->writes[i];
		r->rail = xfers[i].rail_id;
		r->src = local_mr->local_base + d->dst_off + xfers[i].offset;               /* :905-906 */
		r->len = xfers[i].msg_size;
		r->dest = remote_mr->remote_address_offset + d->src_off + xfers[i].offset;  /* :908 */
		r->key = remote_mr->key[r->rail];                                            /* :915 */
		r->more = 0;
	}
	out->num_writes = num_xfers;
	return 0;
}

/* handle_ack_completion, src/rdma/gin/nccl_ofi_gin.cpp:1843-1869, with apply_rx_consumed,
 * include/rdma/gin/nccl_ofi_gin.h:535-543: a wire cursor moves the tail forward only, and
 * by at most half the cursor space; a pending ACK request is satisfied by any cursor at or
 * past the op that asked. */
void oracle_gin_apply_ack(oracle_gin_comm_t *c, uint32_t wire_rx_consumed)
{
	const uint32_t half = (RX_CONSUMED_MASK + 1) / 2;
	uint32_t rx = wire_rx_consumed & RX_CONSUMED_MASK;
	uint32_t delta = cursor_delta(rx, c->tx_tail);
	if (delta > 0 && delta <= half) {
		c->tx_tail = rx;
	}
	if (c->has_pending_ack_request && cursor_delta(rx, c->last_ack_requested_seq) <= half) {
		c->has_pending_ack_request = 0;
	}
}

/* ---- stream checksum (defined by this project): order-sensitive per context ---- */

static uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

uint64_t oracle_gin_fold(uint64_t h, const uint64_t *w, int n)
{
	static const uint64_t K[8] = {
		0x9E3779B97F4A7C15ull, 0xBF58476D1CE4E5B9ull, 0x94D049BB133111EBull, 0xD6E8FEB86659FD93ull,
		0xCA5A826395121157ull, 0x2545F4914F6CDD1Dull, 0xA0761D6478BD642Full, 0xE7037ED1A0B428DBull,
	};
	uint64_t x = 0;
	for (int k = 0; k < n; k++) {
		x += (w[k] + (uint64_t)(k + 1)) * K[k & 7];
	}
	return (rotl64(h, 5) ^ x) * 0x100000001B3ull;
}

/* Sum over contexts of the per-context hash of the seeded descriptor stream
 * (with_wire = 0) or of descriptors interleaved with the wire records iputSignal
 * derives from them (with_wire = 1; comm c uses comm_id c % 1024). */
uint64_t oracle_gin_stream_checksum(uint64_t seed, uint32_t n_contexts, uint64_t ops,
				    uint32_t peer_rank, uint32_t signal_every, uint32_t signal_op,
				    uint32_t aggregate_mask, int with_wire, uint32_t num_rails,
				    uint64_t min_stripe, uint64_t max_small, uint32_t ack_model,
				    const oracle_gin_mr_t *mrs)
{
	uint64_t total = 0;
	for (uint32_t c = 0; c < n_contexts; c++) {
		uint64_t h = 0x9E3779B97F4A7C15ull ^ c;
		oracle_gin_comm_t comm;
		oracle_gin_comm_init(&comm, c % 1024u, num_rails, min_stripe, max_small, ack_model);
		for (uint64_t i = 0; i < ops; i++) {
			oracle_gin_desc_t d;
			oracle_gin_gen_desc(seed, c, i, peer_rank, signal_every, signal_op,
					    aggregate_mask, &d);
			h = oracle_gin_fold(h, (const uint64_t *)&d, 8);
			if (with_wire) {
				oracle_gin_wire_t w;
				if (oracle_gin_iput_signal(&comm, mrs, &d, &w) != 0) {
					return 0;
				}
				h = oracle_gin_fold(h, (const uint64_t *)&w, (int)(sizeof(w) / 8));
			}
		}
		total += h;
	}
	return total;
}

/* ---- CPU producers through the reference's ring protocol ----
 * `producers` threads generate the seeded descriptors of their contexts and push them
 * through one MPSC ring per context (push with CAS, include/nccl_ofi_mpsc_ring.h:79-118);
 * the calling thread is the single consumer of every ring, as the GIN progress loop is
 * (src/rdma/gin/nccl_ofi_gin.cpp:1560-1574), and folds what it pops.  The result equals
 * oracle_gin_stream_checksum(with_wire = 0) of the same stream.  Returns 0 or -errno;
 * *seconds covers thread start to the last pop. */
#include <pthread.h>
#include <stdlib.h>
#include <time.h>

struct cpu_ring_producer {
	oracle_mpsc_t **rings;
	uint64_t seed, ops;
	uint32_t first, last; /* contexts [first, last) */
	uint32_t peer_rank, signal_every, signal_op, aggregate_mask;
};

static void *cpu_ring_producer_main(void *p)
{
	struct cpu_ring_producer *a = (struct cpu_ring_producer *)p;
	uint32_t n = a->last - a->first;
	uint64_t *next = (uint64_t *)calloc(n ? n : 1, sizeof(uint64_t));
	uint32_t open = n;
	if (!next) {
		return (void *)1;
	}
	while (open > 0) {
		open = 0;
		for (uint32_t k = 0; k < n; k++) {
			/* a burst per visit: stay on a ring while it takes entries */
			for (int burst = 0; burst < 64 && next[k] < a->ops; burst++) {
				oracle_gin_desc_t d;
				oracle_gin_gen_desc(a->seed, a->first + k, next[k], a->peer_rank,
						    a->signal_every, a->signal_op, a->aggregate_mask, &d);
				if (!oracle_mpsc_push(a->rings[a->first + k], &d)) {
					break;
				}
				next[k]++;
			}
			open += next[k] < a->ops;
		}
	}
	free(next);
	return NULL;
}

int oracle_gin_cpu_rings_run(uint64_t seed, uint32_t n_contexts, uint64_t ops, uint32_t capacity,
			     uint32_t producers, uint32_t peer_rank, uint32_t signal_every,
			     uint32_t signal_op, uint32_t aggregate_mask, uint64_t *checksum,
			     double *seconds)
{
	if (n_contexts == 0 || producers == 0 || producers > 64 || producers > n_contexts || !checksum ||
	    !seconds) {
		return -22;
	}
	oracle_mpsc_t **rings = (oracle_mpsc_t **)calloc(n_contexts, sizeof(*rings));
	uint64_t *hash = (uint64_t *)calloc(n_contexts, sizeof(uint64_t));
	uint64_t *popped = (uint64_t *)calloc(n_contexts, sizeof(uint64_t));
	struct cpu_ring_producer args[64];
	pthread_t th[64];
	int rc = 0;
	if (!rings || !hash || !popped) {
		rc = -12;
	}
	for (uint32_t c = 0; rc == 0 && c < n_contexts; c++) {
		rings[c] = oracle_mpsc_create(capacity, sizeof(oracle_gin_desc_t));
		hash[c] = 0x9E3779B97F4A7C15ull ^ c;
		if (!rings[c]) {
			rc = -12;
		}
	}
	if (rc == 0) {
		struct timespec t0, t1;
		clock_gettime(CLOCK_MONOTONIC, &t0);
		for (uint32_t p = 0; p < producers; p++) {
			args[p] = (struct cpu_ring_producer){ rings, seed, ops,
				(uint32_t)((uint64_t)n_contexts * p / producers),
				(uint32_t)((uint64_t)n_contexts * (p + 1) / producers),
				peer_rank, signal_every, signal_op, aggregate_mask };
			pthread_create(&th[p], NULL, cpu_ring_producer_main, &args[p]);
		}
		uint64_t left = (uint64_t)n_contexts * ops;
		while (left > 0) {
			for (uint32_t c = 0; c < n_contexts; c++) {
				oracle_gin_desc_t d;
				while (popped[c] < ops && oracle_mpsc_pop(rings[c], &d)) {
					hash[c] = oracle_gin_fold(hash[c], (const uint64_t *)&d, 8);
					popped[c]++;
					left--;
				}
			}
		}
		clock_gettime(CLOCK_MONOTONIC, &t1);
		for (uint32_t p = 0; p < producers; p++) {
			void *ret = NULL;
			pthread_join(th[p], &ret);
			if (ret) {
				rc = -12;
			}
		}
		*seconds = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
		uint64_t total = 0;
		for (uint32_t c = 0; c < n_contexts; c++) {
			total += hash[c];
		}
		*checksum = total;
	}
	for (uint32_t c = 0; rings && c < n_contexts; c++) {
		if (rings[c]) {
			oracle_mpsc_destroy(rings[c]);
		}
	}
	free(rings);
	free(hash);
	free(popped);
	return rc;
}

/*
 * CPU oracle (test infrastructure): GIN receiver side.
 *
 * Completion handlers and in-order retire with same-slot folding follow
 * src/rdma/gin/nccl_ofi_gin.cpp:1016-1019 (map key), :1622-1790 (retire),
 * :1792-1838 (metadata completion), :1871-1924 (write completion), :267-315 and
 * :1608-1620 (standalone ACK).  The worker's batch fold + read-modify-write follows
 * :1193-1256 and :1425-1479.
 *
 * One modelling choice: the reference hands each folded run to an asynchronous worker
 * and stops retiring until that worker reports back, so how long a run grows depends
 * on thread timing.  Here the hand-off completes at once (the reference's own
 * closing-path behaviour, :1298-1304), which makes the emitted work items a pure
 * function of the order in which completions arrive.
 *
 * Parity: the reference has no unit test for this path (tests/functional/rma.cpp checks
 * end values only: 64 put-signals must leave the counter at 64) and its source does not
 * build here -- PARITY UNPINNED beyond that end-value property and the invariants the
 * tests state.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define SEQ_BITS 13
#define SEQ_MASK ((1u << SEQ_BITS) - 1)
#define CURSOR_MASK ((1u << (SEQ_BITS + 1)) - 1)

typedef struct {
	uint8_t present;
	uint8_t metadata_received;
	uint8_t is_ack_requested;
	uint8_t pad;
	uint32_t num_seg_completions;
	uint32_t total_segments;
	uint32_t meta_seq;
	uint64_t base, offset, value;
} rx_req_t;

typedef struct {
	uint32_t comm_id; /* the peer's comm id, goes into ACKs */
	uint32_t rx_consumed;
	uint32_t next_delivered_seq;
	rx_req_t *reqs; /* one slot per sequence number: the (peer << 16 | seq) map */
} rx_peer_t;

struct oracle_gin_rx {
	uint32_t n_peers;
	rx_peer_t *peers;
	oracle_gin_signal_work_t *work;
	uint32_t n_work, cap_work;
	oracle_gin_ack_t *acks;
	uint32_t n_acks, cap_acks;
};

oracle_gin_rx_t *oracle_gin_rx_create(uint32_t n_peers, const uint32_t *peer_comm_ids)
{
	oracle_gin_rx_t *rx = (oracle_gin_rx_t *)calloc(1, sizeof(*rx));
	if (!rx) {
		return NULL;
	}
	rx->n_peers = n_peers;
	rx->peers = (rx_peer_t *)calloc(n_peers, sizeof(rx_peer_t));
	for (uint32_t p = 0; p < n_peers; p++) {
		rx->peers[p].comm_id = peer_comm_ids ? peer_comm_ids[p] : p;
		rx->peers[p].reqs = (rx_req_t *)calloc(SEQ_MASK + 1, sizeof(rx_req_t));
	}
	return rx;
}

void oracle_gin_rx_destroy(oracle_gin_rx_t *rx)
{
	if (!rx) {
		return;
	}
	for (uint32_t p = 0; p < rx->n_peers; p++) {
		free(rx->peers[p].reqs);
	}
	free(rx->peers);
	free(rx->work);
	free(rx->acks);
	free(rx);
}

static void emit_work(oracle_gin_rx_t *rx, const oracle_gin_signal_work_t *w)
{
	if (rx->n_work == rx->cap_work) {
		rx->cap_work = rx->cap_work ? rx->cap_work * 2 : 1024;
		rx->work = (oracle_gin_signal_work_t *)realloc(rx->work, rx->cap_work * sizeof(*w));
	}
	rx->work[rx->n_work++] = *w;
}

static void emit_ack(oracle_gin_rx_t *rx, uint32_t peer, uint32_t rx_consumed)
{
	if (rx->n_acks == rx->cap_acks) {
		rx->cap_acks = rx->cap_acks ? rx->cap_acks * 2 : 256;
		rx->acks = (oracle_gin_ack_t *)realloc(rx->acks, rx->cap_acks * sizeof(oracle_gin_ack_t));
	}
	oracle_gin_ack_t *a = &rx->acks[rx->n_acks++];
	a->peer = peer;
	a->rx_consumed = rx_consumed & CURSOR_MASK;
	a->msg = oracle_gin_ack_msg(rx->peers[peer].comm_id, rx_consumed); /* send_ack, :267-315 */
}

static int complete(const rx_req_t *r)
{
	return r->present && r->num_seg_completions == r->total_segments;
}

/* retire_completed_peer_iput_ops, :1622-1790, with a synchronous hand-off */
static void retire(oracle_gin_rx_t *rx, uint32_t peer)
{
	rx_peer_t *pc = &rx->peers[peer];
	int ack_requested = 0;

	for (;;) {
		uint32_t seq = pc->next_delivered_seq;
		rx_req_t *req = &pc->reqs[seq];
		if (!complete(req)) {
			break;
		}
		if (!req->metadata_received) { /* put without signal: nothing to deliver, :1679-1690 */
			ack_requested |= req->is_ack_requested;
			pc->rx_consumed = (pc->rx_consumed + 1) & CURSOR_MASK;
			pc->next_delivered_seq = (pc->next_delivered_seq + 1) & SEQ_MASK;
			memset(req, 0, sizeof(*req));
			continue;
		}
		oracle_gin_signal_work_t folded;
		memset(&folded, 0, sizeof(folded));
		folded.base = req->base;
		folded.offset = req->offset;
		folded.peer = peer;

		uint32_t cur_seq = seq;
		rx_req_t *cur = req;
		for (;;) { /* greedy run over consecutive ready same-slot signals, :1724-1763 */
			folded.value += cur->value;
			folded.run_len++;
			ack_requested |= cur->is_ack_requested;
			pc->rx_consumed = (pc->rx_consumed + 1) & CURSOR_MASK;
			pc->next_delivered_seq = (pc->next_delivered_seq + 1) & SEQ_MASK;

			uint32_t peek_seq = (cur_seq + 1) & SEQ_MASK;
			rx_req_t *peek = &pc->reqs[peek_seq];
			int extend = complete(peek) && peek->metadata_received &&
				     peek->base == folded.base && peek->offset == folded.offset;
			if (!extend) {
				break; /* cur is the gate */
			}
			memset(cur, 0, sizeof(*cur));
			cur_seq = peek_seq;
			cur = peek;
		}
		folded.gate_seq = (uint16_t)cur->meta_seq; /* hand_off_signal_work, :1295 */
		emit_work(rx, &folded);
		memset(cur, 0, sizeof(*cur));
	}
	if (ack_requested) { /* maybe_send_ack, :1608-1620 */
		emit_ack(rx, peer, pc->rx_consumed);
	}
}

/* handle_signal_write_completion, :1871-1924 */
int oracle_gin_rx_write(oracle_gin_rx_t *rx, uint32_t peer, uint32_t imm)
{
	if (peer >= rx->n_peers) {
		return -22;
	}
	uint32_t total = (imm >> 24) & 0xf;
	uint32_t seq = (imm >> 11) & SEQ_MASK;
	uint32_t ack = (imm >> 28) & 1;
	rx_req_t *req = &rx->peers[peer].reqs[seq];

	if (!req->present) {
		memset(req, 0, sizeof(*req));
		req->present = 1;
		req->num_seg_completions = 1;
		req->total_segments = total;
		req->is_ack_requested = (uint8_t)ack;
	} else {
		req->is_ack_requested |= (uint8_t)ack;
		req->num_seg_completions += 1;
	}
	if (req->num_seg_completions == req->total_segments) {
		req->meta_seq = seq; /* :1912-1914 */
		retire(rx, peer);
	}
	return 0;
}

/* handle_signal_metadata_completion, :1792-1838 */
int oracle_gin_rx_metadata(oracle_gin_rx_t *rx, uint32_t peer, const uint64_t meta[4])
{
	if (peer >= rx->n_peers) {
		return -22;
	}
	if ((meta[0] & 3u) != 0) {
		return -22; /* not a metadata message */
	}
	uint32_t seq = (uint32_t)(meta[0] >> 12) & SEQ_MASK;
	uint32_t total = (uint32_t)(meta[0] >> 25) & 0xf;
	uint32_t ack = (uint32_t)(meta[0] >> 29) & 1;
	rx_req_t *req = &rx->peers[peer].reqs[seq];

	if (!req->present) {
		memset(req, 0, sizeof(*req));
		req->present = 1;
		req->num_seg_completions = 1;
		req->total_segments = total;
		req->is_ack_requested = (uint8_t)ack;
	} else {
		req->num_seg_completions += 1;
		req->is_ack_requested |= (uint8_t)ack;
	}
	req->metadata_received = 1;
	req->meta_seq = seq;
	req->base = meta[1];
	req->offset = meta[2];
	req->value = meta[3];
	if (req->num_seg_completions == req->total_segments) {
		retire(rx, peer);
	}
	return 0;
}

uint32_t oracle_gin_rx_take_work(oracle_gin_rx_t *rx, oracle_gin_signal_work_t *out, uint32_t cap)
{
	uint32_t n = rx->n_work < cap ? rx->n_work : cap;
	if (n == 0) {
		return 0; /* the queue may not be allocated yet */
	}
	memcpy(out, rx->work, n * sizeof(*out));
	memmove(rx->work, rx->work + n, (rx->n_work - n) * sizeof(*out));
	rx->n_work -= n;
	return n;
}

uint32_t oracle_gin_rx_take_acks(oracle_gin_rx_t *rx, oracle_gin_ack_t *out, uint32_t cap)
{
	uint32_t n = rx->n_acks < cap ? rx->n_acks : cap;
	if (n == 0) {
		return 0;
	}
	memcpy(out, rx->acks, n * sizeof(*out));
	memmove(rx->acks, rx->acks + n, (rx->n_acks - n) * sizeof(*out));
	rx->n_acks -= n;
	return n;
}

void oracle_gin_rx_cursors(const oracle_gin_rx_t *rx, uint32_t peer, uint32_t *rx_consumed,
			   uint32_t *next_seq)
{
	*rx_consumed = rx->peers[peer].rx_consumed;
	*next_seq = rx->peers[peer].next_delivered_seq;
}

/* apply_and_complete + apply_signal_work, :1425-1479 and :1193-1256: entries of one batch
 * that hit the same (base, offset) fold into the first of them; each lead is applied with
 * one read-modify-write.  counters[r] is the 8-byte-counter array registered at bases[r];
 * consecutive regions that are contiguous in address are the segments of one window.
 * Returns the number of read-modify-writes, or -22 for an entry outside every region. */
int oracle_gin_signal_apply(const oracle_gin_signal_work_t *batch, uint32_t n, const uint64_t *bases,
			    const uint64_t *sizes, uint64_t *const *counters, uint32_t n_regions)
{
	uint32_t *lead = (uint32_t *)malloc(sizeof(uint32_t) * (n ? n : 1));
	uint64_t *sum = (uint64_t *)malloc(sizeof(uint64_t) * (n ? n : 1));
	int rmw = 0;

	for (uint32_t i = 0; i < n; i++) { /* pass 1: find the lead (first entry of the slot) */
		lead[i] = i;
		sum[i] = batch[i].value;
		for (uint32_t j = 0; j < i; j++) {
			if (lead[j] == j && batch[j].base == batch[i].base &&
			    batch[j].offset == batch[i].offset) {
				lead[i] = j;
				sum[j] += batch[i].value;
				break;
			}
		}
	}
	for (uint32_t i = 0; i < n; i++) { /* pass 2: one r-m-w per lead */
		if (lead[i] != i) {
			continue;
		}
		/* the window by its base address (the MR lookup, :1140-1152), the segment by the counter's
		 * address inside it (ensure_signal_seg, :1038-1122: a window may be backed by several
		 * allocations); regions listed one after the other, each beginning where the one before
		 * it ends, are the segments of one window */
		uint32_t r, seg = n_regions;
		uint64_t off = batch[i].offset;
		for (r = 0; r < n_regions; r++) {
			if (batch[i].base == bases[r]) {
				break;
			}
		}
		for (uint32_t k = r; k < n_regions; k++) {
			if (off <= sizes[k] && sizes[k] - off >= 8) {
				seg = k;
				break;
			}
			if (off < sizes[k] || k + 1 >= n_regions || bases[k + 1] != bases[k] + sizes[k]) {
				break;
			}
			off -= sizes[k];
		}
		if (seg == n_regions || (batch[i].offset & 7) != 0) {
			free(lead);
			free(sum);
			return -22;
		}
		counters[seg][off / 8] += sum[i];
		rmw++;
	}
	free(lead);
	free(sum);
	return rmw;
}

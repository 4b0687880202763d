/*
 * CPU oracle (test infrastructure): wire formats and ordering rules of the RDMA protocol
 * around the eager copy, restated from the reference.  Each function names the lines it
 * follows.  The reference header that defines these (include/nccl_ofi_rdma.h) needs
 * generated configuration and libfabric headers and does not build here; the restatement
 * is pinned by the known answers of tests/unit/ctrl_msg.cpp and the header's
 * static_asserts.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define SEQ_BITS 10
#define COMM_ID_BITS 15
#define RECV_IDX_BITS 3
#define NUM_SEG_BITS 4
#define MSG_SEQ_NUM_MASK ((1u << SEQ_BITS) - 1)
#define MAILBOX_SIZE 256u

/* GET_RDMA_WRITE_IMM_DATA, src/nccl_ofi_rdma.cpp:98-101 */
uint32_t oracle_rdma_imm(uint32_t comm_id, uint32_t seq, uint32_t recv_idx, uint32_t nseg)
{
	return seq | (comm_id << SEQ_BITS) | (recv_idx << (SEQ_BITS + COMM_ID_BITS)) |
	       (nseg << (SEQ_BITS + COMM_ID_BITS + RECV_IDX_BITS));
}

/* GET_*_FROM_IMM, :73-93 */
void oracle_rdma_imm_decode(uint32_t imm, uint32_t *comm_id, uint32_t *seq, uint32_t *recv_idx,
			    uint32_t *nseg)
{
	*comm_id = (imm >> SEQ_BITS) & ((1u << COMM_ID_BITS) - 1);
	*seq = imm & MSG_SEQ_NUM_MASK;
	*nseg = (imm >> (SEQ_BITS + COMM_ID_BITS + RECV_IDX_BITS)) & ((1u << NUM_SEG_BITS) - 1);
	*recv_idx = (imm >> (SEQ_BITS + COMM_ID_BITS)) & ((1u << RECV_IDX_BITS) - 1);
}

uint32_t oracle_ctrl_mailbox_slot(uint16_t msg_seq_num)
{
	return msg_seq_num % MAILBOX_SIZE; /* :3447 */
}

/* allocate_recv_req (called by recv): mailbox update, :3446-3474 */
int oracle_ctrl_msg_fill(oracle_ctrl_msg_t *mailbox, uint16_t msg_seq_num, uint16_t num_recvs,
			 const uint64_t *buff_offsets, const uint32_t *sizes, const int *tags,
			 const uint64_t *mr_keys, uint32_t num_rails, int recv_completion_optional)
{
	if (num_recvs < 1 || num_recvs > 8 || num_rails < 1 || num_rails > 4) {
		return -22;
	}
	oracle_ctrl_msg_t *slot = &mailbox[msg_seq_num % MAILBOX_SIZE];
	memset(slot, 0, sizeof(*slot));
	slot->entries[0].num_recvs = num_recvs;
	if (recv_completion_optional) {
		slot->entries[0].flags |= 1u;
	}
	for (uint16_t i = 0; i < num_recvs; i++) {
		oracle_ctrl_entry_t *e = &slot->entries[i];
		e->buff_offset = buff_offsets[i];
		e->buff_len = sizes[i];
		e->tag = (int16_t)tags[i];
		e->recv_idx = (uint8_t)i;
		e->entry_used = 0;
		e->msg_seq_num = msg_seq_num & MSG_SEQ_NUM_MASK;
		for (uint32_t r = 0; r < num_rails; r++) {
			e->mr_key[r] = mr_keys[i * num_rails + r];
		}
	}
	return 0;
}

/* has_ctrl_msg, :2134-2178 */
int oracle_ctrl_msg_ready(const oracle_ctrl_msg_t *mailbox, uint16_t seq_num, int tag,
			  int ignore_tag_match)
{
	const oracle_ctrl_msg_t *ctrl = &mailbox[seq_num % MAILBOX_SIZE];
	uint16_t expected = (uint16_t)(seq_num & MSG_SEQ_NUM_MASK);

	if (ctrl->entries[0].msg_seq_num != expected) {
		return 0;
	}
	uint16_t num_recvs = ctrl->entries[0].num_recvs;
	for (uint16_t i = 1; i < num_recvs; i++) {
		if (ctrl->entries[i].msg_seq_num != expected) {
			return 0;
		}
	}
	if (ignore_tag_match) {
		return 1;
	}
	for (uint16_t i = 0; i < num_recvs; i++) {
		if (ctrl->entries[i].entry_used == 1) {
			continue;
		}
		if (ctrl->entries[i].tag == tag) {
			return 1;
		}
	}
	return 0;
}

/* find_entry_by_tag as tests/unit/ctrl_msg.cpp:27-34 restates the search */
int oracle_ctrl_msg_find_tag(const oracle_ctrl_msg_t *msg, int tag)
{
	for (uint16_t i = 0; i < msg->entries[0].num_recvs; i++) {
		if (msg->entries[i].tag == tag) {
			return i;
		}
	}
	return -1;
}

/* include/nccl_ofi_rdma.h:670-673 */
int oracle_seq_before(uint16_t a, uint16_t b)
{
	uint16_t diff = (uint16_t)((a - b) & MSG_SEQ_NUM_MASK);
	return diff > (MSG_SEQ_NUM_MASK >> 1);
}

/* :678-681 */
int oracle_eager_seq_before(uint16_t a, uint16_t b)
{
	return (int16_t)(uint16_t)(a - b) < 0;
}

/* :683-689 */
int oracle_eager_entry_less(const oracle_eager_entry_t *a, const oracle_eager_entry_t *b)
{
	if (a->eager_seq != b->eager_seq) {
		return oracle_eager_seq_before(a->eager_seq, b->eager_seq);
	}
	return a->eager_offset < b->eager_offset;
}

/* :709-732 */
int oracle_eager_entry_can_process(int has_processed, uint16_t last_eager_seq, uint8_t last_offset,
				   const oracle_eager_entry_t *entry)
{
	if (!has_processed) {
		return (entry->eager_offset == 0) && (entry->eager_seq == 0);
	} else if (entry->eager_offset == 0) {
		return (entry->eager_seq == (uint16_t)(last_eager_seq + 1)) &&
		       (last_offset == entry->prev_batch_count - 1);
	} else {
		return (entry->eager_seq == last_eager_seq) && (last_offset == entry->eager_offset - 1);
	}
}

/* ---- receiver's ordered queue: a doubly linked list as in the reference ---- */

typedef struct node {
	struct node *prev, *next;
	oracle_eager_entry_t e;
} node_t;

struct oracle_eager_rxq {
	node_t head; /* sentinel */
	uint32_t count;
	int has_processed;
	uint16_t last_eager_seq;
	uint8_t last_offset;
};

oracle_eager_rxq_t *oracle_eager_rxq_create(void)
{
	oracle_eager_rxq_t *q = (oracle_eager_rxq_t *)calloc(1, sizeof(*q));
	if (q) {
		q->head.prev = q->head.next = &q->head;
	}
	return q;
}

void oracle_eager_rxq_destroy(oracle_eager_rxq_t *q)
{
	if (!q) {
		return;
	}
	node_t *n = q->head.next;
	while (n != &q->head) {
		node_t *nx = n->next;
		free(n);
		n = nx;
	}
	free(q);
}

/* recv_eager_sorted_insert, :734-750: walk from the back while the new entry is less */
int oracle_eager_rxq_insert(oracle_eager_rxq_t *q, const oracle_eager_entry_t *e)
{
	node_t *n = (node_t *)malloc(sizeof(*n));
	if (!n) {
		return -12;
	}
	n->e = *e;
	node_t *pos = q->head.prev;
	while (pos != &q->head) {
		if (!oracle_eager_entry_less(e, &pos->e)) {
			break;
		}
		pos = pos->prev;
	}
	n->prev = pos;
	n->next = pos->next;
	pos->next->prev = n;
	pos->next = n;
	q->count++;
	return 0;
}

/* the ordering half of drain_recv_eager_queue, src/nccl_ofi_rdma.cpp:797-816, 878-886:
 * entries leave from the front for as long as each is the next link of the chain */
uint32_t oracle_eager_rxq_drain(oracle_eager_rxq_t *q, oracle_eager_entry_t *out, uint32_t cap)
{
	uint32_t n = 0;
	while (n < cap && q->head.next != &q->head) {
		node_t *front = q->head.next;
		if (!oracle_eager_entry_can_process(q->has_processed, q->last_eager_seq, q->last_offset,
						    &front->e)) {
			break;
		}
		q->last_eager_seq = front->e.eager_seq;
		q->last_offset = front->e.eager_offset;
		q->has_processed = 1;
		out[n++] = front->e;
		front->prev->next = front->next;
		front->next->prev = front->prev;
		free(front);
		q->count--;
	}
	return n;
}

uint32_t oracle_eager_rxq_pending(const oracle_eager_rxq_t *q)
{
	return q->count;
}

uint32_t oracle_eager_rxq_peek(const oracle_eager_rxq_t *q, oracle_eager_entry_t *out, uint32_t cap)
{
	uint32_t n = 0;
	for (const node_t *p = q->head.next; p != &q->head && n < cap; p = p->next) {
		out[n++] = p->e;
	}
	return n;
}

/* ---- sender's batch numbering ---- */

void oracle_eager_tx_init(oracle_eager_tx_t *tx)
{
	memset(tx, 0, sizeof(*tx));
}

/* send(), src/nccl_ofi_rdma.cpp:5783-5806 */
void oracle_eager_tx_assign(oracle_eager_tx_t *tx, int32_t tag, oracle_eager_hdr_t *hdr)
{
	if (tx->eager_offset_next == 0) {
		tx->cur_eager_seq = tx->eager_seq_next;
		tx->eager_seq_next++;
	}
	hdr->eager_offset = tx->eager_offset_next;
	hdr->prev_batch_count = tx->prev_eager_batch_count;
	hdr->eager_seq = tx->cur_eager_seq;
	hdr->tag = tag;
	tx->eager_offset_next++;
}

/* drain_sender_eager_queue, :5594-5598 and :5636-5640 */
void oracle_eager_tx_advance(oracle_eager_tx_t *tx)
{
	if (tx->eager_offset_next > 0) {
		tx->prev_eager_batch_count = tx->eager_offset_next;
		tx->eager_offset_next = 0;
	}
}

/* :5758-5764 */
int oracle_eager_fits(uint64_t size, int64_t eager_send_size)
{
	return (int64_t)(size + 8) <= eager_send_size;
}

/* The sentinel flush.  The GPU flush buffer is one cache line of sentinels
 * (src/nccl_ofi_rdma.cpp:7390-7394); a flush reads it into the 64-byte host slot of every
 * rail (rdma_flush_req::post, :2664-2713; slot = rail * 64, :2103-2106). */
void oracle_flush_post(const uint64_t flush_buf[8], uint64_t *slots, uint32_t num_rails)
{
	for (uint32_t r = 0; r < num_rails; r++) {
		memcpy(&slots[r * 8], flush_buf, 64);
	}
}

/* has_flush_completed, :2110-2126, and nccl_ofi_gin_iflush_req::test,
 * src/rdma/gin/nccl_ofi_gin_reqs.cpp:373-394: the first 8 bytes of every slot */
int oracle_flush_completed(const uint64_t *slots, uint32_t num_rails, uint64_t sentinel)
{
	for (uint32_t r = 0; r < num_rails; r++) {
		if (slots[r * 8] != sentinel) {
			return 0;
		}
	}
	return 1;
}

/* rdma_eager_copy_req::post, :2729-2776, for a batch: payload (after the 8-byte header)
 * of rx buffer i goes to dst[i], truncated to the destination's length; zero-length
 * arrivals copy nothing (:753-762).  copied[i] receives the byte count. */
void oracle_eager_copy_batch(const uint8_t *rx_base, const uint64_t *rx_off, const uint32_t *recv_len,
			     uint8_t *dst_base, const uint64_t *dst_off, const uint32_t *dst_len, uint32_t n,
			     uint32_t *copied)
{
	for (uint32_t i = 0; i < n; i++) {
		uint32_t len = recv_len[i];
		if (dst_len[i] < len) {
			len = dst_len[i];
		}
		if (len) {
			memcpy(dst_base + dst_off[i], rx_base + rx_off[i] + 8, len);
		}
		if (copied) {
			copied[i] = len;
		}
	}
}

/*
 * CPU oracle (test infrastructure): the send/receive protocol's state machines of the RDMA
 * transport without a fabric underneath -- message buffer, sender-side and receiver-side
 * eager queues, control-mailbox matching, completion accounting -- restated from the
 * reference with its own data structures (circular array, linked list, status ring).
 * Whatever the reference would hand to libfabric comes back to the caller as an action.
 *
 * The reference sources (src/nccl_ofi_msgbuff.cpp, src/nccl_ofi_rdma.cpp) include a generated
 * config.h and libfabric headers and do not build here.  Pinned by: the known answers of
 * tests/unit/msgbuff.cpp, tests/unit/ctrl_msg.cpp, and the who-receives-what outcomes of
 * tests/functional/eager_multirecv.cpp replayed through these functions.
 */
#include <stdlib.h>
#include <string.h>

#include "oracle.h"

#define SEQ_MASK 0x3FFu
#define MAILBOX 256u
#define MAX_EAGER_PENDING 32u /* NCCL_OFI_MAX_EAGER_PENDING = NCCL_NET_MAX_REQUESTS */
#define MAX_REQUESTS 128u
#define MAX_SEND_REQUESTS (MAX_REQUESTS * 8u)
#define EAGER_HEADER 8

/* ======================================================== message buffer */

typedef struct {
	int stat;
	int type;
	void *elem;
} mb_elem_t;

struct oracle_msgbuff {
	mb_elem_t *buff;
	uint16_t max_inprogress;
	uint16_t field_size;
	uint16_t field_mask;
	uint16_t msg_last_incomplete;
	uint16_t msg_next;
};

/* constructor, src/nccl_ofi_msgbuff.cpp:14-27 */
oracle_msgbuff_t *oracle_msgbuff_create(uint16_t max_inprogress, uint16_t bit_width, uint16_t start_seq)
{
	uint16_t field_size = (uint16_t)(1 << bit_width);
	if (max_inprogress == 0 || field_size <= 2 * max_inprogress) {
		return NULL;
	}
	oracle_msgbuff_t *m = (oracle_msgbuff_t *)calloc(1, sizeof(*m));
	if (!m) {
		return NULL;
	}
	m->buff = (mb_elem_t *)calloc(max_inprogress, sizeof(mb_elem_t));
	if (!m->buff) {
		free(m);
		return NULL;
	}
	m->max_inprogress = max_inprogress;
	m->field_size = field_size;
	m->field_mask = (uint16_t)(field_size - 1);
	m->msg_last_incomplete = start_seq;
	m->msg_next = start_seq;
	return m;
}

void oracle_msgbuff_destroy(oracle_msgbuff_t *m)
{
	if (m) {
		free(m->buff);
		free(m);
	}
}

/* :29-32 */
static uint16_t mb_distance(const oracle_msgbuff_t *m, uint16_t front, uint16_t back)
{
	return (uint16_t)((front < back ? m->field_size : 0) + front - back);
}

static mb_elem_t *mb_idx(const oracle_msgbuff_t *m, uint16_t idx)
{
	return &m->buff[idx % m->max_inprogress];
}

/* get_idx_status, :49-75 */
static int mb_status(const oracle_msgbuff_t *m, uint16_t msg_index)
{
	uint16_t inflight = mb_distance(m, m->msg_next, m->msg_last_incomplete);
	if (mb_distance(m, msg_index, m->msg_last_incomplete) < inflight) {
		return mb_idx(m, msg_index)->stat;
	}
	if (msg_index != m->msg_last_incomplete &&
	    mb_distance(m, m->msg_last_incomplete, msg_index) <= m->max_inprogress) {
		return ORACLE_MSGBUFF_COMPLETED;
	}
	if (mb_distance(m, msg_index, m->msg_next) < mb_distance(m, m->max_inprogress, inflight)) {
		return ORACLE_MSGBUFF_NOTSTARTED;
	}
	return ORACLE_MSGBUFF_UNAVAILABLE;
}

/* insert, :77-101 */
int oracle_msgbuff_insert(oracle_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status)
{
	*status = mb_status(m, msg_index);
	if (*status == ORACLE_MSGBUFF_NOTSTARTED) {
		mb_idx(m, msg_index)->stat = ORACLE_MSGBUFF_INPROGRESS;
		mb_idx(m, msg_index)->elem = elem;
		mb_idx(m, msg_index)->type = type;
		while (mb_distance(m, msg_index, m->msg_next) <= m->max_inprogress) {
			if (m->msg_next != msg_index) {
				mb_idx(m, m->msg_next)->stat = ORACLE_MSGBUFF_NOTSTARTED;
				mb_idx(m, m->msg_next)->elem = NULL;
			}
			m->msg_next = (uint16_t)((m->msg_next + 1) & m->field_mask);
		}
		return ORACLE_MSGBUFF_SUCCESS;
	}
	return ORACLE_MSGBUFF_INVALID_IDX;
}

/* replace, :103-118 */
int oracle_msgbuff_replace(oracle_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status)
{
	*status = mb_status(m, msg_index);
	if (*status == ORACLE_MSGBUFF_INPROGRESS) {
		mb_idx(m, msg_index)->elem = elem;
		mb_idx(m, msg_index)->type = type;
		return ORACLE_MSGBUFF_SUCCESS;
	}
	return ORACLE_MSGBUFF_INVALID_IDX;
}

/* retrieve, :120-145 */
int oracle_msgbuff_retrieve(oracle_msgbuff_t *m, uint16_t msg_index, void **elem, int *type, int *status)
{
	if (!elem) {
		return ORACLE_MSGBUFF_ERROR;
	}
	*status = mb_status(m, msg_index);
	if (*status == ORACLE_MSGBUFF_INPROGRESS) {
		*elem = mb_idx(m, msg_index)->elem;
		*type = mb_idx(m, msg_index)->type;
		return ORACLE_MSGBUFF_SUCCESS;
	}
	if (*status == ORACLE_MSGBUFF_UNAVAILABLE) {
		*status = ORACLE_MSGBUFF_NOTSTARTED;
	}
	return ORACLE_MSGBUFF_INVALID_IDX;
}

/* complete, :147-166 */
int oracle_msgbuff_complete(oracle_msgbuff_t *m, uint16_t msg_index, int *status)
{
	*status = mb_status(m, msg_index);
	if (*status == ORACLE_MSGBUFF_INPROGRESS) {
		mb_idx(m, msg_index)->stat = ORACLE_MSGBUFF_COMPLETED;
		mb_idx(m, msg_index)->elem = NULL;
		while (m->msg_last_incomplete != m->msg_next &&
		       mb_idx(m, m->msg_last_incomplete)->stat == ORACLE_MSGBUFF_COMPLETED) {
			m->msg_last_incomplete = (uint16_t)((m->msg_last_incomplete + 1) & m->field_mask);
		}
		return ORACLE_MSGBUFF_SUCCESS;
	}
	if (*status == ORACLE_MSGBUFF_UNAVAILABLE) {
		*status = ORACLE_MSGBUFF_NOTSTARTED;
	}
	return ORACLE_MSGBUFF_INVALID_IDX;
}

/* ================================================================ sender */

typedef struct {
	int in_use;
	uint16_t msg_seq_num;
	uint64_t size;     /* req->size */
	uint64_t buff_len; /* send_data->buff_len */
	int32_t tag;
	int eager;
	int eager_ctrl_msg_received;
	int ncompls;
	int total_num_compls;
	int completed;
	uint8_t recv_idx;
} send_req_t;

typedef struct {
	int32_t req;
	int32_t tag;
	uint8_t eager_offset;
} eager_q_entry_t;

struct oracle_send_comm {
	oracle_ctrl_msg_t mailbox[MAILBOX];
	send_req_t reqs[MAX_SEND_REQUESTS];
	eager_q_entry_t eager_queue[MAX_EAGER_PENDING];
	uint8_t eager_queue_head, eager_queue_tail, eager_queue_count;
	uint8_t eager_offset_next, prev_eager_batch_count;
	uint16_t cur_eager_seq, eager_seq_next;
	uint16_t next_msg_seq_num, group_sends_remaining, group_num_recvs;
	uint32_t num_inflight_reqs, num_inflight_writes;
	uint64_t n_ctrl_received;
	uint32_t remote_comm_id, num_rails;
	int64_t eager_send_size;
	oracle_sched_t sched;
};

oracle_send_comm_t *oracle_send_comm_create(uint32_t remote_comm_id, uint32_t num_rails,
					    int64_t eager_send_size, uint64_t min_stripe,
					    uint64_t max_small)
{
	if (num_rails < 1 || num_rails > 4) {
		return NULL;
	}
	oracle_send_comm_t *s = (oracle_send_comm_t *)calloc(1, sizeof(*s));
	if (!s) {
		return NULL;
	}
	s->next_msg_seq_num = 1; /* NCCL_OFI_RDMA_MSG_SEQ_NUM_START, src/nccl_ofi_rdma.cpp:6317 */
	s->remote_comm_id = remote_comm_id;
	s->num_rails = num_rails;
	s->eager_send_size = eager_send_size;
	oracle_sched_init(&s->sched, (int)num_rails, min_stripe, max_small);
	return s;
}

void oracle_send_comm_destroy(oracle_send_comm_t *s)
{
	free(s);
}

oracle_ctrl_msg_t *oracle_send_comm_mailbox(oracle_send_comm_t *s)
{
	return s->mailbox;
}

void oracle_send_comm_state(const oracle_send_comm_t *s, oracle_send_state_t *out)
{
	memset(out, 0, sizeof(*out));
	out->next_msg_seq_num = s->next_msg_seq_num;
	out->group_sends_remaining = s->group_sends_remaining;
	out->group_num_recvs = s->group_num_recvs;
	out->cur_eager_seq = s->cur_eager_seq;
	out->eager_seq_next = s->eager_seq_next;
	out->eager_queue_count = s->eager_queue_count;
	out->eager_offset_next = s->eager_offset_next;
	out->prev_eager_batch_count = s->prev_eager_batch_count;
	out->num_inflight_reqs = s->num_inflight_reqs;
	out->num_inflight_writes = s->num_inflight_writes;
	out->n_ctrl_received = s->n_ctrl_received;
}

static void close_eager_batch(oracle_send_comm_t *s)
{
	if (s->eager_offset_next > 0) {
		s->prev_eager_batch_count = s->eager_offset_next;
		s->eager_offset_next = 0;
	}
}

/* drain_sender_eager_queue, src/nccl_ofi_rdma.cpp:5561-5644 */
static int drain_sender_eager_queue(oracle_send_comm_t *s)
{
	while (s->eager_queue_count > 0) {
		uint16_t seq = s->next_msg_seq_num;
		if (!oracle_ctrl_msg_ready(s->mailbox, seq, 0, 1)) {
			return 0;
		}
		oracle_ctrl_msg_t *ctrl = &s->mailbox[seq % MAILBOX];
		uint16_t num_recvs = ctrl->entries[0].num_recvs;
		uint8_t head = s->eager_queue_head;
		eager_q_entry_t *entry = &s->eager_queue[head];
		send_req_t *send_data = &s->reqs[entry->req];
		s->eager_queue_head = (uint8_t)((head + 1) % MAX_EAGER_PENDING);
		s->eager_queue_count--;

		if (num_recvs <= 1) {
			if (ctrl->entries[0].tag != entry->tag) {
				uint8_t tail = s->eager_queue_tail;
				s->eager_queue[tail] = *entry;
				s->eager_queue_tail = (uint8_t)((tail + 1) % MAX_EAGER_PENDING);
				s->eager_queue_count++;
				break;
			}
			send_data->eager_ctrl_msg_received = 1;
			send_data->msg_seq_num = seq;
			s->n_ctrl_received += 1;
			s->next_msg_seq_num = (uint16_t)((seq + 1) & SEQ_MASK);
			close_eager_batch(s);
			continue;
		}

		if (s->group_sends_remaining == 0) {
			s->n_ctrl_received += 1;
			s->group_num_recvs = num_recvs;
			s->group_sends_remaining = num_recvs;
		}
		int found = 0;
		for (uint16_t e = 0; e < num_recvs; e++) {
			if (ctrl->entries[e].entry_used == 0 && ctrl->entries[e].tag == entry->tag) {
				send_data->eager_ctrl_msg_received = 1;
				ctrl->entries[e].entry_used = 1;
				send_data->msg_seq_num = seq;
				s->group_sends_remaining--;
				found = 1;
				break;
			}
		}
		if (!found) {
			uint8_t tail = s->eager_queue_tail;
			s->eager_queue[tail] = *entry;
			s->eager_queue_tail = (uint8_t)((tail + 1) % MAX_EAGER_PENDING);
			s->eager_queue_count++;
			break;
		}
		if (s->group_sends_remaining == 0) {
			s->next_msg_seq_num = (uint16_t)((seq + 1) & SEQ_MASK);
			s->group_num_recvs = 0;
			close_eager_batch(s);
		}
	}
	return 1;
}

static int alloc_send_req(oracle_send_comm_t *s)
{
	for (uint32_t i = 0; i < MAX_SEND_REQUESTS; i++) {
		if (!s->reqs[i].in_use) {
			memset(&s->reqs[i], 0, sizeof(s->reqs[i]));
			s->reqs[i].in_use = 1;
			return (int)i;
		}
	}
	return -1;
}

/* send, :5646-5860 (the fabric posts come back as the action) */
int oracle_send_comm_send(oracle_send_comm_t *s, uint64_t size, int32_t tag, oracle_send_action_t *act)
{
	int have_ctrl, eager = 0, in_group;
	uint16_t msg_seq_num;

	memset(act, 0, sizeof(*act));
	act->req = -1;
	if (s->num_inflight_reqs == MAX_SEND_REQUESTS) {
		return -22;
	}
	if (s->eager_queue_count > 0) {
		have_ctrl = drain_sender_eager_queue(s);
		if (have_ctrl) {
			have_ctrl = oracle_ctrl_msg_ready(s->mailbox, s->next_msg_seq_num, tag, 0);
		}
	} else {
		have_ctrl = oracle_ctrl_msg_ready(s->mailbox, s->next_msg_seq_num, tag, 0);
	}
	msg_seq_num = s->next_msg_seq_num;
	in_group = s->group_sends_remaining > 0;

	if (have_ctrl && !in_group) {
		uint16_t nr = s->mailbox[msg_seq_num % MAILBOX].entries[0].num_recvs;
		if (nr > 1) {
			s->group_num_recvs = nr;
			s->group_sends_remaining = nr;
			in_group = 1;
		}
	}
	if (!have_ctrl && !in_group && (int64_t)(size + EAGER_HEADER) <= s->eager_send_size &&
	    s->eager_queue_count < MAX_EAGER_PENDING && s->num_inflight_writes == 0 &&
	    (s->eager_queue_count == 0 || s->eager_offset_next > 0)) {
		eager = 1;
	}
	if (!have_ctrl) {
		if (!eager) {
			act->kind = ORACLE_SEND_AGAIN;
			return 0;
		}
	} else if (!in_group || s->group_sends_remaining == s->group_num_recvs) {
		s->n_ctrl_received += 1;
	}

	/* alloc_rdma_send_req, :5374-5425 */
	int r = alloc_send_req(s);
	if (r < 0) {
		return -12;
	}
	send_req_t *req = &s->reqs[r];
	req->msg_seq_num = msg_seq_num;
	req->size = size;
	req->buff_len = size;
	req->tag = tag;
	req->eager = eager;
	act->req = r;
	if (eager) {
		act->num_xfers = (uint32_t)oracle_sched_get_schedule(&s->sched, size, 128, act->xfers);
		req->total_num_compls = (int)act->num_xfers + 1;
		act->imm = oracle_rdma_imm(s->remote_comm_id, msg_seq_num, req->recv_idx, act->num_xfers);

		if (s->eager_offset_next == 0) {
			s->cur_eager_seq = s->eager_seq_next;
			s->eager_seq_next++;
		}
		act->hdr.eager_offset = s->eager_offset_next;
		act->hdr.prev_batch_count = s->prev_eager_batch_count;
		act->hdr.eager_seq = s->cur_eager_seq;
		act->hdr.tag = tag;
		uint8_t idx = s->eager_queue_tail;
		s->eager_queue[idx].req = r;
		s->eager_queue[idx].tag = tag;
		s->eager_queue[idx].eager_offset = s->eager_offset_next;
		s->eager_queue_tail = (uint8_t)((idx + 1) % MAX_EAGER_PENDING);
		s->eager_queue_count++;
		s->eager_offset_next++;
	}
	if (have_ctrl) {
		/* update_send_data_from_remote, :574-640 */
		oracle_ctrl_msg_t *ctrl = &s->mailbox[msg_seq_num % MAILBOX];
		oracle_ctrl_entry_t *entry = NULL;
		if (ctrl->entries[0].num_recvs <= 1) {
			entry = &ctrl->entries[0];
			req->recv_idx = 0;
		} else {
			for (uint16_t i = 0; i < ctrl->entries[0].num_recvs; i++) {
				if (ctrl->entries[i].tag == tag && !ctrl->entries[i].entry_used) {
					entry = &ctrl->entries[i];
					req->recv_idx = entry->recv_idx;
					break;
				}
			}
		}
		if (!entry) {
			req->in_use = 0;
			act->req = -1;
			return -22;
		}
		act->remote_buff_offset = entry->buff_offset;
		for (uint32_t rail = 0; rail < s->num_rails; rail++) {
			act->mr_key[rail] = entry->mr_key[rail];
		}
		entry->entry_used = 1;
		if (entry->buff_len < req->buff_len) {
			req->size = entry->buff_len;
			req->buff_len = entry->buff_len;
		}
		act->num_xfers = (uint32_t)oracle_sched_get_schedule(&s->sched, req->buff_len, 128, act->xfers);
		req->total_num_compls = (int)act->num_xfers;
		act->imm = oracle_rdma_imm(s->remote_comm_id, msg_seq_num, req->recv_idx, act->num_xfers);
		act->no_target_completion = (ctrl->entries[0].flags & 1u) ? 1 : 0;
	}
	s->num_inflight_reqs++;
	if (!eager) {
		s->num_inflight_writes++;
	}
	act->kind = eager ? ORACLE_SEND_EAGER : ORACLE_SEND_WRITE;
	act->msg_seq_num = msg_seq_num;
	act->recv_idx = req->recv_idx;
	act->size = req->buff_len;

	if (!eager) {
		uint16_t orig_seq = s->next_msg_seq_num;
		if (in_group) {
			s->group_sends_remaining--;
			if (s->group_sends_remaining == 0) {
				s->group_num_recvs = 0;
				s->next_msg_seq_num = (uint16_t)((s->next_msg_seq_num + 1) & SEQ_MASK);
			}
		} else {
			s->next_msg_seq_num = (uint16_t)((s->next_msg_seq_num + 1) & SEQ_MASK);
		}
		if (s->eager_offset_next > 0 && orig_seq != s->next_msg_seq_num) {
			s->prev_eager_batch_count = s->eager_offset_next;
			s->eager_offset_next = 0;
		}
	}
	return 0;
}

/* one fabric completion of the request: inc_req_completion, :487-510 */
int oracle_send_comm_completion(oracle_send_comm_t *s, int32_t r)
{
	if (r < 0 || (uint32_t)r >= MAX_SEND_REQUESTS || !s->reqs[r].in_use) {
		return -22;
	}
	send_req_t *req = &s->reqs[r];
	if (++req->ncompls == req->total_num_compls) {
		req->completed = 1;
	}
	return 0;
}

/* get_ctrl_msg_buff_len, :2183-2196 */
static uint32_t ctrl_buff_len(oracle_send_comm_t *s, uint16_t seq, int32_t tag)
{
	oracle_ctrl_msg_t *ctrl = &s->mailbox[seq % MAILBOX];
	if (ctrl->entries[0].num_recvs <= 1) {
		return ctrl->entries[0].buff_len;
	}
	for (uint16_t i = 0; i < ctrl->entries[0].num_recvs; i++) {
		if (ctrl->entries[i].tag == tag) {
			return ctrl->entries[i].buff_len;
		}
	}
	return 0;
}

/* test() for a send request, :2236-2307, with update_send_request :2204-2232 */
int oracle_send_comm_test(oracle_send_comm_t *s, int32_t r, int *done, uint64_t *size)
{
	*done = 0;
	if (r < 0 || (uint32_t)r >= MAX_SEND_REQUESTS || !s->reqs[r].in_use) {
		return -22;
	}
	send_req_t *req = &s->reqs[r];
	if (!req->completed) {
		if (s->eager_queue_count > 0) {
			drain_sender_eager_queue(s);
		}
		if (req->eager && req->eager_ctrl_msg_received && req->ncompls > 0) {
			uint32_t remote_len = ctrl_buff_len(s, req->msg_seq_num, req->tag);
			if (remote_len < req->buff_len) {
				req->size = remote_len;
				req->buff_len = remote_len;
			}
			if (++req->ncompls == req->total_num_compls) {
				req->completed = 1;
			}
		}
	}
	if (req->completed) {
		if (size) {
			*size = req->size;
		}
		*done = 1;
		if (!req->eager) {
			s->num_inflight_writes--;
		}
		s->num_inflight_reqs--;
		req->in_use = 0;
	}
	return 0;
}

/* ============================================================== receiver */

typedef struct {
	uint64_t dst;
	uint64_t dst_len;
	int32_t tag;
	uint64_t recv_size;
	int ncompls;
	uint64_t total_segms;
	int consumed;
	int has_eager_copy;
	uint32_t eager_len; /* recv_len of the rx buffer matched to this sub-receive */
} sub_recv_t;

typedef struct {
	int in_use;
	uint16_t msg_seq_num;
	int num_recvs;
	sub_recv_t recvs[8];
	int total_num_compls;
	int ncompls;
	uint64_t size;
	int completed;
	/* the receive-segments child request */
	int segms_ncompls;
	uint64_t segms_size;
} recv_req_t;

typedef struct rx_node {
	struct rx_node *prev, *next;
	uint64_t rx_cookie;
	uint16_t msg_seq_num;
	uint8_t eager_offset;
	uint8_t prev_batch_count;
	uint16_t eager_seq;
	int32_t tag;
	uint32_t recv_len;
	int handled;
} rx_node_t;

#define COPY_RING 1024u

struct oracle_recv_comm {
	oracle_msgbuff_t *msgbuff;
	recv_req_t reqs[MAX_REQUESTS];
	rx_node_t pool[MAILBOX];
	rx_node_t list; /* sentinel of the sorted arrivals */
	rx_node_t free; /* sentinel of the free entries */
	uint16_t last_eager_seq;
	uint8_t last_eager_offset;
	int has_processed_eager;
	uint16_t eager_drain_recv_seq;
	uint16_t last_completed_seq;
	uint16_t next_msg_seq_num;
	uint32_t num_inflight_reqs;
	uint64_t n_ctrl_sent;
	uint32_t num_rails;
	oracle_eager_copy_item_t copies[COPY_RING];
	uint32_t copy_head, copy_count;
	int flush_live[MAX_REQUESTS];
};

static void list_init(rx_node_t *h)
{
	h->prev = h->next = h;
}

static void list_remove(rx_node_t *n)
{
	n->prev->next = n->next;
	n->next->prev = n->prev;
}

static void list_push_back(rx_node_t *h, rx_node_t *n)
{
	n->prev = h->prev;
	n->next = h;
	h->prev->next = n;
	h->prev = n;
}

oracle_recv_comm_t *oracle_recv_comm_create(uint32_t num_rails)
{
	if (num_rails < 1 || num_rails > 4) {
		return NULL;
	}
	oracle_recv_comm_t *r = (oracle_recv_comm_t *)calloc(1, sizeof(*r));
	if (!r) {
		return NULL;
	}
	/* src/nccl_ofi_rdma.cpp:4917: 256 in flight, 10-bit sequence numbers from 1 */
	r->msgbuff = oracle_msgbuff_create(256, 10, 1);
	if (!r->msgbuff) {
		free(r);
		return NULL;
	}
	list_init(&r->list);
	list_init(&r->free);
	for (uint32_t i = 0; i < MAILBOX; i++) {
		list_push_back(&r->free, &r->pool[i]);
	}
	r->next_msg_seq_num = 1;     /* :4835 */
	r->eager_drain_recv_seq = 1; /* :4558 */
	r->num_rails = num_rails;
	return r;
}

void oracle_recv_comm_destroy(oracle_recv_comm_t *r)
{
	if (r) {
		oracle_msgbuff_destroy(r->msgbuff);
		free(r);
	}
}

/* inc_req_completion on the receive request, :487-510 */
static void recv_inc_completion(recv_req_t *req, uint64_t size)
{
	req->size += size;
	if (++req->ncompls == req->total_num_compls) {
		req->completed = 1;
	}
}

/* inc_recv_seg_completion, :530-572 */
static void recv_inc_seg_completion(recv_req_t *req, uint64_t size)
{
	req->segms_size += size;
	req->segms_ncompls++;
	if (req->segms_ncompls == req->num_recvs) {
		recv_inc_completion(req, req->segms_size);
	}
}

static int push_copy(oracle_recv_comm_t *r, const oracle_eager_copy_item_t *it)
{
	if (r->copy_count == COPY_RING) {
		return -12;
	}
	r->copies[(r->copy_head + r->copy_count) % COPY_RING] = *it;
	r->copy_count++;
	return 0;
}

/* eager_match_recv, :727-737 */
static int eager_match_recv(recv_req_t *req, int32_t tag)
{
	for (int i = 0; i < req->num_recvs; i++) {
		if (!req->recvs[i].consumed && req->recvs[i].tag == tag) {
			req->recvs[i].consumed = 1;
			return i;
		}
	}
	return -1;
}

/* eager_copy_to_sub_recv, :745-780: the loop-back read comes back as a copy item */
static int eager_copy_to_sub_recv(oracle_recv_comm_t *r, int req_id, rx_node_t *entry, int sub_idx)
{
	recv_req_t *req = &r->reqs[req_id];
	oracle_eager_copy_item_t it;
	memset(&it, 0, sizeof(it));
	it.rx_cookie = entry->rx_cookie;
	it.dst = req->recvs[sub_idx].dst;
	it.dst_len = req->recvs[sub_idx].dst_len;
	it.recv_len = entry->recv_len;
	it.req = req_id;
	it.sub_idx = sub_idx;
	it.needs_copy = entry->recv_len != 0;
	if (entry->recv_len == 0) {
		if (req->num_recvs > 1) {
			recv_inc_seg_completion(req, 0);
		} else {
			recv_inc_completion(req, 0);
		}
	} else {
		req->recvs[sub_idx].has_eager_copy = 1;
		/* rdma_eager_copy_req::post, :2738-2743, cuts the rx buffer's recv_len to the
		 * sub-receive's length before the read; the completion (:2936-2937) counts that */
		req->recvs[sub_idx].eager_len = entry->recv_len < req->recvs[sub_idx].dst_len
							? entry->recv_len
							: (uint32_t)req->recvs[sub_idx].dst_len;
	}
	return push_copy(r, &it);
}

static int entry_can_process(int has_processed, uint16_t last_seq, uint8_t last_off, const rx_node_t *e)
{
	oracle_eager_entry_t x;
	memset(&x, 0, sizeof(x));
	x.eager_offset = e->eager_offset;
	x.prev_batch_count = e->prev_batch_count;
	x.eager_seq = e->eager_seq;
	return oracle_eager_entry_can_process(has_processed, last_seq, last_off, &x);
}

/* drain_recv_eager_queue, :791-892 */
static int drain_recv_eager_queue(oracle_recv_comm_t *r)
{
	int skipping = 0;
	uint16_t tmp_last_eager_seq = r->last_eager_seq;
	uint8_t tmp_last_offset = r->last_eager_offset;
	int tmp_has_processed = r->has_processed_eager;
	uint16_t tmp_drain_recv_seq = r->eager_drain_recv_seq;

	rx_node_t *node = r->list.next, *next;
	for (; node != &r->list; node = next) {
		next = node->next;
		rx_node_t *entry = node;
		if (!entry_can_process(tmp_has_processed, tmp_last_eager_seq, tmp_last_offset, entry)) {
			break;
		}
		tmp_last_eager_seq = entry->eager_seq;
		tmp_last_offset = entry->eager_offset;
		tmp_has_processed = 1;

		if (entry->handled) {
			if (!skipping) {
				list_remove(node);
				list_push_back(&r->free, node);
				r->last_eager_seq = entry->eager_seq;
				r->last_eager_offset = entry->eager_offset;
				r->has_processed_eager = 1;
				r->eager_drain_recv_seq = tmp_drain_recv_seq;
			}
			continue;
		}
		if (entry->eager_offset == 0) {
			tmp_drain_recv_seq = entry->msg_seq_num;
		}
		uint16_t recv_seq = tmp_drain_recv_seq;
		int resolved = 0;
		while (!resolved) {
			void *elem;
			int type, stat;
			int res = oracle_msgbuff_retrieve(r->msgbuff, recv_seq, &elem, &type, &stat);
			if (res != ORACLE_MSGBUFF_SUCCESS || type != ORACLE_MSGBUFF_REQ) {
				if (res == ORACLE_MSGBUFF_INVALID_IDX && stat == ORACLE_MSGBUFF_COMPLETED) {
					recv_seq = (uint16_t)((recv_seq + 1) & SEQ_MASK);
					continue;
				}
				break;
			}
			int req_id = (int)((recv_req_t *)elem - r->reqs);
			recv_req_t *req = &r->reqs[req_id];
			int sub_idx = eager_match_recv(req, entry->tag);
			if (sub_idx >= 0) {
				int rc = eager_copy_to_sub_recv(r, req_id, entry, sub_idx);
				if (rc != 0) {
					return rc;
				}
				entry->handled = 1;
				int all_consumed = 1;
				for (int i = 0; i < req->num_recvs; i++) {
					if (!req->recvs[i].consumed) {
						all_consumed = 0;
						break;
					}
				}
				if (all_consumed) {
					tmp_drain_recv_seq = (uint16_t)((tmp_drain_recv_seq + 1) & SEQ_MASK);
				}
				resolved = 1;
			} else {
				recv_seq = (uint16_t)((recv_seq + 1) & SEQ_MASK);
			}
		}
		if (!resolved) {
			skipping = 1;
			continue;
		}
		if (!skipping) {
			list_remove(node);
			list_push_back(&r->free, node);
			r->last_eager_seq = entry->eager_seq;
			r->last_eager_offset = entry->eager_offset;
			r->has_processed_eager = 1;
			r->eager_drain_recv_seq = tmp_drain_recv_seq;
		}
	}
	return 0;
}

/* handle_eager_recv, :897-947; recv_len excludes the 8-byte header */
int oracle_recv_comm_eager_arrival(oracle_recv_comm_t *r, uint16_t msg_seq_num,
				   const oracle_eager_hdr_t *hdr, uint32_t recv_len, uint64_t rx_cookie)
{
	if (r->free.next == &r->free) {
		return -12;
	}
	rx_node_t *n = r->free.next;
	list_remove(n);
	n->rx_cookie = rx_cookie;
	n->msg_seq_num = msg_seq_num;
	n->eager_offset = hdr->eager_offset;
	n->tag = hdr->tag;
	n->prev_batch_count = hdr->prev_batch_count;
	n->eager_seq = hdr->eager_seq;
	n->recv_len = recv_len;
	n->handled = 0;
	/* recv_eager_sorted_insert, include/nccl_ofi_rdma.h:734-750 */
	rx_node_t *pos = r->list.prev;
	while (pos != &r->list) {
		oracle_eager_entry_t a, b;
		memset(&a, 0, sizeof(a));
		memset(&b, 0, sizeof(b));
		a.eager_seq = n->eager_seq;
		a.eager_offset = n->eager_offset;
		b.eager_seq = pos->eager_seq;
		b.eager_offset = pos->eager_offset;
		if (!oracle_eager_entry_less(&a, &b)) {
			break;
		}
		pos = pos->prev;
	}
	n->prev = pos;
	n->next = pos->next;
	pos->next->prev = n;
	pos->next = n;
	return drain_recv_eager_queue(r);
}

/* recv, :3545-3745, with allocate_recv_req :3398-3474 and
 * insert_rdma_recv_req_into_msgbuff :3478-3520 */
int oracle_recv_comm_recv(oracle_recv_comm_t *r, int n, const uint64_t *dsts, const uint64_t *sizes,
			  const int *tags, const uint64_t *mr_keys, int completion_optional,
			  oracle_ctrl_msg_t *mailbox, int32_t *req_out, uint16_t *seq_out)
{
	*req_out = -1;
	if (n < 1 || n > 8) {
		return -22;
	}
	if (r->num_inflight_reqs == MAX_REQUESTS) {
		return -28;
	}
	uint16_t msg_seq_num = r->next_msg_seq_num;
	void *elem;
	int type, stat;
	int res = oracle_msgbuff_retrieve(r->msgbuff, msg_seq_num, &elem, &type, &stat);
	if (res == ORACLE_MSGBUFF_SUCCESS) {
		return -22; /* duplicate request (eager arrivals never enter the message buffer) */
	} else if (!(res == ORACLE_MSGBUFF_INVALID_IDX && stat == ORACLE_MSGBUFF_NOTSTARTED)) {
		return -22;
	}
	int id = -1;
	for (uint32_t i = 0; i < MAX_REQUESTS; i++) {
		if (!r->reqs[i].in_use) {
			id = (int)i;
			break;
		}
	}
	if (id < 0) {
		return -22;
	}
	recv_req_t *req = &r->reqs[id];
	memset(req, 0, sizeof(*req));
	req->in_use = 1;
	req->msg_seq_num = msg_seq_num;
	req->total_num_compls = completion_optional ? 1 : 2;
	req->num_recvs = n;
	uint32_t lens[8];
	for (int i = 0; i < n; i++) {
		req->recvs[i].dst = dsts[i];
		req->recvs[i].dst_len = sizes[i];
		req->recvs[i].tag = tags[i];
		lens[i] = (uint32_t)sizes[i];
	}
	/* the control message into the sender's mailbox, :3446-3474 */
	int rc = oracle_ctrl_msg_fill(mailbox, msg_seq_num, (uint16_t)n, dsts, lens, tags, mr_keys,
				      r->num_rails, completion_optional);
	if (rc != 0) {
		req->in_use = 0;
		return rc;
	}
	res = oracle_msgbuff_insert(r->msgbuff, msg_seq_num, req, ORACLE_MSGBUFF_REQ, &stat);
	if (res != ORACLE_MSGBUFF_SUCCESS) {
		req->in_use = 0;
		return -22;
	}
	r->num_inflight_reqs++;
	r->n_ctrl_sent += 1;
	*req_out = id;
	*seq_out = msg_seq_num;
	r->next_msg_seq_num = (uint16_t)((r->next_msg_seq_num + 1) & SEQ_MASK);
	if (r->list.next != &r->list) {
		return drain_recv_eager_queue(r);
	}
	return 0;
}

/* completion of the control-message post */
int oracle_recv_comm_ctrl_sent(oracle_recv_comm_t *r, int32_t id)
{
	if (id < 0 || (uint32_t)id >= MAX_REQUESTS || !r->reqs[id].in_use) {
		return -22;
	}
	recv_inc_completion(&r->reqs[id], 0);
	return 0;
}

/* handle_write_comp, :1102-1130, with get_req_from_imm_data :1060-1097 */
int oracle_recv_comm_write_arrival(oracle_recv_comm_t *r, uint32_t imm, uint64_t len)
{
	uint32_t comm_id, seq, recv_idx, nseg;
	oracle_rdma_imm_decode(imm, &comm_id, &seq, &recv_idx, &nseg);
	void *elem;
	int type, stat;
	if (oracle_msgbuff_retrieve(r->msgbuff, (uint16_t)seq, &elem, &type, &stat) != ORACLE_MSGBUFF_SUCCESS ||
	    type != ORACLE_MSGBUFF_REQ) {
		return -22;
	}
	recv_req_t *req = (recv_req_t *)elem;
	sub_recv_t *sub = &req->recvs[recv_idx];
	sub->recv_size += len;
	sub->total_segms = nseg;
	sub->ncompls++;
	if (sub->ncompls == (int)nseg) {
		recv_inc_seg_completion(req, sub->recv_size);
	}
	return 0;
}

uint32_t oracle_recv_comm_take_copies(oracle_recv_comm_t *r, oracle_eager_copy_item_t *out, uint32_t cap)
{
	uint32_t n = 0;
	while (n < cap && r->copy_count > 0) {
		out[n++] = r->copies[r->copy_head];
		r->copy_head = (r->copy_head + 1) % COPY_RING;
		r->copy_count--;
	}
	return n;
}

/* rdma_eager_copy_req::handle_completion, :2920-2957 */
int oracle_recv_comm_copy_done(oracle_recv_comm_t *r, int32_t id, int32_t sub_idx)
{
	if (id < 0 || (uint32_t)id >= MAX_REQUESTS || !r->reqs[id].in_use || sub_idx < 0 ||
	    sub_idx >= r->reqs[id].num_recvs || !r->reqs[id].recvs[sub_idx].has_eager_copy) {
		return -22;
	}
	recv_req_t *req = &r->reqs[id];
	uint64_t eager_size = req->recvs[sub_idx].eager_len;
	req->recvs[sub_idx].has_eager_copy = 0;
	req->recvs[sub_idx].recv_size += eager_size;
	if (req->num_recvs > 1) {
		recv_inc_seg_completion(req, eager_size);
	} else {
		recv_inc_completion(req, eager_size);
	}
	return 0;
}

/* test() for a receive request, :2236-2307, sizes by write_completion_size :2340-2353,
 * freed through rdma_recv_req::free :1677-1695 */
int oracle_recv_comm_test(oracle_recv_comm_t *r, int32_t id, int *done, int *sizes)
{
	*done = 0;
	if (id < 0 || (uint32_t)id >= MAX_REQUESTS || !r->reqs[id].in_use) {
		return -22;
	}
	recv_req_t *req = &r->reqs[id];
	if (!req->completed) {
		return 0;
	}
	if (sizes) {
		if (req->num_recvs > 1) {
			for (int i = 0; i < req->num_recvs; i++) {
				sizes[i] = (int)req->recvs[i].recv_size;
			}
		} else {
			sizes[0] = (int)req->size;
		}
	}
	*done = 1;
	int stat;
	if (oracle_msgbuff_complete(r->msgbuff, req->msg_seq_num, &stat) != ORACLE_MSGBUFF_SUCCESS) {
		return -22;
	}
	r->last_completed_seq = req->msg_seq_num;
	r->num_inflight_reqs--;
	req->in_use = 0;
	return 0;
}

/* flush, src/nccl_ofi_rdma.cpp:4405-4510 (the fabric post is the caller's) */
int oracle_recv_comm_flush(oracle_recv_comm_t *r, int n, const int *sizes, int32_t *req)
{
	*req = -1;
	if (n < 1 || n > 8) {
		return -22;
	}
	if (r->num_inflight_reqs == MAX_REQUESTS) {
		return -28;
	}
	int flush_n = -1;
	for (int recv_n = 0; recv_n < n; recv_n++) {
		if (sizes[recv_n] != 0) {
			flush_n = recv_n;
			break;
		}
	}
	if (flush_n == -1) {
		return 0;
	}
	for (uint32_t i = 0; i < MAX_REQUESTS; i++) {
		if (!r->flush_live[i]) {
			r->flush_live[i] = 1;
			r->num_inflight_reqs++;
			*req = (int32_t)i;
			return 0;
		}
	}
	return -28;
}

/* has_flush_completed, :2110-2126, then the request is released */
int oracle_recv_comm_flush_test(oracle_recv_comm_t *r, int32_t req, const uint64_t *slots,
				uint32_t num_rails, uint64_t sentinel, int *done)
{
	if (req < 0 || (uint32_t)req >= MAX_REQUESTS || !r->flush_live[req]) {
		return -22;
	}
	*done = oracle_flush_completed(slots, num_rails, sentinel);
	if (*done) {
		r->flush_live[req] = 0;
		r->num_inflight_reqs--;
	}
	return 0;
}

void oracle_recv_comm_state(const oracle_recv_comm_t *r, oracle_recv_state_t *out)
{
	memset(out, 0, sizeof(*out));
	out->next_msg_seq_num = r->next_msg_seq_num;
	out->eager_drain_recv_seq = r->eager_drain_recv_seq;
	out->last_eager_seq = r->last_eager_seq;
	out->last_completed_seq = r->last_completed_seq;
	out->last_eager_offset = r->last_eager_offset;
	out->has_processed_eager = (uint8_t)r->has_processed_eager;
	out->num_inflight_reqs = r->num_inflight_reqs;
	uint32_t pending = 0;
	for (const rx_node_t *p = r->list.next; p != &r->list; p = p->next) {
		pending++;
	}
	out->eager_pending = pending;
	out->n_ctrl_sent = r->n_ctrl_sent;
}

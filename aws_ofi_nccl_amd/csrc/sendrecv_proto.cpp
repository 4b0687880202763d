/*
 * Send/receive protocol state machines (include/ofi_amd_sendrecv.h): the decisions of the
 * reference's RDMA transport around a message, with the fabric posts returned as actions.
 * Decision rules and sequence arithmetic are the reference's; each function cites its source.
 * Storage is this library's own: index windows over flat arrays, free-index stacks for the
 * request pools, a sorted vector for the receiver's arrivals.
 */
#include <cerrno>
#include <cstring>
#include <deque>
#include <mutex>
#include <new>
#include <vector>

#include "ofi_amd_sendrecv.h"

namespace {

constexpr uint16_t kSeqMask = (1u << OFI_AMD_RDMA_SEQ_BITS) - 1;
constexpr uint64_t kStripeAlign = 128;

inline uint16_t seq_next(uint16_t s)
{
	return static_cast<uint16_t>((s + 1) & kSeqMask);
}

/* Fixed pool of T with O(1) take/give of indices. */
template <typename T, uint32_t N>
struct Pool {
	T items[N];
	bool live[N] = {};
	uint16_t free_ids[N];
	uint32_t n_free = N;

	Pool()
	{
		for (uint32_t i = 0; i < N; i++) {
			free_ids[i] = static_cast<uint16_t>(N - 1 - i); /* lowest index first */
		}
	}
	int take()
	{
		if (n_free == 0) {
			return -1;
		}
		const int id = free_ids[--n_free];
		items[id] = T();
		live[id] = true;
		return id;
	}
	void give(int id)
	{
		live[id] = false;
		free_ids[n_free++] = static_cast<uint16_t>(id);
	}
	bool valid(int32_t id) const
	{
		return id >= 0 && static_cast<uint32_t>(id) < N && live[id];
	}
};

} // namespace

/* ======================================================== message buffer */

struct ofi_amd_msgbuff {
	struct Slot {
		uint8_t stat = OFI_AMD_MSGBUFF_COMPLETED;
		uint8_t type = OFI_AMD_MSGBUFF_REQ;
		void *elem = nullptr;
	};
	std::vector<Slot> slots;
	uint16_t window;   /* most messages in progress */
	uint16_t mask;     /* sequence numbers are 0..mask */
	uint16_t low;      /* oldest message not completed */
	uint16_t high;     /* one past the newest message inserted */
	std::mutex lock;

	Slot &at(uint16_t seq)
	{
		return slots[seq % window];
	}
	uint16_t ahead(uint16_t a, uint16_t b) const /* steps from b up to a, wrapping */
	{
		return static_cast<uint16_t>((a - b) & mask);
	}
	/* get_idx_status, src/nccl_ofi_msgbuff.cpp:49-75 */
	int status(uint16_t seq)
	{
		const uint16_t inflight = ahead(high, low);
		if (ahead(seq, low) < inflight) {
			return at(seq).stat;
		}
		if (seq != low && ahead(low, seq) <= window) {
			return OFI_AMD_MSGBUFF_COMPLETED; /* the window's worth of numbers behind `low` */
		}
		if (ahead(seq, high) < static_cast<uint16_t>(window - inflight)) {
			return OFI_AMD_MSGBUFF_NOTSTARTED;
		}
		return OFI_AMD_MSGBUFF_UNAVAILABLE;
	}
};

extern "C" {

/* constructor, src/nccl_ofi_msgbuff.cpp:14-27 */
int ofi_amd_msgbuff_create(uint16_t max_inprogress, uint16_t bit_width, uint16_t start_seq,
			   ofi_amd_msgbuff_t **out)
{
	if (!out || bit_width == 0 || bit_width > 15) {
		return -EINVAL;
	}
	const uint32_t field = 1u << bit_width;
	if (max_inprogress == 0 || field <= 2u * max_inprogress || start_seq >= field) {
		return -EINVAL;
	}
	ofi_amd_msgbuff_t *m = new (std::nothrow) ofi_amd_msgbuff();
	if (!m) {
		return -ENOMEM;
	}
	try {
		m->slots.resize(max_inprogress);
	} catch (...) {
		delete m;
		return -ENOMEM;
	}
	m->window = max_inprogress;
	m->mask = static_cast<uint16_t>(field - 1);
	m->low = m->high = start_seq;
	*out = m;
	return 0;
}

int ofi_amd_msgbuff_destroy(ofi_amd_msgbuff_t *m)
{
	if (!m) {
		return -EINVAL;
	}
	delete m;
	return 0;
}

/* insert, :77-101 */
int ofi_amd_msgbuff_insert(ofi_amd_msgbuff_t *m, uint16_t seq, void *elem, int type, int *status)
{
	if (!m || !status || seq > m->mask) {
		return OFI_AMD_MSGBUFF_ERROR;
	}
	std::lock_guard<std::mutex> guard(m->lock);
	*status = m->status(seq);
	if (*status != OFI_AMD_MSGBUFF_NOTSTARTED) {
		return OFI_AMD_MSGBUFF_INVALID_IDX;
	}
	ofi_amd_msgbuff::Slot &slot = m->at(seq);
	slot.stat = OFI_AMD_MSGBUFF_INPROGRESS;
	slot.type = static_cast<uint8_t>(type);
	slot.elem = elem;
	if (m->ahead(seq, m->low) >= m->ahead(m->high, m->low)) {
		/* at or beyond `high`: the numbers skipped over become known-but-empty slots and
		 * `high` moves past seq.  (A number skipped earlier is filled in place.)  The
		 * skipped slots are written after seq's own, as the reference does: when the
		 * window does not divide the sequence space two numbers of one window can share
		 * a slot across the wrap, and then the later write is the one that stays. */
		for (uint16_t s = m->high; s != seq; s = static_cast<uint16_t>((s + 1) & m->mask)) {
			m->at(s).stat = OFI_AMD_MSGBUFF_NOTSTARTED;
			m->at(s).elem = nullptr;
		}
		m->high = static_cast<uint16_t>((seq + 1) & m->mask);
	}
	return OFI_AMD_MSGBUFF_SUCCESS;
}

/* replace, :103-118 */
int ofi_amd_msgbuff_replace(ofi_amd_msgbuff_t *m, uint16_t seq, void *elem, int type, int *status)
{
	if (!m || !status || seq > m->mask) {
		return OFI_AMD_MSGBUFF_ERROR;
	}
	std::lock_guard<std::mutex> guard(m->lock);
	*status = m->status(seq);
	if (*status != OFI_AMD_MSGBUFF_INPROGRESS) {
		return OFI_AMD_MSGBUFF_INVALID_IDX;
	}
	m->at(seq).elem = elem;
	m->at(seq).type = static_cast<uint8_t>(type);
	return OFI_AMD_MSGBUFF_SUCCESS;
}

/* retrieve, :120-145 */
int ofi_amd_msgbuff_retrieve(ofi_amd_msgbuff_t *m, uint16_t seq, void **elem, int *type, int *status)
{
	if (!m || !elem || !type || !status || seq > m->mask) {
		return OFI_AMD_MSGBUFF_ERROR;
	}
	std::lock_guard<std::mutex> guard(m->lock);
	*status = m->status(seq);
	if (*status == OFI_AMD_MSGBUFF_INPROGRESS) {
		*elem = m->at(seq).elem;
		*type = m->at(seq).type;
		return OFI_AMD_MSGBUFF_SUCCESS;
	}
	if (*status == OFI_AMD_MSGBUFF_UNAVAILABLE) {
		*status = OFI_AMD_MSGBUFF_NOTSTARTED; /* "unavailable" only means something to insert */
	}
	return OFI_AMD_MSGBUFF_INVALID_IDX;
}

/* complete, :147-166 */
int ofi_amd_msgbuff_complete(ofi_amd_msgbuff_t *m, uint16_t seq, int *status)
{
	if (!m || !status || seq > m->mask) {
		return OFI_AMD_MSGBUFF_ERROR;
	}
	std::lock_guard<std::mutex> guard(m->lock);
	*status = m->status(seq);
	if (*status == OFI_AMD_MSGBUFF_INPROGRESS) {
		m->at(seq).stat = OFI_AMD_MSGBUFF_COMPLETED;
		m->at(seq).elem = nullptr;
		while (m->low != m->high && m->at(m->low).stat == OFI_AMD_MSGBUFF_COMPLETED) {
			m->low = static_cast<uint16_t>((m->low + 1) & m->mask);
		}
		return OFI_AMD_MSGBUFF_SUCCESS;
	}
	if (*status == OFI_AMD_MSGBUFF_UNAVAILABLE) {
		*status = OFI_AMD_MSGBUFF_NOTSTARTED;
	}
	return OFI_AMD_MSGBUFF_INVALID_IDX;
}

} // extern "C"

/* ================================================================ sender */

namespace {

struct SendReq {
	uint16_t msg_seq_num = 0;
	uint64_t size = 0;     /* what test() reports */
	uint64_t buff_len = 0; /* what is left to move after truncation */
	int32_t tag = 0;
	bool eager = false;
	bool ctrl_seen = false; /* eager only: its control message has been matched */
	bool completed = false;
	int ncompls = 0;
	int total_compls = 0;
	uint8_t recv_idx = 0;
};

struct PendingEager {
	int32_t req;
	int32_t tag;
};

} // namespace

struct ofi_amd_send_comm {
	ofi_amd_ctrl_msg_t mailbox[OFI_AMD_CTRL_MAILBOX_SIZE];
	Pool<SendReq, OFI_AMD_MAX_SEND_REQUESTS> reqs;
	std::deque<PendingEager> unmatched; /* eager sends whose control message is still to come */
	uint8_t eager_offset_next = 0;
	uint8_t prev_eager_batch_count = 0;
	uint16_t cur_eager_seq = 0;
	uint16_t eager_seq_next = 0;
	uint16_t next_msg_seq_num = OFI_AMD_RDMA_MSG_SEQ_NUM_START;
	uint16_t group_sends_remaining = 0;
	uint16_t group_num_recvs = 0;
	uint32_t inflight_reqs = 0;
	uint32_t inflight_writes = 0;
	uint64_t n_ctrl_received = 0;
	uint32_t remote_comm_id = 0;
	uint32_t num_rails = 0;
	int64_t eager_send_size = 0;
	ofi_amd_sched_state_t sched = {};

	ofi_amd_ctrl_msg_t &slot_of(uint16_t seq)
	{
		return mailbox[ofi_amd_ctrl_mailbox_slot(seq)];
	}
	/* the sequence number moves on: an open eager batch is closed and its length kept for
	 * the next batch's header */
	void advance_seq()
	{
		next_msg_seq_num = seq_next(next_msg_seq_num);
		if (eager_offset_next > 0) {
			prev_eager_batch_count = eager_offset_next;
			eager_offset_next = 0;
		}
	}
	bool match_unmatched();
};

/* drain_sender_eager_queue, src/nccl_ofi_rdma.cpp:5561-5644: walk the eager sends that went out
 * ahead of their control messages against the mailbox, oldest first; one that does not match
 * the control message at hand goes to the back and the walk stops.  False when the control
 * message for next_msg_seq_num has not arrived. */
bool ofi_amd_send_comm::match_unmatched()
{
	while (!unmatched.empty()) {
		const uint16_t seq = next_msg_seq_num;
		if (!ofi_amd_ctrl_msg_ready(mailbox, seq, 0, 1)) {
			return false;
		}
		ofi_amd_ctrl_msg_t &ctrl = slot_of(seq);
		const uint16_t num_recvs = ctrl.entries[0].num_recvs;
		const PendingEager front = unmatched.front();
		unmatched.pop_front();
		SendReq &req = reqs.items[front.req];

		if (num_recvs <= 1) {
			if (ctrl.entries[0].tag != front.tag) {
				unmatched.push_back(front);
				break;
			}
			req.ctrl_seen = true;
			req.msg_seq_num = seq;
			n_ctrl_received++;
			advance_seq();
			continue;
		}
		if (group_sends_remaining == 0) { /* first send of a grouped receive */
			n_ctrl_received++;
			group_num_recvs = num_recvs;
			group_sends_remaining = num_recvs;
		}
		int hit = -1;
		for (uint16_t e = 0; e < num_recvs && hit < 0; e++) {
			if (ctrl.entries[e].entry_used == 0 && ctrl.entries[e].tag == front.tag) {
				hit = e;
			}
		}
		if (hit < 0) {
			unmatched.push_back(front);
			break;
		}
		ctrl.entries[hit].entry_used = 1;
		req.ctrl_seen = true;
		req.msg_seq_num = seq;
		if (--group_sends_remaining == 0) {
			group_num_recvs = 0;
			advance_seq();
		}
	}
	return true;
}

extern "C" {

int ofi_amd_send_comm_create(uint32_t remote_comm_id, uint32_t num_rails, int64_t eager_send_size,
			     uint64_t min_stripe_size, uint64_t max_small_msg_size,
			     ofi_amd_send_comm_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS ||
	    remote_comm_id >= (1u << OFI_AMD_RDMA_COMM_ID_BITS)) {
		return -EINVAL;
	}
	ofi_amd_send_comm_t *s = new (std::nothrow) ofi_amd_send_comm();
	if (!s) {
		return -ENOMEM;
	}
	std::memset(s->mailbox, 0, sizeof(s->mailbox));
	s->remote_comm_id = remote_comm_id;
	s->num_rails = num_rails;
	s->eager_send_size = eager_send_size;
	s->sched.max_small_msg_size = max_small_msg_size;
	s->sched.min_stripe_size = min_stripe_size;
	s->sched.num_rails = static_cast<int32_t>(num_rails);
	*out = s;
	return 0;
}

int ofi_amd_send_comm_destroy(ofi_amd_send_comm_t *s)
{
	if (!s) {
		return -EINVAL;
	}
	delete s;
	return 0;
}

ofi_amd_ctrl_msg_t *ofi_amd_send_comm_mailbox(ofi_amd_send_comm_t *s)
{
	return s ? s->mailbox : nullptr;
}

void ofi_amd_send_comm_state(const ofi_amd_send_comm_t *s, ofi_amd_send_state_t *out)
{
	if (!s || !out) {
		return;
	}
	std::memset(out, 0, sizeof(*out));
	out->next_msg_seq_num = s->next_msg_seq_num;
	out->group_sends_remaining = s->group_sends_remaining;
	out->group_num_recvs = s->group_num_recvs;
	out->cur_eager_seq = s->cur_eager_seq;
	out->eager_seq_next = s->eager_seq_next;
	out->eager_queue_count = static_cast<uint8_t>(s->unmatched.size());
	out->eager_offset_next = s->eager_offset_next;
	out->prev_eager_batch_count = s->prev_eager_batch_count;
	out->num_inflight_reqs = s->inflight_reqs;
	out->num_inflight_writes = s->inflight_writes;
	out->n_ctrl_received = s->n_ctrl_received;
}

/* send, src/nccl_ofi_rdma.cpp:5646-5860 */
int ofi_amd_send_comm_send(ofi_amd_send_comm_t *s, uint64_t size, int32_t tag,
			   ofi_amd_send_action_t *action)
{
	if (!s || !action) {
		return -EINVAL;
	}
	std::memset(action, 0, sizeof(*action));
	action->kind = OFI_AMD_SEND_AGAIN;
	action->req = -1;
	if (s->inflight_reqs == OFI_AMD_MAX_SEND_REQUESTS) {
		return -EINVAL;
	}

	/* settle earlier eager sends first; only then may this send look at the mailbox */
	bool have_ctrl = s->unmatched.empty() || s->match_unmatched();
	if (have_ctrl) {
		have_ctrl = ofi_amd_ctrl_msg_ready(s->mailbox, s->next_msg_seq_num, tag, 0) != 0;
	}
	const uint16_t seq = s->next_msg_seq_num;
	bool in_group = s->group_sends_remaining > 0;
	if (have_ctrl && !in_group) {
		const uint16_t nr = s->slot_of(seq).entries[0].num_recvs;
		if (nr > 1) {
			s->group_num_recvs = nr;
			s->group_sends_remaining = nr;
			in_group = true;
		}
	}

	/* eager: no control message yet, small enough, room in the queue, nothing written and
	 * still in flight, and not behind an unmatched batch that has already been closed */
	const bool eager = !have_ctrl && !in_group && ofi_amd_eager_fits(size, s->eager_send_size) &&
			   s->unmatched.size() < OFI_AMD_MAX_EAGER_PENDING && s->inflight_writes == 0 &&
			   (s->unmatched.empty() || s->eager_offset_next > 0);
	if (!have_ctrl && !eager) {
		return 0; /* call again */
	}
	if (have_ctrl && (!in_group || s->group_sends_remaining == s->group_num_recvs)) {
		s->n_ctrl_received++;
	}

	const int id = s->reqs.take();
	if (id < 0) {
		return -ENOMEM;
	}
	SendReq &req = s->reqs.items[id];
	req.msg_seq_num = seq;
	req.size = req.buff_len = size;
	req.tag = tag;
	req.eager = eager;

	if (eager) {
		/* alloc_rdma_send_req, :5409-5421: one stripe, plus one completion for the control
		 * message that has yet to arrive */
		action->num_xfers = static_cast<uint32_t>(
			ofi_amd_sched_get_schedule(&s->sched, size, kStripeAlign, action->xfers));
		req.total_compls = static_cast<int>(action->num_xfers) + 1;
		if (s->eager_offset_next == 0) { /* a new batch takes the next batch number */
			s->cur_eager_seq = s->eager_seq_next++;
		}
		action->hdr.eager_offset = s->eager_offset_next++;
		action->hdr.prev_batch_count = s->prev_eager_batch_count;
		action->hdr.eager_seq = s->cur_eager_seq;
		action->hdr.tag = tag;
		s->unmatched.push_back(PendingEager{ id, tag });
	} else {
		/* update_send_data_from_remote, :574-640 */
		ofi_amd_ctrl_msg_t &ctrl = s->slot_of(seq);
		ofi_amd_ctrl_entry_t *entry = nullptr;
		if (ctrl.entries[0].num_recvs <= 1) {
			entry = &ctrl.entries[0];
		} else {
			for (uint16_t i = 0; i < ctrl.entries[0].num_recvs && !entry; i++) {
				if (ctrl.entries[i].tag == tag && !ctrl.entries[i].entry_used) {
					entry = &ctrl.entries[i];
					req.recv_idx = entry->recv_idx;
				}
			}
		}
		if (!entry) {
			s->reqs.give(id);
			return -EINVAL;
		}
		entry->entry_used = 1;
		action->remote_buff_offset = entry->buff_offset;
		for (uint32_t rail = 0; rail < s->num_rails; rail++) {
			action->mr_key[rail] = entry->mr_key[rail];
		}
		if (entry->buff_len < req.buff_len) { /* the receive buffer is the smaller one */
			req.size = req.buff_len = entry->buff_len;
		}
		action->num_xfers = static_cast<uint32_t>(
			ofi_amd_sched_get_schedule(&s->sched, req.buff_len, kStripeAlign, action->xfers));
		req.total_compls = static_cast<int>(action->num_xfers);
		action->no_target_completion =
			(ctrl.entries[0].flags & OFI_AMD_CTRL_FLAG_RECV_COMPLETION_OPT) ? 1 : 0;
	}
	action->kind = eager ? OFI_AMD_SEND_EAGER : OFI_AMD_SEND_WRITE;
	action->req = id;
	action->msg_seq_num = seq;
	action->recv_idx = req.recv_idx;
	action->size = req.buff_len;
	action->imm = ofi_amd_rdma_imm(s->remote_comm_id, seq, req.recv_idx, action->num_xfers);
	s->inflight_reqs++;

	if (!eager) {
		s->inflight_writes++;
		/* an eager send leaves the sequence number alone: the match settles it later */
		if (!in_group) {
			s->advance_seq();
		} else if (--s->group_sends_remaining == 0) {
			s->group_num_recvs = 0;
			s->advance_seq();
		}
	}
	return 0;
}

/* inc_req_completion, :487-510 */
int ofi_amd_send_comm_completion(ofi_amd_send_comm_t *s, int32_t id)
{
	if (!s || !s->reqs.valid(id)) {
		return -EINVAL;
	}
	SendReq &req = s->reqs.items[id];
	if (++req.ncompls == req.total_compls) {
		req.completed = true;
	}
	return 0;
}

/* nccl_net_ofi_rdma_req::test for a send, :2236-2307, with update_send_request :2204-2232 */
int ofi_amd_send_comm_test(ofi_amd_send_comm_t *s, int32_t id, int *done, uint64_t *size)
{
	if (!s || !done || !s->reqs.valid(id)) {
		return -EINVAL;
	}
	*done = 0;
	SendReq &req = s->reqs.items[id];
	if (!req.completed) {
		if (!s->unmatched.empty()) {
			s->match_unmatched();
		}
		/* an eager send is over once it is on the wire and its control message is known */
		if (req.eager && req.ctrl_seen && req.ncompls > 0) {
			/* get_ctrl_msg_buff_len, :2183-2196 */
			const ofi_amd_ctrl_msg_t &ctrl = s->slot_of(req.msg_seq_num);
			uint32_t remote_len = 0;
			if (ctrl.entries[0].num_recvs <= 1) {
				remote_len = ctrl.entries[0].buff_len;
			} else {
				const int e = ofi_amd_ctrl_msg_find_tag(&ctrl, req.tag);
				remote_len = e >= 0 ? ctrl.entries[e].buff_len : 0;
			}
			if (remote_len < req.buff_len) {
				req.size = req.buff_len = remote_len;
			}
			if (++req.ncompls == req.total_compls) {
				req.completed = true;
			}
		}
	}
	if (req.completed) {
		if (size) {
			*size = req.size;
		}
		*done = 1;
		if (!req.eager) {
			s->inflight_writes--;
		}
		s->inflight_reqs--;
		s->reqs.give(id);
	}
	return 0;
}

} // extern "C"

/* ============================================================== receiver */

namespace {

struct SubRecv {
	uint64_t dst = 0;
	uint64_t dst_len = 0;
	int32_t tag = 0;
	uint64_t recv_size = 0;
	int ncompls = 0;
	bool consumed = false;   /* an eager arrival has been matched to it */
	bool copy_posted = false;
	uint32_t eager_len = 0;
};

struct RecvReq {
	uint16_t msg_seq_num = 0;
	int num_recvs = 0;
	SubRecv recvs[OFI_AMD_WIRE_MAX_RECVS];
	int total_compls = 0;
	int ncompls = 0;
	uint64_t size = 0;
	bool completed = false;
	int subs_done = 0;       /* the "receive segments" child request */
	uint64_t subs_size = 0;

	void add_completion(uint64_t bytes) /* inc_req_completion, :487-510 */
	{
		size += bytes;
		if (++ncompls == total_compls) {
			completed = true;
		}
	}
	void sub_recv_done(uint64_t bytes) /* inc_recv_seg_completion, :530-572 */
	{
		subs_size += bytes;
		if (++subs_done == num_recvs) {
			add_completion(subs_size);
		}
	}
	bool all_consumed() const
	{
		for (int i = 0; i < num_recvs; i++) {
			if (!recvs[i].consumed) {
				return false;
			}
		}
		return true;
	}
};

struct Arrival {
	ofi_amd_eager_entry_t e;
	bool handled = false;
};

} // namespace

struct ofi_amd_recv_comm {
	ofi_amd_msgbuff_t *msgbuff = nullptr;
	Pool<RecvReq, OFI_AMD_MAX_REQUESTS> reqs;
	std::vector<Arrival> arrivals; /* sorted by (eager_seq, eager_offset), front first */
	std::deque<ofi_amd_eager_copy_item_t> copies;
	uint16_t last_eager_seq = 0;
	uint8_t last_eager_offset = 0;
	bool has_processed_eager = false;
	uint16_t eager_drain_recv_seq = OFI_AMD_RDMA_MSG_SEQ_NUM_START;
	uint16_t last_completed_seq = 0;
	uint16_t next_msg_seq_num = OFI_AMD_RDMA_MSG_SEQ_NUM_START;
	uint32_t inflight_reqs = 0;
	uint64_t n_ctrl_sent = 0;
	uint32_t num_rails = 0;
	bool flush_live[OFI_AMD_MAX_REQUESTS] = {}; /* flush requests share the in-flight limit */

	int match_arrivals();
	RecvReq *posted(uint16_t seq, int *stat);
};

/* The posted receive with this sequence number, if the message buffer holds one. */
RecvReq *ofi_amd_recv_comm::posted(uint16_t seq, int *stat)
{
	void *elem = nullptr;
	int type = 0;
	if (ofi_amd_msgbuff_retrieve(msgbuff, seq, &elem, &type, stat) != OFI_AMD_MSGBUFF_SUCCESS ||
	    type != OFI_AMD_MSGBUFF_REQ) {
		return nullptr;
	}
	*stat = OFI_AMD_MSGBUFF_INPROGRESS;
	return static_cast<RecvReq *>(elem);
}

/* drain_recv_eager_queue, src/nccl_ofi_rdma.cpp:791-892.  Arrivals are taken in chain order;
 * each looks for its receive from the sequence number its batch started at, stepping over
 * receives that are already complete and over receives with no free sub-receive of its tag.
 * One that finds no posted receive yet stays queued, and so does everything behind it, but
 * those behind it are still matched (and marked) where they can be. */
int ofi_amd_recv_comm::match_arrivals()
{
	bool skipping = false;
	uint16_t chain_seq = last_eager_seq;
	uint8_t chain_offset = last_eager_offset;
	bool chain_started = has_processed_eager;
	uint16_t fill_seq = eager_drain_recv_seq;
	size_t retired = 0;

	for (size_t k = 0; k < arrivals.size(); k++) {
		Arrival &a = arrivals[k];
		if (!ofi_amd_eager_entry_can_process(chain_started, chain_seq, chain_offset, &a.e)) {
			break;
		}
		chain_seq = a.e.eager_seq;
		chain_offset = a.e.eager_offset;
		chain_started = true;

		bool settled = a.handled;
		if (!settled) {
			if (a.e.eager_offset == 0) {
				fill_seq = a.e.msg_seq_num;
			}
			for (uint16_t seq = fill_seq;; seq = seq_next(seq)) {
				int stat = 0;
				RecvReq *req = posted(seq, &stat);
				if (!req) {
					if (stat == OFI_AMD_MSGBUFF_COMPLETED) {
						continue;
					}
					break; /* that receive has not been posted yet */
				}
				/* eager_match_recv, :727-737 */
				int sub = -1;
				for (int i = 0; i < req->num_recvs && sub < 0; i++) {
					if (!req->recvs[i].consumed && req->recvs[i].tag == a.e.tag) {
						sub = i;
					}
				}
				if (sub < 0) {
					continue;
				}
				SubRecv &sr = req->recvs[sub];
				sr.consumed = true;
				/* eager_copy_to_sub_recv, :745-780 */
				ofi_amd_eager_copy_item_t item = {};
				item.rx_cookie = a.e.cookie;
				item.dst = sr.dst;
				item.dst_len = sr.dst_len;
				item.recv_len = a.e.recv_len;
				item.req = static_cast<int32_t>(req - reqs.items);
				item.sub_idx = sub;
				item.needs_copy = a.e.recv_len != 0;
				if (a.e.recv_len == 0) {
					if (req->num_recvs > 1) {
						req->sub_recv_done(0);
					} else {
						req->add_completion(0);
					}
				} else {
					sr.copy_posted = true;
					/* the copy is cut to the receive buffer (rdma_eager_copy_req::post,
					 * src/nccl_ofi_rdma.cpp:2738-2743) and its completion counts the
					 * bytes copied (:2936-2937) */
					sr.eager_len = a.e.recv_len < sr.dst_len ? a.e.recv_len
										: static_cast<uint32_t>(sr.dst_len);
				}
				try {
					copies.push_back(item);
				} catch (...) {
					return -ENOMEM;
				}
				a.handled = true;
				if (req->all_consumed()) {
					fill_seq = seq_next(fill_seq);
				}
				settled = true;
				break;
			}
		}
		if (!settled) {
			skipping = true;
			continue;
		}
		if (!skipping) {
			retired = k + 1;
			last_eager_seq = a.e.eager_seq;
			last_eager_offset = a.e.eager_offset;
			has_processed_eager = true;
			eager_drain_recv_seq = fill_seq;
		}
	}
	arrivals.erase(arrivals.begin(), arrivals.begin() + static_cast<ptrdiff_t>(retired));
	return 0;
}

extern "C" {

int ofi_amd_recv_comm_create(uint32_t num_rails, ofi_amd_recv_comm_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS) {
		return -EINVAL;
	}
	ofi_amd_recv_comm_t *r = new (std::nothrow) ofi_amd_recv_comm();
	if (!r) {
		return -ENOMEM;
	}
	/* src/nccl_ofi_rdma.cpp:4917 */
	const int rc = ofi_amd_msgbuff_create(OFI_AMD_RDMA_MSGBUFF_SIZE, OFI_AMD_RDMA_SEQ_BITS,
					      OFI_AMD_RDMA_MSG_SEQ_NUM_START, &r->msgbuff);
	if (rc != 0) {
		delete r;
		return rc;
	}
	try {
		r->arrivals.reserve(OFI_AMD_CTRL_MAILBOX_SIZE);
	} catch (...) {
		ofi_amd_msgbuff_destroy(r->msgbuff);
		delete r;
		return -ENOMEM;
	}
	r->num_rails = num_rails;
	*out = r;
	return 0;
}

int ofi_amd_recv_comm_destroy(ofi_amd_recv_comm_t *r)
{
	if (!r) {
		return -EINVAL;
	}
	ofi_amd_msgbuff_destroy(r->msgbuff);
	delete r;
	return 0;
}

/* recv, :3545-3745 */
int ofi_amd_recv_comm_recv(ofi_amd_recv_comm_t *r, int n, const uint64_t *dsts, const uint64_t *sizes,
			   const int *tags, const uint64_t *mr_keys, int completion_optional,
			   ofi_amd_ctrl_msg_t *mailbox, int32_t *req_out, uint16_t *seq_out)
{
	if (!r || !dsts || !sizes || !tags || !mr_keys || !mailbox || !req_out || !seq_out || n < 1 ||
	    n > OFI_AMD_WIRE_MAX_RECVS) {
		return -EINVAL;
	}
	*req_out = -1;
	if (r->inflight_reqs == OFI_AMD_MAX_REQUESTS) {
		return -ENOSPC;
	}
	const uint16_t seq = r->next_msg_seq_num;
	int stat = 0;
	if (r->posted(seq, &stat) || stat != OFI_AMD_MSGBUFF_NOTSTARTED) {
		return -EINVAL; /* a request is already there, or the number is out of the window */
	}
	const int id = r->reqs.take();
	if (id < 0) {
		return -EINVAL;
	}
	RecvReq &req = r->reqs.items[id];
	req.msg_seq_num = seq;
	req.total_compls = completion_optional ? 1 : 2; /* control message sent [+ data arrived] */
	req.num_recvs = n;
	uint32_t lens[OFI_AMD_WIRE_MAX_RECVS];
	for (int i = 0; i < n; i++) {
		req.recvs[i].dst = dsts[i];
		req.recvs[i].dst_len = sizes[i];
		req.recvs[i].tag = tags[i];
		lens[i] = static_cast<uint32_t>(sizes[i]);
	}
	int rc = ofi_amd_ctrl_msg_fill(mailbox, seq, static_cast<uint16_t>(n), dsts, lens, tags, mr_keys,
				       r->num_rails, completion_optional);
	if (rc == 0 && ofi_amd_msgbuff_insert(r->msgbuff, seq, &req, OFI_AMD_MSGBUFF_REQ, &stat) !=
			       OFI_AMD_MSGBUFF_SUCCESS) {
		rc = -EINVAL;
	}
	if (rc != 0) {
		r->reqs.give(id);
		return rc;
	}
	r->inflight_reqs++;
	r->n_ctrl_sent++;
	*req_out = id;
	*seq_out = seq;
	r->next_msg_seq_num = seq_next(seq);
	/* a new receive may be what queued eager arrivals were waiting for */
	return r->arrivals.empty() ? 0 : r->match_arrivals();
}

/* handle_eager_recv, :897-947 */
int ofi_amd_recv_comm_eager_arrival(ofi_amd_recv_comm_t *r, uint16_t msg_seq_num,
				    const ofi_amd_eager_hdr_t *hdr, uint32_t recv_len, uint64_t rx_cookie)
{
	if (!r || !hdr) {
		return -EINVAL;
	}
	if (r->arrivals.size() >= OFI_AMD_CTRL_MAILBOX_SIZE) {
		return -ENOMEM;
	}
	Arrival a;
	a.e.eager_offset = hdr->eager_offset;
	a.e.prev_batch_count = hdr->prev_batch_count;
	a.e.eager_seq = hdr->eager_seq;
	a.e.msg_seq_num = msg_seq_num;
	a.e.pad = 0;
	a.e.tag = hdr->tag;
	a.e.recv_len = recv_len;
	a.e.cookie = rx_cookie;
	/* recv_eager_sorted_insert, include/nccl_ofi_rdma.h:734-750: behind every entry not greater */
	size_t pos = r->arrivals.size();
	while (pos > 0 && ofi_amd_eager_entry_less(&a.e, &r->arrivals[pos - 1].e)) {
		pos--;
	}
	r->arrivals.insert(r->arrivals.begin() + static_cast<ptrdiff_t>(pos), a);
	return r->match_arrivals();
}

/* handle_write_comp, :1102-1130 */
int ofi_amd_recv_comm_write_arrival(ofi_amd_recv_comm_t *r, uint32_t imm, uint64_t len)
{
	if (!r) {
		return -EINVAL;
	}
	uint32_t seq = 0, recv_idx = 0, nseg = 0;
	ofi_amd_rdma_imm_decode(imm, nullptr, &seq, &recv_idx, &nseg);
	int stat = 0;
	RecvReq *req = r->posted(static_cast<uint16_t>(seq), &stat);
	if (!req) {
		return -EINVAL; /* no receive in flight under that number */
	}
	SubRecv &sr = req->recvs[recv_idx];
	sr.recv_size += len;
	if (++sr.ncompls == static_cast<int>(nseg)) {
		req->sub_recv_done(sr.recv_size);
	}
	return 0;
}

int ofi_amd_recv_comm_ctrl_sent(ofi_amd_recv_comm_t *r, int32_t id)
{
	if (!r || !r->reqs.valid(id)) {
		return -EINVAL;
	}
	r->reqs.items[id].add_completion(0);
	return 0;
}

uint32_t ofi_amd_recv_comm_take_copies(ofi_amd_recv_comm_t *r, ofi_amd_eager_copy_item_t *out,
				       uint32_t cap)
{
	if (!r || !out) {
		return 0;
	}
	uint32_t n = 0;
	while (n < cap && !r->copies.empty()) {
		out[n++] = r->copies.front();
		r->copies.pop_front();
	}
	return n;
}

/* rdma_eager_copy_req::handle_completion, :2920-2957 */
int ofi_amd_recv_comm_copy_done(ofi_amd_recv_comm_t *r, int32_t id, int32_t sub_idx)
{
	if (!r || !r->reqs.valid(id) || sub_idx < 0 || sub_idx >= r->reqs.items[id].num_recvs ||
	    !r->reqs.items[id].recvs[sub_idx].copy_posted) {
		return -EINVAL;
	}
	RecvReq &req = r->reqs.items[id];
	SubRecv &sr = req.recvs[sub_idx];
	sr.copy_posted = false;
	sr.recv_size += sr.eager_len;
	if (req.num_recvs > 1) {
		req.sub_recv_done(sr.eager_len);
	} else {
		req.add_completion(sr.eager_len);
	}
	return 0;
}

/* nccl_net_ofi_rdma_req::test for a receive, :2236-2307; sizes as write_completion_size
 * :2340-2353; the message buffer entry retires as in rdma_recv_req::free :1677-1695 */
int ofi_amd_recv_comm_test(ofi_amd_recv_comm_t *r, int32_t id, int *done, int *sizes)
{
	if (!r || !done || !r->reqs.valid(id)) {
		return -EINVAL;
	}
	*done = 0;
	RecvReq &req = r->reqs.items[id];
	if (!req.completed) {
		return 0;
	}
	if (sizes) {
		if (req.num_recvs > 1) {
			for (int i = 0; i < req.num_recvs; i++) {
				sizes[i] = static_cast<int>(req.recvs[i].recv_size);
			}
		} else {
			sizes[0] = static_cast<int>(req.size);
		}
	}
	int stat = 0;
	if (ofi_amd_msgbuff_complete(r->msgbuff, req.msg_seq_num, &stat) != OFI_AMD_MSGBUFF_SUCCESS) {
		return -EINVAL;
	}
	*done = 1;
	r->last_completed_seq = req.msg_seq_num;
	r->inflight_reqs--;
	r->reqs.give(id);
	return 0;
}

/* flush, src/nccl_ofi_rdma.cpp:4405-4510: one flush covers every buffer of the call, and a
 * call whose receives were all empty needs none */
int ofi_amd_recv_comm_flush(ofi_amd_recv_comm_t *r, int n, const int *sizes, int32_t *req)
{
	if (!r || !sizes || !req || n < 1 || n > OFI_AMD_WIRE_MAX_RECVS) {
		return -EINVAL;
	}
	*req = -1;
	if (r->inflight_reqs == OFI_AMD_MAX_REQUESTS) {
		return -ENOSPC;
	}
	bool any = false;
	for (int i = 0; i < n; i++) {
		any = any || sizes[i] != 0;
	}
	if (!any) {
		return 0;
	}
	for (int32_t id = 0; id < OFI_AMD_MAX_REQUESTS; id++) {
		if (!r->flush_live[id]) {
			r->flush_live[id] = true;
			r->inflight_reqs++;
			*req = id;
			return 0;
		}
	}
	return -ENOSPC;
}

/* test() of a flush request: has_flush_completed, :2110-2126 */
int ofi_amd_recv_comm_flush_test(ofi_amd_recv_comm_t *r, int32_t req, const void *slots_host,
				 uint32_t num_rails, uint64_t sentinel, int *done)
{
	if (!r || !done || req < 0 || req >= OFI_AMD_MAX_REQUESTS || !r->flush_live[req] || !slots_host ||
	    num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS) {
		return -EINVAL;
	}
	*done = ofi_amd_flush_test(slots_host, num_rails, sentinel) == 1;
	if (*done) {
		r->flush_live[req] = false;
		r->inflight_reqs--;
	}
	return 0;
}

void ofi_amd_recv_comm_state(const ofi_amd_recv_comm_t *r, ofi_amd_recv_state_t *out)
{
	if (!r || !out) {
		return;
	}
	std::memset(out, 0, sizeof(*out));
	out->next_msg_seq_num = r->next_msg_seq_num;
	out->eager_drain_recv_seq = r->eager_drain_recv_seq;
	out->last_eager_seq = r->last_eager_seq;
	out->last_completed_seq = r->last_completed_seq;
	out->last_eager_offset = r->last_eager_offset;
	out->has_processed_eager = r->has_processed_eager ? 1 : 0;
	out->num_inflight_reqs = r->inflight_reqs;
	out->eager_pending = static_cast<uint32_t>(r->arrivals.size());
	out->n_ctrl_sent = r->n_ctrl_sent;
}

} // extern "C"

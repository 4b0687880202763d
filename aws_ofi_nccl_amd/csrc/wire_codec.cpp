/*
 * RDMA-protocol wire formats and ordering rules on the host (include/ofi_amd_wire.h).
 * Bit layouts and decision rules are the reference's; each function cites its source.
 * The receiver's eager queue keeps its (at most a few dozen) arrivals in a sorted vector
 * instead of the reference's intrusive list: same order, same hand-out rule.
 */
#include <atomic>
#include <cerrno>
#include <cstring>
#include <new>
#include <vector>

#include "ofi_amd_hotpath.h"
#include "ofi_amd_wire.h"

namespace {

constexpr uint32_t kSeqMask = (1u << OFI_AMD_RDMA_SEQ_BITS) - 1;
constexpr uint32_t kCommMask = (1u << OFI_AMD_RDMA_COMM_ID_BITS) - 1;
constexpr uint32_t kRecvIdxMask = (1u << OFI_AMD_RDMA_RECV_IDX_BITS) - 1;
constexpr uint32_t kNumSegMask = (1u << OFI_AMD_RDMA_NUM_SEG_BITS) - 1;
constexpr uint32_t kCommShift = OFI_AMD_RDMA_SEQ_BITS;
constexpr uint32_t kRecvIdxShift = kCommShift + OFI_AMD_RDMA_COMM_ID_BITS;
constexpr uint32_t kNumSegShift = kRecvIdxShift + OFI_AMD_RDMA_RECV_IDX_BITS;
static_assert(kNumSegShift + OFI_AMD_RDMA_NUM_SEG_BITS == 32, "immediate data is 32 bits");

inline uint16_t read_once(const uint16_t &v)
{
	return reinterpret_cast<const std::atomic<uint16_t> &>(v).load(std::memory_order_relaxed);
}

} // namespace

struct ofi_amd_eager_rxq {
	std::vector<ofi_amd_eager_entry_t> entries; /* sorted, front first */
	bool has_processed = false;
	uint16_t last_eager_seq = 0;
	uint8_t last_offset = 0;
};

extern "C" {

/* GET_RDMA_WRITE_IMM_DATA, src/nccl_ofi_rdma.cpp:98-101 */
uint32_t ofi_amd_rdma_imm(uint32_t comm_id, uint32_t seq, uint32_t recv_idx, uint32_t nseg)
{
	return seq | (comm_id << kCommShift) | (recv_idx << kRecvIdxShift) | (nseg << kNumSegShift);
}

/* GET_COMM_ID_FROM_IMM .. GET_RECV_IDX_FROM_IMM, :73-93 */
void ofi_amd_rdma_imm_decode(uint32_t imm, uint32_t *comm_id, uint32_t *seq, uint32_t *recv_idx,
			     uint32_t *nseg)
{
	if (comm_id) {
		*comm_id = (imm >> kCommShift) & kCommMask;
	}
	if (seq) {
		*seq = imm & kSeqMask;
	}
	if (recv_idx) {
		*recv_idx = (imm >> kRecvIdxShift) & kRecvIdxMask;
	}
	if (nseg) {
		*nseg = (imm >> kNumSegShift) & kNumSegMask;
	}
}

uint32_t ofi_amd_ctrl_mailbox_slot(uint16_t msg_seq_num)
{
	return msg_seq_num % OFI_AMD_CTRL_MAILBOX_SIZE;
}

/* nccl_net_ofi_rdma_recv_comm::allocate_recv_req, mailbox update, src/nccl_ofi_rdma.cpp:3446-3474 */
int ofi_amd_ctrl_msg_fill(ofi_amd_ctrl_msg_t *mailbox, uint16_t msg_seq_num, uint16_t num_recvs,
			  const uint64_t *buff_offsets, const uint32_t *sizes, const int *tags,
			  const uint64_t *mr_keys, uint32_t num_rails, int recv_completion_optional)
{
	if (!mailbox || !buff_offsets || !sizes || !tags || !mr_keys || num_recvs < 1 ||
	    num_recvs > OFI_AMD_WIRE_MAX_RECVS || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS) {
		return -EINVAL;
	}
	ofi_amd_ctrl_msg_t &slot = mailbox[ofi_amd_ctrl_mailbox_slot(msg_seq_num)];
	std::memset(&slot, 0, sizeof(slot));
	slot.entries[0].num_recvs = num_recvs;
	slot.entries[0].flags = recv_completion_optional ? OFI_AMD_CTRL_FLAG_RECV_COMPLETION_OPT : 0;
	const uint16_t ready = msg_seq_num & kSeqMask;
	for (uint16_t i = 0; i < num_recvs; i++) {
		ofi_amd_ctrl_entry_t &e = slot.entries[i];
		e.buff_offset = buff_offsets[i];
		e.buff_len = sizes[i];
		e.tag = static_cast<int16_t>(tags[i]);
		e.recv_idx = static_cast<uint8_t>(i);
		for (uint32_t r = 0; r < num_rails; r++) {
			e.mr_key[r] = mr_keys[(size_t)i * num_rails + r];
		}
	}
	/* the ready bits go last: a reader that sees them sees the rest */
	std::atomic_thread_fence(std::memory_order_release);
	for (uint16_t i = 0; i < num_recvs; i++) {
		reinterpret_cast<std::atomic<uint16_t> &>(slot.entries[i].msg_seq_num)
			.store(ready, std::memory_order_relaxed);
	}
	return 0;
}

/* has_ctrl_msg, :2134-2178 */
int ofi_amd_ctrl_msg_ready(const ofi_amd_ctrl_msg_t *mailbox, uint16_t seq_num, int tag,
			   int ignore_tag_match)
{
	if (!mailbox) {
		return 0;
	}
	const ofi_amd_ctrl_msg_t &ctrl = mailbox[ofi_amd_ctrl_mailbox_slot(seq_num)];
	const uint16_t expected = seq_num & kSeqMask;
	/* entries[0] carries num_recvs: validate it before trusting the loop bound */
	if (read_once(ctrl.entries[0].msg_seq_num) != expected) {
		return 0;
	}
	std::atomic_thread_fence(std::memory_order_acquire);
	const uint16_t num_recvs = read_once(ctrl.entries[0].num_recvs);
	if (num_recvs > OFI_AMD_WIRE_MAX_RECVS) {
		return 0;
	}
	for (uint16_t i = 1; i < num_recvs; i++) {
		if (read_once(ctrl.entries[i].msg_seq_num) != expected) {
			return 0;
		}
	}
	std::atomic_thread_fence(std::memory_order_acquire);
	if (ignore_tag_match) {
		return 1;
	}
	for (uint16_t i = 0; i < num_recvs; i++) {
		if (ctrl.entries[i].entry_used != 1 && ctrl.entries[i].tag == tag) {
			return 1;
		}
	}
	return 0;
}

int ofi_amd_ctrl_msg_find_tag(const ofi_amd_ctrl_msg_t *msg, int tag)
{
	if (!msg) {
		return -1;
	}
	const uint16_t n = msg->entries[0].num_recvs < OFI_AMD_WIRE_MAX_RECVS ? msg->entries[0].num_recvs
									       : OFI_AMD_WIRE_MAX_RECVS;
	for (uint16_t i = 0; i < n; i++) {
		if (msg->entries[i].tag == tag) {
			return i;
		}
	}
	return -1;
}

/* seq_before, include/nccl_ofi_rdma.h:670-673 */
int ofi_amd_seq_before(uint16_t a, uint16_t b)
{
	return ((uint32_t)(a - b) & kSeqMask) > (kSeqMask >> 1);
}

/* eager_seq_before, :678-681 */
int ofi_amd_eager_seq_before(uint16_t a, uint16_t b)
{
	return static_cast<int16_t>(static_cast<uint16_t>(a - b)) < 0;
}

/* eager_entry_less, :683-689 */
int ofi_amd_eager_entry_less(const ofi_amd_eager_entry_t *a, const ofi_amd_eager_entry_t *b)
{
	if (a->eager_seq != b->eager_seq) {
		return ofi_amd_eager_seq_before(a->eager_seq, b->eager_seq);
	}
	return a->eager_offset < b->eager_offset;
}

/* eager_entry_can_process, :709-732 */
int ofi_amd_eager_entry_can_process(int has_processed, uint16_t last_eager_seq, uint8_t last_offset,
				    const ofi_amd_eager_entry_t *entry)
{
	if (!has_processed) {
		/* first batch on the comm */
		return entry->eager_offset == 0 && entry->eager_seq == 0;
	}
	if (entry->eager_offset == 0) {
		/* a new batch: next eager_seq, and the previous batch was seen to its end */
		return entry->eager_seq == static_cast<uint16_t>(last_eager_seq + 1) &&
		       static_cast<int>(last_offset) == static_cast<int>(entry->prev_batch_count) - 1;
	}
	/* continuation of the open batch */
	return entry->eager_seq == last_eager_seq &&
	       static_cast<int>(last_offset) == static_cast<int>(entry->eager_offset) - 1;
}

int ofi_amd_eager_rxq_create(ofi_amd_eager_rxq_t **out)
{
	if (!out) {
		return -EINVAL;
	}
	*out = new (std::nothrow) ofi_amd_eager_rxq();
	return *out ? 0 : -ENOMEM;
}

int ofi_amd_eager_rxq_destroy(ofi_amd_eager_rxq_t *q)
{
	if (!q) {
		return -EINVAL;
	}
	delete q;
	return 0;
}

/* recv_eager_sorted_insert, :734-750: behind every entry that is not greater */
int ofi_amd_eager_rxq_insert(ofi_amd_eager_rxq_t *q, const ofi_amd_eager_entry_t *e)
{
	if (!q || !e) {
		return -EINVAL;
	}
	try {
		size_t pos = q->entries.size();
		while (pos > 0 && ofi_amd_eager_entry_less(e, &q->entries[pos - 1])) {
			pos--;
		}
		q->entries.insert(q->entries.begin() + pos, *e);
	} catch (...) {
		return -ENOMEM;
	}
	return 0;
}

/* ordering half of drain_recv_eager_queue, src/nccl_ofi_rdma.cpp:797-816, 878-886 */
uint32_t ofi_amd_eager_rxq_drain(ofi_amd_eager_rxq_t *q, ofi_amd_eager_entry_t *out, uint32_t cap)
{
	if (!q || !out) {
		return 0;
	}
	uint32_t n = 0;
	while (n < cap && n < q->entries.size()) {
		const ofi_amd_eager_entry_t &front = q->entries[n];
		if (!ofi_amd_eager_entry_can_process(q->has_processed, q->last_eager_seq, q->last_offset,
						     &front)) {
			break;
		}
		q->has_processed = true;
		q->last_eager_seq = front.eager_seq;
		q->last_offset = front.eager_offset;
		out[n++] = front;
	}
	q->entries.erase(q->entries.begin(), q->entries.begin() + n);
	return n;
}

uint32_t ofi_amd_eager_rxq_pending(const ofi_amd_eager_rxq_t *q)
{
	return q ? static_cast<uint32_t>(q->entries.size()) : 0;
}

uint32_t ofi_amd_eager_rxq_peek(const ofi_amd_eager_rxq_t *q, ofi_amd_eager_entry_t *out, uint32_t cap)
{
	if (!q || !out) {
		return 0;
	}
	const uint32_t n = q->entries.size() < cap ? static_cast<uint32_t>(q->entries.size()) : cap;
	std::memcpy(out, q->entries.data(), n * sizeof(*out));
	return n;
}

void ofi_amd_eager_tx_init(ofi_amd_eager_tx_t *tx)
{
	std::memset(tx, 0, sizeof(*tx));
}

/* nccl_net_ofi_rdma_send_comm::send, src/nccl_ofi_rdma.cpp:5783-5806 */
void ofi_amd_eager_tx_assign(ofi_amd_eager_tx_t *tx, int32_t tag, ofi_amd_eager_hdr_t *hdr)
{
	if (tx->eager_offset_next == 0) {
		/* a batch starts: it takes the next eager sequence number (wraps at 2^16) */
		tx->cur_eager_seq = tx->eager_seq_next++;
	}
	hdr->eager_offset = tx->eager_offset_next++;
	hdr->prev_batch_count = tx->prev_eager_batch_count;
	hdr->eager_seq = tx->cur_eager_seq;
	hdr->tag = tag;
}

/* drain_sender_eager_queue, :5594-5598 and :5636-5640 */
void ofi_amd_eager_tx_advance(ofi_amd_eager_tx_t *tx)
{
	if (tx->eager_offset_next > 0) {
		tx->prev_eager_batch_count = tx->eager_offset_next;
		tx->eager_offset_next = 0;
	}
}

/* :5758-5764 */
int ofi_amd_eager_fits(uint64_t size, int64_t eager_send_size)
{
	return static_cast<int64_t>(size + OFI_AMD_EAGER_HEADER_SIZE) <= eager_send_size;
}

/* has_flush_completed, src/nccl_ofi_rdma.cpp:2110-2126: one 64-byte slot per rail, only the
 * first 8 bytes of a slot count (declared in ofi_amd_hotpath.h beside the flush kernels) */
int ofi_amd_flush_test(const void *slots_host, uint32_t num_rails, uint64_t sentinel)
{
	if (!slots_host || num_rails < 1 || num_rails > OFI_AMD_WIRE_MAX_RAILS) {
		return -EINVAL;
	}
	const uint64_t *slots = static_cast<const uint64_t *>(slots_host);
	for (uint32_t r = 0; r < num_rails; r++) {
		if (__atomic_load_n(&slots[r * 8u], __ATOMIC_ACQUIRE) != sentinel) {
			return 0;
		}
	}
	return 1;
}

} /* extern "C" */

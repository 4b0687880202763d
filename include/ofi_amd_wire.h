/*
 * Wire formats and ordering rules of the RDMA protocol either side of the eager / bounce
 * copy.  The layouts are the reference's, bit for bit, so that a peer running the reference
 * plugin interoperates; each item cites the definition it mirrors.  Host-only code: nothing
 * here needs a GPU.
 */
#ifndef OFI_AMD_WIRE_H_
#define OFI_AMD_WIRE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OFI_AMD_WIRE_MAX_RAILS 4          /* MAX_NUM_RAILS, include/nccl_ofi_rdma.h:37 */
#define OFI_AMD_WIRE_MAX_RECVS 8          /* NCCL_OFI_MAX_RECVS, include/nccl_ofi.h:54 */
#define OFI_AMD_WIRE_MAX_EP_ADDR 56       /* MAX_EP_ADDR, include/nccl_ofi.h:38 */
#define OFI_AMD_CTRL_MAILBOX_SIZE 256     /* 2 * NCCL_OFI_MAX_REQUESTS, include/nccl_ofi_rdma.h:311 */
#define OFI_AMD_EAGER_HEADER_SIZE 8       /* include/nccl_ofi_rdma.h:209 */
#define OFI_AMD_EAGER_RX_ALIGNMENT 128    /* EAGER_RX_BUFFER_ALIGNMENT, include/nccl_ofi_rdma.h:336 */
#define OFI_AMD_MAX_EAGER_PENDING 32      /* NCCL_NET_MAX_REQUESTS, nccl/net.h:32 */
#define OFI_AMD_RDMA_SEQ_BITS 10          /* include/nccl_ofi_rdma.h:83 */
#define OFI_AMD_RDMA_COMM_ID_BITS 15      /* :50 */
#define OFI_AMD_RDMA_RECV_IDX_BITS 3      /* :55 */
#define OFI_AMD_RDMA_NUM_SEG_BITS 4
#define OFI_AMD_RDMA_MSG_SEQ_NUM_START 1  /* :66 */
#define OFI_AMD_CTRL_FLAG_RECV_COMPLETION_OPT 1u /* :200 */
#define OFI_AMD_RDMA_FLUSH_SENTINEL 0x00000000ffffffffull /* :45 and src/nccl_ofi_rdma.cpp:7390-7394 */
#define OFI_AMD_GIN_FLUSH_SENTINEL 0xdeadbeefdeadbeefull  /* include/rdma/gin/nccl_ofi_gin_reqs.h:274 */

/* ---- RDMA write immediate data (src/nccl_ofi_rdma.cpp:73-103) ----
 * | 4-bit segment count | 3-bit recv_idx | 15-bit comm id | 10-bit msg_seq_num | */
uint32_t ofi_amd_rdma_imm(uint32_t comm_id, uint32_t seq, uint32_t recv_idx, uint32_t nseg);
void ofi_amd_rdma_imm_decode(uint32_t imm, uint32_t *comm_id, uint32_t *seq, uint32_t *recv_idx,
			     uint32_t *nseg);

/* ---- eager header (nccl_ofi_eager_msg_header_t, include/nccl_ofi_rdma.h:217-228) ---- */
typedef struct {
	uint8_t eager_offset;
	uint8_t prev_batch_count; /* meaningful when eager_offset == 0 */
	uint16_t eager_seq;
	int32_t tag;
} ofi_amd_eager_hdr_t;

/* ---- control message (nccl_net_ofi_ctrl_msg_entry_t / _ctrl_msg_t, :235-290) ---- */
typedef struct {
	uint64_t buff_offset;
	uint64_t mr_key[OFI_AMD_WIRE_MAX_RAILS];
	uint32_t buff_len;
	int16_t tag;
	uint16_t flags;     /* entries[0] only */
	uint16_t num_recvs; /* entries[0] only */
	uint8_t recv_idx;
	uint8_t entry_used;
	uint8_t pad[10];
	uint16_t msg_seq_num; /* written last: the ready bit */
} ofi_amd_ctrl_entry_t;

typedef struct {
	ofi_amd_ctrl_entry_t entries[OFI_AMD_WIRE_MAX_RECVS];
} ofi_amd_ctrl_msg_t;

/* ---- close message (nccl_net_ofi_rdma_close_msg_t, :314-323) ---- */
typedef struct {
	uint16_t type : 4;
	uint64_t ctrl_counter;
	uint32_t send_comm_id;
} ofi_amd_close_msg_t;

/* ---- connect message (nccl_ofi_rdma_connection_info_t, :1116-1149): 560 bytes ---- */
typedef struct {
	char ep_name[OFI_AMD_WIRE_MAX_EP_ADDR];
	size_t ep_name_len;
} ofi_amd_ep_name_t;

typedef struct {
	uint16_t num_rails;
	uint16_t num_control_rails;
	uint32_t comm_id;
	ofi_amd_ep_name_t control_ep_names[OFI_AMD_WIRE_MAX_RAILS];
	ofi_amd_ep_name_t ep_names[OFI_AMD_WIRE_MAX_RAILS];
	uint64_t ctrl_addr;
	uint64_t ctrl_mr_key[OFI_AMD_WIRE_MAX_RAILS];
} ofi_amd_connection_info_t;

/* ---- flush slot (nccl_net_ofi_flush_data_t, :326-332): one cache line per rail ---- */
typedef struct {
	uint64_t flag;
	char padding[56];
} ofi_amd_flush_data_t;

#ifdef __cplusplus
static_assert(sizeof(ofi_amd_eager_hdr_t) == OFI_AMD_EAGER_HEADER_SIZE, "eager header is 8 bytes");
static_assert(sizeof(ofi_amd_ctrl_entry_t) == 64, "control entry is one cache line");
static_assert(sizeof(ofi_amd_ctrl_msg_t) == 64 * OFI_AMD_WIRE_MAX_RECVS, "control message size");
static_assert(sizeof(ofi_amd_connection_info_t) == 560, "connect message size");
static_assert(sizeof(ofi_amd_flush_data_t) == 64, "flush slot size");
#endif

/* Slot of a message in the control mailbox: seq % 256 (src/nccl_ofi_rdma.cpp:3447). */
uint32_t ofi_amd_ctrl_mailbox_slot(uint16_t msg_seq_num);

/*
 * Receiver side: zero the mailbox slot and describe a (grouped) receive in it, the ready bit
 * of every entry last (src/nccl_ofi_rdma.cpp:3446-3474).  mr_keys is [num_recvs][num_rails].
 * -EINVAL for num_recvs outside 1..8 or num_rails outside 1..4.
 */
int ofi_amd_ctrl_msg_fill(ofi_amd_ctrl_msg_t *mailbox, uint16_t msg_seq_num, uint16_t num_recvs,
			  const uint64_t *buff_offsets, const uint32_t *sizes, const int *tags,
			  const uint64_t *mr_keys, uint32_t num_rails, int recv_completion_optional);

/*
 * Sender side: has the control message for seq_num arrived, and (unless ignore_tag_match)
 * does it hold an unused entry for `tag`?  has_ctrl_msg, src/nccl_ofi_rdma.cpp:2134-2178.
 */
int ofi_amd_ctrl_msg_ready(const ofi_amd_ctrl_msg_t *mailbox, uint16_t seq_num, int tag,
			   int ignore_tag_match);

/* Index of the first entry below entries[0].num_recvs carrying `tag`, or -1
 * (the search of get_ctrl_msg_buff_len / update_send_data_from_remote as
 * tests/unit/ctrl_msg.cpp:27-34 restates it). */
int ofi_amd_ctrl_msg_find_tag(const ofi_amd_ctrl_msg_t *msg, int tag);

/* ---- ordering of sequence numbers (include/nccl_ofi_rdma.h:670-683) ---- */
int ofi_amd_seq_before(uint16_t a, uint16_t b);       /* 10-bit message sequence */
int ofi_amd_eager_seq_before(uint16_t a, uint16_t b); /* 16-bit eager batch sequence */

/* Receiver's record of one eager arrival (nccl_ofi_recv_eager_entry_t, :650-663, the fields
 * the ordering uses; `cookie` stands for the rx buffer request). */
typedef struct {
	uint8_t eager_offset;
	uint8_t prev_batch_count;
	uint16_t eager_seq;
	uint16_t msg_seq_num;
	uint16_t pad;
	int32_t tag;
	uint32_t recv_len;
	uint64_t cookie;
} ofi_amd_eager_entry_t;

int ofi_amd_eager_entry_less(const ofi_amd_eager_entry_t *a, const ofi_amd_eager_entry_t *b); /* :685-691 */
int ofi_amd_eager_entry_can_process(int has_processed, uint16_t last_eager_seq, uint8_t last_offset,
				    const ofi_amd_eager_entry_t *entry); /* :709-732 */

/*
 * Receiver's ordered eager queue: arrivals are kept sorted by (eager_seq, eager_offset)
 * (recv_eager_sorted_insert, :734-750) and handed out strictly along the batch chain
 * (the ordering half of drain_recv_eager_queue, src/nccl_ofi_rdma.cpp:791-892; matching
 * against posted receives stays with the caller).
 */
typedef struct ofi_amd_eager_rxq ofi_amd_eager_rxq_t;
int ofi_amd_eager_rxq_create(ofi_amd_eager_rxq_t **out);
int ofi_amd_eager_rxq_destroy(ofi_amd_eager_rxq_t *q);
int ofi_amd_eager_rxq_insert(ofi_amd_eager_rxq_t *q, const ofi_amd_eager_entry_t *e);
/* Pops the entries that are next in the chain (at most cap); returns how many. */
uint32_t ofi_amd_eager_rxq_drain(ofi_amd_eager_rxq_t *q, ofi_amd_eager_entry_t *out, uint32_t cap);
uint32_t ofi_amd_eager_rxq_pending(const ofi_amd_eager_rxq_t *q);
/* The queue as it stands, front to back (for inspection). */
uint32_t ofi_amd_eager_rxq_peek(const ofi_amd_eager_rxq_t *q, ofi_amd_eager_entry_t *out, uint32_t cap);

/* Sender's eager batch numbering (nccl_net_ofi_rdma_send_comm::send,
 * src/nccl_ofi_rdma.cpp:5783-5806, and the reset on msg_seq_num advance, :5594-5598). */
typedef struct {
	uint16_t eager_seq_next;
	uint16_t cur_eager_seq;
	uint8_t eager_offset_next;
	uint8_t prev_eager_batch_count;
	uint16_t pad;
} ofi_amd_eager_tx_t;
void ofi_amd_eager_tx_init(ofi_amd_eager_tx_t *tx);
/* Header of the next eager send. */
void ofi_amd_eager_tx_assign(ofi_amd_eager_tx_t *tx, int32_t tag, ofi_amd_eager_hdr_t *hdr);
/* The sender's msg_seq_num moved on: the open batch, if any, is closed. */
void ofi_amd_eager_tx_advance(ofi_amd_eager_tx_t *tx);

/* An eager send is possible for this payload size (size + 8 <= eager_send_size,
 * src/nccl_ofi_rdma.cpp:5758-5764). */
int ofi_amd_eager_fits(uint64_t size, int64_t eager_send_size);

#ifdef __cplusplus
}
#endif
#endif /* OFI_AMD_WIRE_H_ */

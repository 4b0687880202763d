/*
 * Send/receive protocol of the RDMA transport as transport-free state machines: what the
 * plugin decides around a message -- eager or rendezvous, which control-mailbox entry a send
 * consumes, which posted receive an eager arrival belongs to, when a request is complete --
 * with everything the reference would hand to libfabric returned to the caller as an action.
 * A caller with a fabric underneath posts the actions; a caller without one (one process, one
 * GPU) executes them as device copies.  The eager copies the receiver decides on come out as
 * work items for ofi_amd_eager_copy_batch, many per launch instead of one loop-back read each.
 *
 * Host-only code: nothing here needs a GPU.  A comm is driven by one thread at a time, as the
 * reference's are under the endpoint lock.
 */
#ifndef OFI_AMD_SENDRECV_H_
#define OFI_AMD_SENDRECV_H_

#include <stddef.h>
#include <stdint.h>

#include "ofi_amd_hotpath.h"
#include "ofi_amd_wire.h"

#ifdef __cplusplus
extern "C" {
#endif

#define OFI_AMD_MAX_REQUESTS 128       /* NCCL_OFI_MAX_REQUESTS, include/nccl_ofi.h:62 */
#define OFI_AMD_MAX_SEND_REQUESTS 1024 /* NCCL_OFI_MAX_SEND_REQUESTS, include/nccl_ofi.h:71 */
#define OFI_AMD_RDMA_MSGBUFF_SIZE 256  /* NCCL_OFI_RDMA_MSGBUFF_SIZE, src/nccl_ofi_rdma.cpp:41 */

/* ======================================================================
 * Message buffer: in-flight messages by wrapping sequence number.
 *   Replaces class nccl_ofi_msgbuff, include/nccl_ofi_msgbuff.h:84-166,
 *   src/nccl_ofi_msgbuff.cpp:14-166.  Status, result and element-type codes are the
 *   reference's enums (include/nccl_ofi_msgbuff.h:42-69).
 * ====================================================================== */
#define OFI_AMD_MSGBUFF_COMPLETED 0
#define OFI_AMD_MSGBUFF_INPROGRESS 1
#define OFI_AMD_MSGBUFF_NOTSTARTED 2
#define OFI_AMD_MSGBUFF_UNAVAILABLE 3

#define OFI_AMD_MSGBUFF_SUCCESS 0
#define OFI_AMD_MSGBUFF_INVALID_IDX 1
#define OFI_AMD_MSGBUFF_ERROR 2

#define OFI_AMD_MSGBUFF_REQ 0
#define OFI_AMD_MSGBUFF_BUFF 1

typedef struct ofi_amd_msgbuff ofi_amd_msgbuff_t;

/* -EINVAL where the reference's constructor throws std::invalid_argument
 * (max_inprogress == 0 or 2^bit_width <= 2 * max_inprogress).  Slots are indexed by
 * sequence number modulo max_inprogress, as in the reference: choose max_inprogress
 * dividing 2^bit_width (the transport's 256 of 1024 does), or two numbers of one window
 * share a slot across the wrap. */
int ofi_amd_msgbuff_create(uint16_t max_inprogress, uint16_t bit_width, uint16_t start_seq,
			   ofi_amd_msgbuff_t **out);
int ofi_amd_msgbuff_destroy(ofi_amd_msgbuff_t *m);
/* Each returns a result code and writes the status of msg_index as the reference does. */
int ofi_amd_msgbuff_insert(ofi_amd_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status);
int ofi_amd_msgbuff_replace(ofi_amd_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status);
int ofi_amd_msgbuff_retrieve(ofi_amd_msgbuff_t *m, uint16_t msg_index, void **elem, int *type,
			     int *status);
int ofi_amd_msgbuff_complete(ofi_amd_msgbuff_t *m, uint16_t msg_index, int *status);

/* ======================================================================
 * Send communicator.
 *   Replaces the decisions of nccl_net_ofi_rdma_send_comm::send
 *   (src/nccl_ofi_rdma.cpp:5646-5860), drain_sender_eager_queue (:5561-5644),
 *   update_send_data_from_remote (:574-640), update_send_request (:2204-2232) and the
 *   send half of nccl_net_ofi_rdma_req::test (:2236-2307).
 * ====================================================================== */
#define OFI_AMD_SEND_AGAIN 0 /* the reference returns a NULL request: call send again */
#define OFI_AMD_SEND_EAGER 1 /* one fi_send of header + payload, immediate data `imm` */
#define OFI_AMD_SEND_WRITE 2 /* num_xfers RDMA writes, each with immediate data `imm` */

typedef struct {
	int32_t kind;
	int32_t req; /* handle for _completion / _test; -1 with OFI_AMD_SEND_AGAIN */
	uint16_t msg_seq_num;
	uint8_t recv_idx;
	uint8_t no_target_completion; /* receiver asked for no write completions (flag bit 0) */
	uint32_t imm;
	ofi_amd_eager_hdr_t hdr;      /* eager only: goes in front of the payload */
	uint64_t size;                /* bytes to move, after truncation to the receive buffer */
	uint64_t remote_buff_offset;  /* write only */
	uint64_t mr_key[OFI_AMD_WIRE_MAX_RAILS];
	uint32_t num_xfers;
	uint32_t pad;
	ofi_amd_xfer_info_t xfers[OFI_AMD_WIRE_MAX_RAILS]; /* the rail schedule of `size` */
} ofi_amd_send_action_t;

typedef struct {
	uint16_t next_msg_seq_num;
	uint16_t group_sends_remaining;
	uint16_t group_num_recvs;
	uint16_t cur_eager_seq;
	uint16_t eager_seq_next;
	uint8_t eager_queue_count;
	uint8_t eager_offset_next;
	uint8_t prev_eager_batch_count;
	uint8_t pad[3];
	uint32_t num_inflight_reqs;
	uint32_t num_inflight_writes;
	uint64_t n_ctrl_received;
} ofi_amd_send_state_t;

typedef struct ofi_amd_send_comm ofi_amd_send_comm_t;

int ofi_amd_send_comm_create(uint32_t remote_comm_id, uint32_t num_rails, int64_t eager_send_size,
			     uint64_t min_stripe_size, uint64_t max_small_msg_size,
			     ofi_amd_send_comm_t **out);
int ofi_amd_send_comm_destroy(ofi_amd_send_comm_t *s);
/* The 256-slot control mailbox the receiver's control messages are written into. */
ofi_amd_ctrl_msg_t *ofi_amd_send_comm_mailbox(ofi_amd_send_comm_t *s);
/* 0, or -EINVAL with OFI_AMD_MAX_SEND_REQUESTS requests in flight. */
int ofi_amd_send_comm_send(ofi_amd_send_comm_t *s, uint64_t size, int32_t tag,
			   ofi_amd_send_action_t *action);
/* One fabric completion of the request (the eager send, or one write of the schedule). */
int ofi_amd_send_comm_completion(ofi_amd_send_comm_t *s, int32_t req);
/* *done = 1 frees the request; *size is the size moved (truncated to the receive buffer). */
int ofi_amd_send_comm_test(ofi_amd_send_comm_t *s, int32_t req, int *done, uint64_t *size);
void ofi_amd_send_comm_state(const ofi_amd_send_comm_t *s, ofi_amd_send_state_t *out);

/* ======================================================================
 * Receive communicator.
 *   Replaces the decisions of nccl_net_ofi_rdma_recv_comm::recv (:3545-3745) with
 *   allocate_recv_req (:3398-3474) and insert_rdma_recv_req_into_msgbuff (:3478-3520),
 *   handle_eager_recv (:897-947), drain_recv_eager_queue (:791-892) with eager_match_recv
 *   (:727-737) and eager_copy_to_sub_recv (:745-780), handle_write_comp (:1102-1130),
 *   rdma_eager_copy_req::handle_completion (:2920-2957), inc_recv_seg_completion (:530-572),
 *   write_completion_size (:2340-2353) and rdma_recv_req::free (:1677-1695).
 * ====================================================================== */

/* One eager arrival matched to a posted receive.  Feed rx_cookie's buffer, dst, dst_len and
 * recv_len to ofi_amd_eager_copy_batch, then report each item with needs_copy != 0 through
 * ofi_amd_recv_comm_copy_done; the rx buffer can be posted again after the copy. */
typedef struct {
	uint64_t rx_cookie;
	uint64_t dst;
	uint64_t dst_len;
	uint32_t recv_len;
	int32_t req;
	int32_t sub_idx;
	int32_t needs_copy; /* 0: zero-length message, already counted as complete */
} ofi_amd_eager_copy_item_t;

typedef struct {
	uint16_t next_msg_seq_num;
	uint16_t eager_drain_recv_seq;
	uint16_t last_eager_seq;
	uint16_t last_completed_seq;
	uint8_t last_eager_offset;
	uint8_t has_processed_eager;
	uint8_t pad[2];
	uint32_t num_inflight_reqs;
	uint32_t eager_pending;
	uint32_t pad2;
	uint64_t n_ctrl_sent;
} ofi_amd_recv_state_t;

typedef struct ofi_amd_recv_comm ofi_amd_recv_comm_t;

int ofi_amd_recv_comm_create(uint32_t num_rails, ofi_amd_recv_comm_t **out);
int ofi_amd_recv_comm_destroy(ofi_amd_recv_comm_t *r);
/* Posts n (1..8) receives as one request.  The control message is built in `mailbox`
 * (256 slots: the sender's own in one process, a staging copy to RDMA-write otherwise).
 * -ENOSPC with OFI_AMD_MAX_REQUESTS requests in flight.  mr_keys is n x num_rails. */
int ofi_amd_recv_comm_recv(ofi_amd_recv_comm_t *r, int n, const uint64_t *dsts, const uint64_t *sizes,
			   const int *tags, const uint64_t *mr_keys, int completion_optional,
			   ofi_amd_ctrl_msg_t *mailbox, int32_t *req, uint16_t *msg_seq_num);
/* An eager message landed in rx buffer `rx_cookie`; recv_len excludes the 8-byte header.
 * -ENOMEM when 256 arrivals are already waiting. */
int ofi_amd_recv_comm_eager_arrival(ofi_amd_recv_comm_t *r, uint16_t msg_seq_num,
				    const ofi_amd_eager_hdr_t *hdr, uint32_t recv_len, uint64_t rx_cookie);
/* The completion of one remote write carrying `imm`, `len` bytes long. */
int ofi_amd_recv_comm_write_arrival(ofi_amd_recv_comm_t *r, uint32_t imm, uint64_t len);
/* The completion of the request's control-message post. */
int ofi_amd_recv_comm_ctrl_sent(ofi_amd_recv_comm_t *r, int32_t req);
uint32_t ofi_amd_recv_comm_take_copies(ofi_amd_recv_comm_t *r, ofi_amd_eager_copy_item_t *out,
				       uint32_t cap);
int ofi_amd_recv_comm_copy_done(ofi_amd_recv_comm_t *r, int32_t req, int32_t sub_idx);
/* *done = 1 frees the request; sizes[0] for one receive, sizes[0..n) for a grouped one. */
int ofi_amd_recv_comm_test(ofi_amd_recv_comm_t *r, int32_t req, int *done, int *sizes);
/* The flush NCCL asks for after a receive into GPU memory (nccl_net_ofi_rdma_recv_comm::flush,
 * :4405-4510).  One flush covers all n buffers; when every size is 0 none is needed and *req is
 * -1.  Otherwise *req is a flush request (its own handle space; it counts against the same
 * OFI_AMD_MAX_REQUESTS in-flight limit as receives: -ENOSPC when full) and the caller posts the
 * read-back: ofi_amd_flush_post of the flush buffer into one 64-byte host slot per rail.
 * _flush_test is has_flush_completed (:2110-2126) on those slots and frees the request when
 * every slot shows the sentinel.  (The reference keeps the request until the completions of
 * its loop-back reads have drained as well; a read-back done by a kernel has none.) */
int ofi_amd_recv_comm_flush(ofi_amd_recv_comm_t *r, int n, const int *sizes, int32_t *req);
int ofi_amd_recv_comm_flush_test(ofi_amd_recv_comm_t *r, int32_t req, const void *slots_host,
				 uint32_t num_rails, uint64_t sentinel, int *done);
void ofi_amd_recv_comm_state(const ofi_amd_recv_comm_t *r, ofi_amd_recv_state_t *out);

/* ======================================================================
 * The whole send/receive path in one process on one GPU.
 *   Stands where the reference needs two ranks and a libfabric provider: the isend / irecv /
 *   test loop of tests/functional/nccl_message_transfer.cpp:19-56 (ten send/receive size
 *   pairs, NCCL_NET_MAX_REQUESTS requests in flight, tests/functional/functional_test.h:28).
 *   Message i moves min(sizes[i], dst_sizes[i]) bytes from
 *   src_addrs[i] to dst_addrs[i] (device addresses); `inflight` (1..128) messages are open at
 *   a time.  Small messages leave as eager sends ahead of their control message (header +
 *   payload copied into an rx buffer of rx_pool, then out of it by ofi_amd_eager_copy_batch);
 *   the others wait for the receive and go as striped RDMA writes (ofi_amd_copy_table).
 *   `group` (1..8) consecutive messages share one grouped receive request, matched by tag
 *   (tags NULL: 1..group within each request; tags given: distinct within a request).
 *   rx_pool: device-accessible memory, inflight x 8320 bytes.  flags bit 0: the receiver
 *   posts first, so nothing goes eager.  Each round of `inflight` messages ends with the
 *   receiver's flush (ofi_amd_recv_comm_flush, the sentinel read-back of ofi_amd_flush_post)
 *   and completes when the sentinels are in the host slots.  Blocks until done;
 *   `stream` carries the launches.  -EPROTO if the state machines disagree with the wire,
 *   -EIO if a size reported back is not the size moved.
 * ====================================================================== */
typedef struct {
	uint64_t messages;
	uint64_t payload_bytes;
	uint64_t eager_messages;
	uint64_t write_messages;
	uint64_t rdma_writes;   /* stripes */
	uint64_t copy_entries;  /* table entries of the wire launches: one per eager header, eager payload and RDMA write */
	uint64_t rounds;
	uint64_t launches;
	uint64_t send_again;    /* isend calls answered "call again" */
	uint64_t flushes;       /* receiver flushes (one per round that moved data) */
	double seconds;
} ofi_amd_sendrecv_loopback_stats_t;

int ofi_amd_sendrecv_loopback_run(const uint64_t *src_addrs, const uint64_t *dst_addrs,
				  const uint64_t *sizes, const uint64_t *dst_sizes, const int32_t *tags,
				  uint64_t n_msgs, uint32_t inflight, uint32_t num_rails, uint32_t group,
				  void *rx_pool, uint64_t rx_pool_bytes, uint32_t flags, void *stream,
				  ofi_amd_sendrecv_loopback_stats_t *stats);

#ifdef __cplusplus
}
#endif
#endif /* OFI_AMD_SENDRECV_H_ */

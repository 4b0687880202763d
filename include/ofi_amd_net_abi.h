/*
 * The send/receive data path behind the reference's own entry-point signatures.
 *
 * NCCL reaches the plugin's two-sided path through the function table ncclNet_vN_t
 * (3rd-party/nccl/cuda/include/nccl/net_v6.h ... net_v12.h in the reference; v12:
 * net_v12.h:77-138).  Its data-path members
 *
 *     isend, irecv, iflush, test                                 (net_v12.h:110-119)
 *
 * are declared here as free functions with exactly those parameter lists (and with the two
 * older spellings the reference also exports: int sizes up to v8, no profiler handles up to
 * v9), returning ncclResult_t through the reference's argument checks
 * (nccl_net_ofi_isend / _irecv / _iflush / _test, src/nccl_ofi_api.cpp:440-567) and errno
 * translation (nccl_net_ofi_retval_translate, include/nccl_ofi_api.h:30-75).  Behind them run
 * this library's send and receive state machines (ofi_amd_send_comm_*, ofi_amd_recv_comm_*:
 * the decisions of nccl_net_ofi_rdma_send_comm::send, ::recv, ::flush and
 * nccl_net_ofi_rdma_req::test) and its copy kernels.
 *
 * What sendComm and recvComm point to here are the two ends of a link inside one process
 * on one GPU: the "network" between them is device copies on a stream.  An eager send is a copy
 * of header and payload into an rx buffer of the receiving end, a rendezvous write one table
 * entry per rail stripe (ofi_amd_copy_table_pieces), a matched eager arrival leaves its rx
 * buffer through ofi_amd_eager_copy_batch, a flush is the sentinel read-back of
 * ofi_amd_flush_post.  This is the reference's two-rank functional test
 * (tests/functional/nccl_message_transfer.cpp) in one process, through the signatures NCCL
 * uses.  The control-plane members (listen, connect, accept, regMr, ...) are the reference's;
 * ofi_amd_net_link_create stands where they would have produced the two comms.
 *
 * Plain C: compiles as C11 and as C++.
 */
#ifndef OFI_AMD_NET_ABI_H_
#define OFI_AMD_NET_ABI_H_

#include <stddef.h>
#include <stdint.h>

#include "ofi_amd_nccl_err.h"
#include "ofi_amd_sendrecv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- the fabric under the two comms: what libfabric is to the reference ---- */

/* What a comm asks of the fabric (rdma_send_req::post / post_eager, src/nccl_ofi_rdma.cpp:2368-2496;
 * rdma_recv_req::post of the control message, :2566-2615; rdma_flush_req::post, :2664-2713). */
#define OFI_AMD_NET_POST_EAGER 1 /* sending end: one send of the 8-byte header `hdr` followed by `len` bytes at `src`, immediate data `imm` (fi_senddata into an rx buffer of the peer) */
#define OFI_AMD_NET_POST_WRITE 2 /* sending end: one rail stripe, `len` bytes from `src` to the peer's address `dest` under `key`, immediate data `imm` (fi_writedata) */
#define OFI_AMD_NET_POST_CTRL 3  /* receiving end: the control message at `src` (`len` bytes) into the sending end's mailbox at byte offset `dest` (fi_write) */
#define OFI_AMD_NET_POST_FLUSH 4 /* receiving end: 64 bytes of the flush buffer at `dest` read into the host slot at `src` (fi_read) */

typedef struct {
	uint32_t kind;
	uint32_t rail;
	uint32_t context; /* comes back through cq_read when the post has completed */
	uint32_t imm;
	uint64_t src;
	uint64_t len;
	uint64_t dest;
	uint64_t key;
	ofi_amd_eager_hdr_t hdr; /* eager only */
} ofi_amd_net_post_t; /* 56 bytes */

/* What the fabric reports to a comm (the CQ entries handled by ofi_process_cq's callees:
 * a completed post of this end; handle_eager_recv, src/nccl_ofi_rdma.cpp:897-947;
 * handle_write_comp, :1102-1130). */
#define OFI_AMD_NET_CQ_POSTED 1 /* a post of this end has completed: `context` */
#define OFI_AMD_NET_CQ_EAGER 2  /* receiving end: an eager message is in the rx buffer `rx_cookie` (byte offset in the rx pool): `imm`, header `hdr`, `len` payload bytes behind the header */
#define OFI_AMD_NET_CQ_WRITE 3  /* receiving end: a remote write of `len` bytes carrying `imm` has landed */

typedef struct {
	uint32_t kind;
	uint32_t context;
	uint32_t imm;
	uint32_t pad;
	uint64_t len;
	uint64_t rx_cookie;
	ofi_amd_eager_hdr_t hdr;
} ofi_amd_net_cqe_t; /* 40 bytes */

typedef struct {
	/* 0, -EAGAIN (no room now: the comm queues the post and tries again from its next progress, in
	 * order, as the reference queues a request whose post returned -FI_EAGAIN), any other negative
	 * errno */
	int (*post)(void *end, const ofi_amd_net_post_t *post);
	/* entries for this end: writes up to `max`, returns how many (0: none now) or a negative errno */
	int (*cq_read)(void *end, ofi_amd_net_cqe_t *out, uint32_t max);
	/* receiving end: the rx buffer `rx_cookie` has been emptied and can take the next eager message
	 * (repost_rx_buff, src/nccl_ofi_rdma.cpp:656-670) */
	int (*repost_rx)(void *end, uint64_t rx_cookie);
	void *end;
} ofi_amd_net_fabric_ops_t;

/*
 * A sending end over a fabric: the state machine of nccl_net_ofi_rdma_send_comm (ofi_amd_send_comm_*)
 * with its posts, the queue of refused posts and the completions.  Arguments as
 * ofi_amd_net_link_create.  The fabric delivers the peer's control messages into
 * ofi_amd_net_send_comm_mailbox (256 slots of 512 bytes; a control post's `dest` is the byte
 * offset into it).
 */
int ofi_amd_net_send_comm_create(uint32_t num_rails, int64_t eager_max_size, uint64_t min_stripe_size,
				 uint64_t max_small_msg_size, const ofi_amd_net_fabric_ops_t *fabric, void **sendComm);
void *ofi_amd_net_send_comm_mailbox(void *sendComm);
/*
 * A receiving end over a fabric: the state machine of nccl_net_ofi_rdma_recv_comm, its control and
 * flush posts, and the launches that empty rx buffers into the posted receives
 * (ofi_amd_eager_copy_batch on `stream`, rx buffers addressed as rx_pool_base + rx_cookie; each
 * launch ends in a sentinel read-back, and a buffer goes back through repost_rx once its sentinel
 * has been seen).  -ENODEV without a GPU.
 */
int ofi_amd_net_recv_comm_create(uint32_t num_rails, const ofi_amd_net_fabric_ops_t *fabric, const void *rx_pool_base,
				 void *stream, void **recvComm);
/* Either kind.  A receiving end waits for its stream first; open requests die with the comm. */
int ofi_amd_net_comm_destroy(void *comm);

/*
 * The fabric of an in-process link: both ends are this process, the wire is device copies on
 * `stream`.  An eager send becomes a copy of header and payload into one of rx_buffers rx buffers
 * (-EAGAIN while none is free), a write one entry of ofi_amd_copy_table_pieces, a control message a
 * copy into the sending end's mailbox (ofi_amd_netfab_connect).  Posts travel in launch groups that
 * end in a sentinel read-back of the flush buffer; when it is seen (inside cq_read), the group's
 * completions appear on both ends' queues in posting order.  A flush read rides on such a read-back
 * (the newest one in flight, else the next): one read for all the flushes waiting.  A group leaves
 * when an end polls and finds nothing, unless two are already in flight: then posts keep gathering.
 */
typedef struct ofi_amd_netfab ofi_amd_netfab_t;
int ofi_amd_netfab_create(uint32_t num_rails, uint32_t rx_buffers, void *stream, ofi_amd_netfab_t **out);
int ofi_amd_netfab_destroy(ofi_amd_netfab_t *fab);
/* The two ends' callbacks, and the rx pool the receiving end's cookies are offsets into. */
int ofi_amd_netfab_ops(ofi_amd_netfab_t *fab, ofi_amd_net_fabric_ops_t *send_end, ofi_amd_net_fabric_ops_t *recv_end);
const void *ofi_amd_netfab_rx_pool(const ofi_amd_netfab_t *fab);
/* Where control posts land: the sending end's mailbox. */
int ofi_amd_netfab_connect(ofi_amd_netfab_t *fab, void *send_comm_mailbox);
/* Kernel launches so far (copies and sentinels) and the table entries they carried. */
int ofi_amd_netfab_counts(const ofi_amd_netfab_t *fab, uint64_t *launches, uint64_t *copy_entries);

/* ---- set-up: what connect / accept hand over (no counterpart signature in the table) ---- */

typedef struct ofi_amd_net_link ofi_amd_net_link_t;

typedef struct {
	uint64_t isend_calls;     /* all, "call again" answers included */
	uint64_t isend_again;     /* answered with a NULL request */
	uint64_t eager_sends;
	uint64_t write_sends;
	uint64_t rdma_writes;     /* rail stripes */
	uint64_t payload_bytes;   /* bytes handed to the wire: an eager message in full, a rendezvous
				   * message after truncation to its receive buffer */
	uint64_t irecv_calls;
	uint64_t flushes;         /* iflush calls that needed a read-back */
	uint64_t launches;        /* kernel launches: wire copies, eager copies, sentinels */
	uint64_t copy_entries;    /* table entries of the wire launches */
	uint64_t eager_copies;    /* rx buffers emptied by the eager copy */
	uint64_t progress_calls;
	uint64_t posts_refused;   /* posts the fabric answered -EAGAIN at the first attempt (queued, retried) */
} ofi_amd_net_link_stats_t;

/*
 * One connected pair on the current device.  num_rails 1..4; eager_max_size is
 * OFI_NCCL_EAGER_MAX_SIZE (src/nccl_ofi_rdma.cpp:6808: 8192, the most this link takes; a message
 * may go eager when its size plus the 8-byte header fits, :5758-5764; negative = no eager protocol);
 * min_stripe_size and max_small_msg_size are the scheduler's thresholds (0 = the reference's
 * defaults 131072 and 64); rx_buffers is how many eager rx buffers the receiving end keeps
 * posted (0 = 256, which is also the most: the receiving end queues at most 256 eager arrivals; 8320 bytes of
 * device memory each).  `stream` carries every
 * launch; it must outlive the link.  The calls on one link come from one thread (NCCL calls
 * each comm from one proxy thread).  -ENODEV without a GPU.
 */
int ofi_amd_net_link_create(uint32_t num_rails, int64_t eager_max_size, uint64_t min_stripe_size,
			    uint64_t max_small_msg_size, uint32_t rx_buffers, void *stream,
			    ofi_amd_net_link_t **out);
/* Waits for the stream, then frees everything; open requests die with the link. */
int ofi_amd_net_link_destroy(ofi_amd_net_link_t *link);
/* The two ends, as the sendComm / recvComm arguments below expect them. */
void *ofi_amd_net_link_send_comm(ofi_amd_net_link_t *link);
void *ofi_amd_net_link_recv_comm(ofi_amd_net_link_t *link);
int ofi_amd_net_link_stats(const ofi_amd_net_link_t *link, ofi_amd_net_link_stats_t *out);
/* The state machines under the two ends, for inspection (sequence numbers, requests in flight). */
int ofi_amd_net_link_state(const ofi_amd_net_link_t *link, ofi_amd_send_state_t *send, ofi_amd_recv_state_t *recv);

/* ---- data path: the members of ncclNet_v10_t .. v12_t, net_v12.h:110-119 ---- */

/*
 * nccl_net_ofi_isend (src/nccl_ofi_api.cpp:440-467) over nccl_net_ofi_rdma_send_comm::send
 * (src/nccl_ofi_rdma.cpp:5646-5860).  `data` is a device-accessible address.  Success with
 * *request == NULL means "call again" (net_v12.h:108-109): the matching receive's control
 * message has not arrived and the message cannot go eager; the call has then made progress on
 * its end, as the reference's does on its completion queue.  A post the fabric refuses with
 * -EAGAIN does not make the call fail: the request is returned and its posts wait in the end's
 * queue (post_with_pending_retry, :1375-1387); while posts are waiting there, the next isend
 * progresses first and answers "call again" if they still are (process_cq_if_pending,
 * :3523-3545, :5682-5692).  mhandle and phandle are not looked at (the
 * control message carries the mhandle's value as the key).  NULL comm or request ->
 * ncclInternalError; 1,024 sends in flight -> ncclInternalError (-EINVAL, :5683-5688).
 */
ncclResult_t ofi_amd_net_isend(void *sendComm, void *data, size_t size, int tag, void *mhandle, void *phandle,
			       void **request);
/*
 * nccl_net_ofi_irecv (:470-514) over nccl_net_ofi_rdma_recv_comm::recv
 * (src/nccl_ofi_rdma.cpp:3545-3745): n (1..8) receives as one request, matched to sends by tag.
 * NULL data, sizes, tags, mhandles or request, or n outside 1..8 -> ncclInvalidArgument; NULL
 * comm -> ncclInternalError; 128 receives and flushes in flight -> ncclSystemError (-ENOSPC);
 * a NULL request with success while posts of this end wait in its queue (:3595-3605).
 * The control message carries a 32-bit length: a size above 4 GiB - 1 is refused with
 * ncclInternalError (the reference stores its low 32 bits, :3461).
 */
ncclResult_t ofi_amd_net_irecv(void *recvComm, int n, void **data, size_t *sizes, int *tags, void **mhandles,
			       void **phandles, void **request);
/*
 * nccl_net_ofi_iflush (:530-567) over nccl_net_ofi_rdma_recv_comm::flush
 * (src/nccl_ofi_rdma.cpp:4405-4510): one flush for all n buffers; when every size is 0 none is
 * needed and *request is NULL.  n above 8, NULL comm, mhandles or request ->
 * ncclInternalError.
 */
ncclResult_t ofi_amd_net_iflush(void *recvComm, int n, void **data, int *sizes, void **mhandles, void **request);
/*
 * nccl_net_ofi_test (:517-527) over nccl_net_ofi_rdma_req::test (src/nccl_ofi_rdma.cpp:2236-2307):
 * progresses the link, then says whether the request is complete.  sizes (optional): the bytes
 * sent, or the bytes received by each receive of the request.  A request that has reported
 * done = 1 is back in the pool and must not be tested again (ncclInternalError if it is,
 * until the entry is reused).  NULL request -> ncclInternalError.
 */
ncclResult_t ofi_amd_net_test(void *request, int *done, int *sizes);

/* ---- the same members as the older tables spell them (src/nccl_ofi_interface_nvidia.cpp:
 * 502-555): ncclNet_v6_t .. v8_t carry int sizes (isend_v5, irecv_v5), ncclNet_v9_t size_t
 * sizes and no profiler handles (isend_v9, irecv_v9); iflush and test are the same in all ---- */
ncclResult_t ofi_amd_net_isend_v5(void *sendComm, void *data, int size, int tag, void *mhandle, void **request);
ncclResult_t ofi_amd_net_irecv_v5(void *recvComm, int n, void **data, int *sizes, int *tags, void **mhandles,
				  void **request);
ncclResult_t ofi_amd_net_isend_v9(void *sendComm, void *data, size_t size, int tag, void *mhandle,
				  void **request);
ncclResult_t ofi_amd_net_irecv_v9(void *recvComm, int n, void **data, size_t *sizes, int *tags, void **mhandles,
				  void **request);

#ifdef __cplusplus
}
#endif

#endif /* OFI_AMD_NET_ABI_H_ */

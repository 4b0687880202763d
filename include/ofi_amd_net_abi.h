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
 * message has not arrived and the message cannot go eager, or the link is out of room (rx
 * buffers, copy tables); the call has then made progress on the link, as the reference's does
 * on its completion queue.  mhandle and phandle are not looked at (in one process the
 * destination's address is its own key).  NULL comm or request -> ncclInternalError;
 * 1,024 sends in flight -> ncclInternalError (-EINVAL, :5683-5688).
 */
ncclResult_t ofi_amd_net_isend(void *sendComm, void *data, size_t size, int tag, void *mhandle, void *phandle,
			       void **request);
/*
 * nccl_net_ofi_irecv (:470-514) over nccl_net_ofi_rdma_recv_comm::recv
 * (src/nccl_ofi_rdma.cpp:3545-3745): n (1..8) receives as one request, matched to sends by tag.
 * NULL data, sizes, tags, mhandles or request, or n outside 1..8 -> ncclInvalidArgument; NULL
 * comm -> ncclInternalError; 128 receives and flushes in flight -> ncclSystemError (-ENOSPC).
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

/*
 * The GIN / RMA data path behind the reference's own entry-point signatures.
 *
 * NCCL reaches the plugin's one-sided path through the function table ncclRma_v15_t
 * (3rd-party/nccl/cuda/include/nccl/rma_v15.h:24-62 in the reference).  Its data-path members
 *
 *     iput, iputSignal, iget, iflush, test, rmaProgress          (rma_v15.h:43-56)
 *
 * are declared here as free functions with exactly those parameter lists, returning
 * ncclResult_t through the reference's errno translation (nccl_net_ofi_retval_translate,
 * include/nccl_ofi_api.h:30-75).  A maintainer points the six members of the table at them
 * (the wrappers they replace: nccl_ofi_rma_iput_v15 .. nccl_ofi_gin_ginProgress,
 * src/rdma/gin/nccl_ofi_gin_api.cpp:284-296, 363-419, 690-751); the control-plane members
 * (init, devices, listen, connect, createContext, regMrSym, ...) stay the reference's, and hand
 * what they set up to this library through the three set-up calls below.
 *
 * Plain C: compiles as C11 and as C++.
 */
#ifndef OFI_AMD_RMA_ABI_H_
#define OFI_AMD_RMA_ABI_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include "ofi_amd_hotpath.h"
#include "ofi_amd_nccl_err.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- set-up: what createContext / regMrSym hand over (no counterpart signature in the table) ---- */

/* What `rmaCtx` and `collComm` point to: one initiator state per peer rank (sequence window,
 * scheduler, pin: ofi_amd_gin_comm_t, the state of nccl_ofi_rdma_gin_put_comm), one transmit
 * engine (request pool, pending list, bounded CQ drain: nccl_ofi_gin_resources) over the
 * caller's fabric callbacks. */
typedef struct ofi_amd_rma_ctx ofi_amd_rma_ctx_t;

/* What an `mhandle` points to: a symmetric registration -- the local base address and, per
 * peer rank, the remote address, the offset the peer's NIC addresses it by and one key per rail
 * (nccl_ofi_rdma_gin_symm_mr_handle with its gin_remote_mr per rank,
 * include/rdma/gin/nccl_ofi_gin.h:168-183, 202-217). */
typedef struct ofi_amd_rma_mr ofi_amd_rma_mr_t;

/*
 * nranks peers (comm ids 0..nranks-1 must be below 1024, GIN_IMM_COMM_BITS), num_rails 1..4,
 * the endpoint scheduler's thresholds, the fabric (post / cq_read callbacks, as for
 * ofi_amd_gin_tx_create, with the reference's CQ defaults 4 x 4), max_requests pool entries.
 * window_wait_ms bounds how long iput / iputSignal keep calling progress for room in a peer's
 * sequence window (the reference's await_tx_window, src/rdma/gin/nccl_ofi_gin.cpp:518-537,
 * spins without a bound); 0 = 10,000.  An operation that finds the pool full (an operation holds
 * one entry plus one per write or read and one for its metadata message until test() has
 * reported it done) is refused with ncclSystemError before anything is posted and leaves the
 * peer's sequence numbers, window and rail state as they were: it may be issued again after
 * completions have been tested.  The reference's pool grows instead and throws when it cannot.
 */
int ofi_amd_rma_ctx_create(uint32_t nranks, uint32_t num_rails, uint64_t min_stripe_size,
			   uint64_t max_small_msg_size, const ofi_amd_gin_fabric_ops_t *fabric,
			   uint32_t max_requests, uint32_t window_wait_ms, ofi_amd_rma_ctx_t **out);
int ofi_amd_rma_ctx_destroy(ofi_amd_rma_ctx_t *ctx);

/* remote_address / remote_address_offset: nranks entries; keys: nranks x OFI_AMD_MAX_NUM_RAILS. */
int ofi_amd_rma_mr_create(ofi_amd_rma_ctx_t *ctx, uint64_t local_base, const uint64_t *remote_address,
			  const uint64_t *remote_address_offset, const uint64_t *keys, ofi_amd_rma_mr_t **out);
int ofi_amd_rma_mr_destroy(ofi_amd_rma_mr_t *mr);

/* The buffers iflush works on: one 64-byte host slot per rail the fabric can write, the device
 * address of the 64-byte flush buffer (filled with `sentinel`, ofi_amd_flush_buffer_fill). */
int ofi_amd_rma_set_flush_buffers(ofi_amd_rma_ctx_t *ctx, void *host_slots, uint64_t device_flush_buffer,
				  uint64_t sentinel);

/* An ACK message from peer `rank` has arrived (handle_ack_completion,
 * src/rdma/gin/nccl_ofi_gin.cpp:1843-1869): ack_msg is the 8-byte gin_ack_msg_t.  In the reference
 * that is a receive completion handled inside a progress call; here the owner of the fabric calls
 * this when it sees one, and may do so from inside its cq_read callback -- which is how the
 * window opens for an iput / iputSignal that is waiting in its progress loop. */
int ofi_amd_rma_ack_received(ofi_amd_rma_ctx_t *ctx, uint32_t rank, uint64_t ack_msg);

/* The initiator state towards one peer (sequence numbers, window, ACK requests: per rank as in
 * the reference's rank_comms[]) and the engine's counters, for inspection.  The scheduler, the
 * doorbell pin and the rail cursor of signal-only operations are one for all ranks, as the
 * reference's endpoint scheduler and put-comm pin are: rank UINT32_MAX returns the state that
 * holds them. */
const ofi_amd_gin_comm_t *ofi_amd_rma_peer_state(const ofi_amd_rma_ctx_t *ctx, uint32_t rank);
int ofi_amd_rma_tx_stats(const ofi_amd_rma_ctx_t *ctx, ofi_amd_gin_tx_stats_t *out);

/* ---- data path: the members of ncclRma_v15_t, rma_v15.h:43-56 ---- */

/* iput: "just implemented as an iputSignal with a zero'd signal address"
 * (nccl_ofi_gin_iput, src/rdma/gin/nccl_ofi_gin_api.cpp:393-401).  optFlags carries
 * ncclRmaOptFlags (bit 0: aggregate requests, the doorbell-coalescing hint). */
ncclResult_t ofi_amd_rma_iput(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
			      uint64_t dstOff, void *dstMhandle, uint32_t rank, uint32_t optFlags,
			      void **request);
/* nccl_ofi_rma_iputSignal_v15, :705-718 (context and isStrongSignal unused there too: "the
 * plugin's signals are always strong"); signalOp 0 none, 1 increment, 2 add. */
ncclResult_t ofi_amd_rma_iputSignal(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
				    uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
				    void *signalMhandle, uint64_t signalValue, uint32_t signalOp,
				    bool isStrongSignal, uint32_t optFlags, void **request);
/* nccl_ofi_gin_iget, :403-419 */
ncclResult_t ofi_amd_rma_iget(void *rmaCtx, int context, uint64_t remoteOff, void *remoteMhandle, size_t size,
			      uint64_t localOff, void *localMhandle, uint32_t rank, uint32_t optFlags,
			      void **request);
/* nccl_ofi_rdma_gin_put_comm::iflush, src/rdma/gin/nccl_ofi_gin.cpp:941-1003 (mhandle and rank
 * are not looked at there either: the flush reads the endpoint's own flush buffer) */
ncclResult_t ofi_amd_rma_iflush(void *rmaCtx, int context, void *mhandle, uint32_t rank, void **request);
/* nccl_ofi_gin_test, src/rdma/gin/nccl_ofi_gin_api.cpp:363-368: done once every post of the
 * operation has completed; the request is then back in the pool and must not be tested again */
ncclResult_t ofi_amd_rma_test(void *collComm, void *request, int *done);
/* nccl_ofi_gin_ginProgress, :284-296: bounded CQ drain on every rail, then the pending posts */
ncclResult_t ofi_amd_rma_rmaProgress(void *rmaCtx);

/* ---- the same data path behind the older op-tables the reference also exports ----
 *
 * ncclRma_v14_t (rma_v14.h:49-57), ncclGin_v13_t (gin_v13.h:48-57) and ncclGin_v11_t
 * (net_v11.h:222-227) carry the same operations without optFlags (the reference's wrappers
 * forward 0, src/rdma/gin/nccl_ofi_gin_api.cpp:505-564, 651-663), v13 and v11 without
 * isStrongSignal, v11 without the context number and without iget / iflush.  iflush, test and
 * the progress call have one signature in all of them: ofi_amd_rma_iflush, ofi_amd_rma_test and
 * ofi_amd_rma_rmaProgress serve every table (ginProgress in the GIN ones). */
ncclResult_t ofi_amd_rma_iput_v14(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
				  uint64_t dstOff, void *dstMhandle, uint32_t rank, void **request);
ncclResult_t ofi_amd_rma_iputSignal_v14(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp,
					bool isStrongSignal, void **request);
ncclResult_t ofi_amd_rma_iget_v14(void *rmaCtx, int context, uint64_t remoteOff, void *remoteMhandle, size_t size,
				  uint64_t localOff, void *localMhandle, uint32_t rank, void **request);
/* ncclGin_v13_t: iput and iget as in ncclRma_v14_t (the reference uses one pair of wrappers for
 * both tables, :680-682); iputSignal without isStrongSignal */
ncclResult_t ofi_amd_gin_iputSignal_v13(void *ginCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp, void **request);
/* ncclGin_v11_t: the first argument is the collective comm, which is also the context there
 * (createContext returns ginCtx = collComm, :481-498) */
ncclResult_t ofi_amd_gin_iput_v11(void *collComm, uint64_t srcOff, void *srcMhandle, size_t size, uint64_t dstOff,
				  void *dstMhandle, uint32_t rank, void **request);
ncclResult_t ofi_amd_gin_iputSignal_v11(void *collComm, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp, void **request);

#ifdef __cplusplus
}
#endif

#endif /* OFI_AMD_RMA_ABI_H_ */

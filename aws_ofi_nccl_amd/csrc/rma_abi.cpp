/*
 * The data-path members of ncclRma_v15_t (3rd-party/nccl/cuda/include/nccl/rma_v15.h:43-56),
 * and of the older ncclRma_v14_t / ncclGin_v13_t / ncclGin_v11_t the reference also exports,
 * as free functions over this library's derivation (gin_wire.cpp) and transmit engine
 * (gin_tx.cpp).  Each packs its arguments into the 64-byte descriptor the device-side put
 * would have written, resolves the caller's registration handles for the target rank,
 * derives the wire record and posts it; what comes back is a request for test().  The
 * wrappers they stand for: src/rdma/gin/nccl_ofi_gin_api.cpp:284-296, 363-419, 690-751.
 * Plain C++, no device needed.
 */
#include <cerrno>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <new>
#include <vector>

#include "nccl_translate.hpp"
#include "ofi_amd_rma_abi.h"

struct ofi_amd_rma_mr {
	ofi_amd_rma_ctx_t *ctx;
	uint64_t local_base;
	std::vector<ofi_amd_gin_mr_t> per_rank; /* remote side as rank r sees it; local_base repeated */
};

struct ofi_amd_rma_ctx {
	uint32_t nranks = 0, num_rails = 0, window_wait_ms = 0, max_requests = 0;
	/* per peer rank: sequence numbers, window and ACK-request state (nccl_ofi_gin_peer_rank_info,
	 * rank_comms[dst_rank] in the reference) */
	std::vector<ofi_amd_gin_comm_t> peers;
	/* one for all ranks, as in the reference: the endpoint's scheduler (gin_ep.get_scheduler(),
	 * src/rdma/gin/nccl_ofi_gin.cpp:590, 893), the put comm's doorbell pin (pinned_rail_id /
	 * pinned_rail_run, include/rdma/gin/nccl_ofi_gin.h:665-668) and the rail cursor of
	 * signal-only operations (get_next_rail).  Kept in the matching fields of one more
	 * ofi_amd_gin_comm_t and lent to the peer's state for the length of a derivation. */
	ofi_amd_gin_comm_t shared;
	ofi_amd_gin_tx_t *tx = nullptr;
	/* a request is the address of its pool index in this array: stable, and test() finds the
	 * context's engine through collComm as the reference's does */
	std::vector<int32_t> request_slot;
	void *flush_slots = nullptr;
	uint64_t flush_buffer = 0, flush_sentinel = 0;
};

namespace {

ncclResult_t translate(int rc)
{
	return ofi_amd::nccl_result_of(rc);
}

const ofi_amd_gin_mr_t kNoMr = {0, 0, 0, {0, 0, 0, 0}};

/* derive + post of one put / put-signal / get; the handles become a three-entry table for the
 * target rank (source, destination, signal) */
int submit(ofi_amd_rma_ctx_t *ctx, uint16_t kind, uint64_t src_off, const ofi_amd_rma_mr_t *src, uint64_t size,
	   uint64_t dst_off, const ofi_amd_rma_mr_t *dst, uint32_t rank, uint64_t signal_off,
	   const ofi_amd_rma_mr_t *sig, uint64_t signal_value, uint32_t signal_op, uint32_t opt_flags,
	   void **request)
{
	if (request) {
		*request = nullptr;
	}
	if (!ctx || !request || rank >= ctx->nranks) {
		return -EINVAL;
	}
	/* a transfer needs both registrations (the reference dereferences them); a signal may come
	 * without one only when there is no signal */
	if (size > 0 && (!src || !dst)) {
		return -EINVAL;
	}
	if ((src && src->ctx != ctx) || (dst && dst->ctx != ctx) || (sig && sig->ctx != ctx)) {
		return -EINVAL;
	}
	ofi_amd_gin_mr_t table[3] = {src ? src->per_rank[rank] : kNoMr, dst ? dst->per_rank[rank] : kNoMr,
				     sig ? sig->per_rank[rank] : kNoMr};
	ofi_amd_gin_desc_t d;
	std::memset(&d, 0, sizeof(d));
	d.src_off = src_off;
	d.dst_off = dst_off;
	d.size = size;
	d.signal_off = signal_off;
	d.signal_value = signal_value;
	d.rank = rank;
	d.signal_op = signal_op;
	d.opt_flags = opt_flags;
	d.src_mr = 0;
	d.dst_mr = 1;
	d.sig_mr = sig ? 2 : 0xffff;
	d.kind = (kind == OFI_AMD_GIN_KIND_PUT && signal_op != 0) ? OFI_AMD_GIN_KIND_PUT_SIGNAL : kind;

	ofi_amd_gin_comm_t *peer = &ctx->peers[rank];
	ofi_amd_gin_wire_t wire;
	ofi_amd_gin_comm_t peer_before, shared_before;
	auto derive = [&]() -> int {
		peer_before = *peer;
		shared_before = ctx->shared;
		peer->sched = ctx->shared.sched;
		peer->pinned_rail_id = ctx->shared.pinned_rail_id;
		peer->pinned_rail_run = ctx->shared.pinned_rail_run;
		peer->next_rail_id = ctx->shared.next_rail_id;
		const int e = ofi_amd_gin_derive(peer, table, 3, &d, &wire);
		ctx->shared.sched = peer->sched;
		ctx->shared.pinned_rail_id = peer->pinned_rail_id;
		ctx->shared.pinned_rail_run = peer->pinned_rail_run;
		ctx->shared.next_rail_id = peer->next_rail_id;
		return e;
	};
	int rc = derive();
	if (rc == -EAGAIN) {
		/* the peer's sequence window is full: progress until its ACKs have made room
		 * (await_tx_window, src/rdma/gin/nccl_ofi_gin.cpp:518-537) */
		using clock = std::chrono::steady_clock;
		const auto t0 = clock::now();
		while (rc == -EAGAIN) {
			rc = ofi_amd_gin_tx_progress(ctx->tx);
			if (rc != 0) {
				return rc;
			}
			rc = derive();
			if (rc == -EAGAIN && std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - t0).count() >
						     (long long)ctx->window_wait_ms) {
				return -ETIMEDOUT;
			}
		}
	}
	if (rc != 0) {
		return rc;
	}
	/* A full request pool is found before anything is posted, and then the operation never
	 * happened: its sequence number, its place in the window and the rails it would have taken
	 * go back.  A number used up without a post would stall the target's in-order retire for good. */
	ofi_amd_gin_tx_stats_t ts;
	(void)ofi_amd_gin_tx_stats(ctx->tx, &ts);
	if (ctx->max_requests - ts.requests < 1u + wire.num_writes + (wire.has_meta ? 1u : 0u)) {
		*peer = peer_before;
		ctx->shared = shared_before;
		return -ENOMEM;
	}
	int32_t op = -1;
	rc = kind == OFI_AMD_GIN_KIND_GET ? ofi_amd_gin_tx_iget(ctx->tx, rank, &wire, &op)
					  : ofi_amd_gin_tx_iput_signal(ctx->tx, rank, &wire, &op);
	if (rc != 0) {
		return rc;
	}
	ctx->request_slot[(size_t)op] = op;
	*request = &ctx->request_slot[(size_t)op];
	return 0;
}

} // namespace

extern "C" {

int ofi_amd_rma_ctx_create(uint32_t nranks, uint32_t num_rails, uint64_t min_stripe_size,
			   uint64_t max_small_msg_size, const ofi_amd_gin_fabric_ops_t *fabric,
			   uint32_t max_requests, uint32_t window_wait_ms, ofi_amd_rma_ctx_t **out)
{
	if (!out || !fabric || nranks == 0 || nranks > 1024 || max_requests == 0) {
		return -EINVAL;
	}
	ofi_amd_rma_ctx *ctx = new (std::nothrow) ofi_amd_rma_ctx;
	if (!ctx) {
		return -ENOMEM;
	}
	try {
		ctx->peers.resize(nranks);
		ctx->request_slot.assign(max_requests, -1);
	} catch (...) {
		delete ctx;
		return -ENOMEM;
	}
	int rc = 0;
	for (uint32_t r = 0; r < nranks && rc == 0; r++) {
		/* ack_model 0: ACKs arrive from the peer (ofi_amd_rma_ack_received) */
		rc = ofi_amd_gin_comm_init(&ctx->peers[r], r, num_rails, min_stripe_size, max_small_msg_size, 0);
	}
	/* OFI_NCCL_CQ_READ_COUNT and OFI_NCCL_GIN_CQ_PROCESS_MAX_ITER, include/nccl_ofi_param.h:104-109 */
	if (rc == 0) {
		rc = ofi_amd_gin_comm_init(&ctx->shared, 0, num_rails, min_stripe_size, max_small_msg_size, 0);
	}
	if (rc == 0) {
		rc = ofi_amd_gin_tx_create(num_rails, 4, 4, max_requests, fabric, &ctx->tx);
	}
	if (rc != 0) {
		delete ctx;
		return rc;
	}
	ctx->nranks = nranks;
	ctx->num_rails = num_rails;
	ctx->max_requests = max_requests;
	ctx->window_wait_ms = window_wait_ms ? window_wait_ms : 10000;
	*out = ctx;
	return 0;
}

int ofi_amd_rma_ctx_destroy(ofi_amd_rma_ctx_t *ctx)
{
	if (!ctx) {
		return -EINVAL;
	}
	(void)ofi_amd_gin_tx_destroy(ctx->tx);
	delete ctx;
	return 0;
}

int ofi_amd_rma_mr_create(ofi_amd_rma_ctx_t *ctx, uint64_t local_base, const uint64_t *remote_address,
			  const uint64_t *remote_address_offset, const uint64_t *keys, ofi_amd_rma_mr_t **out)
{
	if (!ctx || !remote_address || !remote_address_offset || !keys || !out) {
		return -EINVAL;
	}
	ofi_amd_rma_mr *mr = new (std::nothrow) ofi_amd_rma_mr;
	if (!mr) {
		return -ENOMEM;
	}
	try {
		mr->per_rank.resize(ctx->nranks);
	} catch (...) {
		delete mr;
		return -ENOMEM;
	}
	mr->ctx = ctx;
	mr->local_base = local_base;
	for (uint32_t r = 0; r < ctx->nranks; r++) {
		ofi_amd_gin_mr_t &e = mr->per_rank[r];
		e.local_base = local_base;
		e.remote_address = remote_address[r];
		e.remote_address_offset = remote_address_offset[r];
		for (uint32_t k = 0; k < OFI_AMD_MAX_NUM_RAILS; k++) {
			e.key[k] = keys[(size_t)r * OFI_AMD_MAX_NUM_RAILS + k];
		}
	}
	*out = mr;
	return 0;
}

int ofi_amd_rma_mr_destroy(ofi_amd_rma_mr_t *mr)
{
	if (!mr) {
		return -EINVAL;
	}
	delete mr;
	return 0;
}

int ofi_amd_rma_set_flush_buffers(ofi_amd_rma_ctx_t *ctx, void *host_slots, uint64_t device_flush_buffer,
				  uint64_t sentinel)
{
	if (!ctx || !host_slots || (reinterpret_cast<uintptr_t>(host_slots) & 7u) != 0) {
		return -EINVAL;
	}
	ctx->flush_slots = host_slots;
	ctx->flush_buffer = device_flush_buffer;
	ctx->flush_sentinel = sentinel;
	return 0;
}

int ofi_amd_rma_ack_received(ofi_amd_rma_ctx_t *ctx, uint32_t rank, uint64_t ack_msg)
{
	if (!ctx || rank >= ctx->nranks) {
		return -EINVAL;
	}
	/* gin_ack_msg_t: rx_consumed in bits 12..25 */
	ofi_amd_gin_apply_ack(&ctx->peers[rank], (uint32_t)(ack_msg >> 12) & 0x3fffu);
	return 0;
}

const ofi_amd_gin_comm_t *ofi_amd_rma_peer_state(const ofi_amd_rma_ctx_t *ctx, uint32_t rank)
{
	if (ctx && rank == UINT32_MAX) {
		return &ctx->shared; /* scheduler, pin and rail cursor shared by all ranks */
	}
	return (ctx && rank < ctx->nranks) ? &ctx->peers[rank] : nullptr;
}

int ofi_amd_rma_tx_stats(const ofi_amd_rma_ctx_t *ctx, ofi_amd_gin_tx_stats_t *out)
{
	return ctx ? ofi_amd_gin_tx_stats(ctx->tx, out) : -EINVAL;
}

ncclResult_t ofi_amd_rma_iputSignal(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
				    uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
				    void *signalMhandle, uint64_t signalValue, uint32_t signalOp,
				    bool isStrongSignal, uint32_t optFlags, void **request)
{
	(void)context;
	(void)isStrongSignal; /* "the plugin's signals are always strong" (:713-714) */
	return translate(submit(static_cast<ofi_amd_rma_ctx_t *>(rmaCtx), OFI_AMD_GIN_KIND_PUT, srcOff,
				static_cast<ofi_amd_rma_mr_t *>(srcMhandle), size, dstOff,
				static_cast<ofi_amd_rma_mr_t *>(dstMhandle), rank, signalOff,
				static_cast<ofi_amd_rma_mr_t *>(signalMhandle), signalValue, signalOp, optFlags,
				request));
}

ncclResult_t ofi_amd_rma_iput(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
			      uint64_t dstOff, void *dstMhandle, uint32_t rank, uint32_t optFlags, void **request)
{
	return ofi_amd_rma_iputSignal(rmaCtx, context, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, 0, nullptr, 0,
				      0, false, optFlags, request);
}

ncclResult_t ofi_amd_rma_iget(void *rmaCtx, int context, uint64_t remoteOff, void *remoteMhandle, size_t size,
			      uint64_t localOff, void *localMhandle, uint32_t rank, uint32_t optFlags,
			      void **request)
{
	(void)context;
	if (!remoteMhandle || !localMhandle) {
		if (request) {
			*request = nullptr;
		}
		return ncclInternalError;
	}
	/* a get's descriptor: the source side is the remote registration, the destination the local one */
	return translate(submit(static_cast<ofi_amd_rma_ctx_t *>(rmaCtx), OFI_AMD_GIN_KIND_GET, remoteOff,
				static_cast<ofi_amd_rma_mr_t *>(remoteMhandle), size, localOff,
				static_cast<ofi_amd_rma_mr_t *>(localMhandle), rank, 0, nullptr, 0, 0, optFlags, request));
}

ncclResult_t ofi_amd_rma_iflush(void *rmaCtx, int context, void *mhandle, uint32_t rank, void **request)
{
	(void)context;
	(void)mhandle;
	(void)rank;
	ofi_amd_rma_ctx_t *ctx = static_cast<ofi_amd_rma_ctx_t *>(rmaCtx);
	if (!ctx || !request) {
		return ncclInternalError;
	}
	*request = nullptr;
	if (!ctx->flush_slots) {
		return ncclInternalError; /* ofi_amd_rma_set_flush_buffers has not been called */
	}
	int32_t op = -1;
	const int rc = ofi_amd_gin_tx_iflush(ctx->tx, ctx->flush_slots, ctx->flush_buffer, ctx->flush_sentinel, &op);
	if (rc != 0) {
		return translate(rc);
	}
	ctx->request_slot[(size_t)op] = op;
	*request = &ctx->request_slot[(size_t)op];
	return ncclSuccess;
}

ncclResult_t ofi_amd_rma_test(void *collComm, void *request, int *done)
{
	ofi_amd_rma_ctx_t *ctx = static_cast<ofi_amd_rma_ctx_t *>(collComm);
	if (!ctx || !request || !done || ctx->request_slot.empty()) {
		return ncclInternalError;
	}
	/* a request is the address of an entry of request_slot: anything else (another context's,
	 * a stray pointer, an address inside an entry) is refused before it is read */
	const uintptr_t first = reinterpret_cast<uintptr_t>(ctx->request_slot.data());
	const uintptr_t at = reinterpret_cast<uintptr_t>(request);
	if (at < first || at - first >= ctx->request_slot.size() * sizeof(int32_t) || (at - first) % sizeof(int32_t) != 0) {
		return ncclInternalError;
	}
	const size_t index = (at - first) / sizeof(int32_t);
	if (ctx->request_slot[index] != (int32_t)index) {
		return ncclInternalError; /* already completed */
	}
	const int rc = ofi_amd_gin_tx_test(ctx->tx, (int32_t)index, done);
	if (rc == 0 && *done) {
		ctx->request_slot[index] = -1;
	}
	return translate(rc);
}

ncclResult_t ofi_amd_rma_rmaProgress(void *rmaCtx)
{
	ofi_amd_rma_ctx_t *ctx = static_cast<ofi_amd_rma_ctx_t *>(rmaCtx);
	return ctx ? translate(ofi_amd_gin_tx_progress(ctx->tx)) : ncclInternalError;
}

/* The older op-tables: no optFlags (0, as the reference's wrappers forward,
 * src/rdma/gin/nccl_ofi_gin_api.cpp:505-564, 651-663). */
ncclResult_t ofi_amd_rma_iput_v14(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
				  uint64_t dstOff, void *dstMhandle, uint32_t rank, void **request)
{
	return ofi_amd_rma_iput(rmaCtx, context, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, 0, request);
}

ncclResult_t ofi_amd_rma_iputSignal_v14(void *rmaCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp,
					bool isStrongSignal, void **request)
{
	return ofi_amd_rma_iputSignal(rmaCtx, context, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, signalOff,
				      signalMhandle, signalValue, signalOp, isStrongSignal, 0, request);
}

ncclResult_t ofi_amd_rma_iget_v14(void *rmaCtx, int context, uint64_t remoteOff, void *remoteMhandle, size_t size,
				  uint64_t localOff, void *localMhandle, uint32_t rank, void **request)
{
	return ofi_amd_rma_iget(rmaCtx, context, remoteOff, remoteMhandle, size, localOff, localMhandle, rank, 0, request);
}

ncclResult_t ofi_amd_gin_iputSignal_v13(void *ginCtx, int context, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp, void **request)
{
	return ofi_amd_rma_iputSignal(ginCtx, context, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, signalOff,
				      signalMhandle, signalValue, signalOp, true, 0, request);
}

ncclResult_t ofi_amd_gin_iput_v11(void *collComm, uint64_t srcOff, void *srcMhandle, size_t size, uint64_t dstOff,
				  void *dstMhandle, uint32_t rank, void **request)
{
	return ofi_amd_rma_iput(collComm, 0, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, 0, request);
}

ncclResult_t ofi_amd_gin_iputSignal_v11(void *collComm, uint64_t srcOff, void *srcMhandle, size_t size,
					uint64_t dstOff, void *dstMhandle, uint32_t rank, uint64_t signalOff,
					void *signalMhandle, uint64_t signalValue, uint32_t signalOp, void **request)
{
	return ofi_amd_rma_iputSignal(collComm, 0, srcOff, srcMhandle, size, dstOff, dstMhandle, rank, signalOff,
				      signalMhandle, signalValue, signalOp, true, 0, request);
}

} /* extern "C" */

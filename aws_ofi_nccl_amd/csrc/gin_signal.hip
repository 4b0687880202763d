/*
 * Signal delivery on the GPU: a batch of folded signal work items becomes one launch of
 * 64-bit device-scope atomic adds on the counters in HBM.
 *
 * The reference updates each counter from a CPU worker thread through GDRCopy -- a PCIe
 * read and a PCIe write per slot (apply_signal_work, src/rdma/gin/nccl_ofi_gin.cpp:
 * 1193-1256) -- and therefore folds a batch by slot first to save round trips
 * (apply_and_complete, :1425-1479).  With the adds executed next to the memory the fold
 * is unnecessary for speed and, additions being commutative, for the result: N items on
 * one slot leave it at the same value as the reference's single +sum write.
 */
#include "common.hpp"
#include "ofi_amd_hotpath.h"

namespace {

constexpr uint32_t kMaxRegions = 16;
constexpr uint32_t kMaxApplyPost = 65536; /* items one workgroup applies in front of a flush read */

struct regions_t {
	uint64_t base[kMaxRegions];
	uint64_t size[kMaxRegions];
	uint64_t *counters[kMaxRegions];
	uint32_t n;
};

__device__ __forceinline__ void apply_one(const ofi_amd_gin_signal_work_t &w, const regions_t &regions,
					  uint32_t *__restrict__ rejected)
{
	uint64_t *slot = nullptr;
	/* The window is found by its base; the counter by its address inside the window, which may
	 * continue through the regions listed next while each begins where the one before it ends
	 * (a window backed by several allocations: the reference looks the segment up by address
	 * too, ensure_signal_seg, src/rdma/gin/nccl_ofi_gin.cpp:1038-1122, 1156-1166). */
	for (uint32_t r = 0; r < regions.n; r++) {
		if (w.base != regions.base[r]) {
			continue;
		}
		uint64_t off = w.offset;
		for (uint32_t k = r;; k++) {
			if (off <= regions.size[k] && regions.size[k] - off >= 8) {
				slot = regions.counters[k] + (off >> 3);
				break;
			}
			if (off < regions.size[k] || k + 1 >= regions.n ||
			    regions.base[k + 1] != regions.base[k] + regions.size[k]) {
				break; /* a counter across the end of a segment, or past the window */
			}
			off -= regions.size[k];
		}
		break;
	}
	if (slot == nullptr || (w.offset & 7u) != 0) {
		if (rejected) {
			atomicAdd(rejected, 1u);
		}
		return;
	}
	/* relaxed: ordering against the payload is the put-before-signal protocol's business
	 * (the reference uses a relaxed fetch_add on its host path for the same reason, :1209) */
	__hip_atomic_fetch_add(slot, w.value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(256) void gin_signal_apply_kernel(
	const ofi_amd_gin_signal_work_t *__restrict__ work, uint32_t n, regions_t regions,
	uint32_t *__restrict__ rejected)
{
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i < n) {
		apply_one(work[i], regions, rejected);
	}
}

/* The adds of a batch and the flush read behind them in one launch of one workgroup: every
 * thread's adds have been performed at the memory before the workgroup meets, and only then is
 * the flush buffer read back into the host's slots -- what two launches order by the kernel
 * boundary between them. */
__global__ __launch_bounds__(256) void gin_signal_apply_post_kernel(
	const ofi_amd_gin_signal_work_t *__restrict__ work, uint32_t n, regions_t regions,
	uint32_t *__restrict__ rejected, const uint64_t *__restrict__ flush_buf, uint64_t *__restrict__ slots,
	uint32_t num_rails)
{
	for (uint32_t i = threadIdx.x; i < n; i += 256u) {
		apply_one(work[i], regions, rejected);
	}
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
	__syncthreads();
	if (threadIdx.x < 64u) {
		ofi_amd::flush_post_lanes(flush_buf, slots, num_rails, threadIdx.x);
	}
}

} // namespace

using namespace ofi_amd;

static int pack_regions(const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions, regions_t *r)
{
	if (!regions || n_regions == 0 || n_regions > kMaxRegions) {
		return -EINVAL;
	}
	r->n = n_regions;
	for (uint32_t i = 0; i < kMaxRegions; i++) {
		const bool live = i < n_regions;
		if (live && (!regions[i].d_counters || (reinterpret_cast<uintptr_t>(regions[i].d_counters) & 7u))) {
			return -EINVAL;
		}
		r->base[i] = live ? regions[i].base : 0;
		r->size[i] = live ? regions[i].size : 0;
		r->counters[i] = live ? static_cast<uint64_t *>(regions[i].d_counters) : nullptr;
	}
	return 0;
}

extern "C" int ofi_amd_gin_signal_apply(const ofi_amd_gin_signal_work_t *d_work, uint32_t n,
					const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
					uint32_t *d_rejected, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	regions_t r;
	if (!d_work || pack_regions(regions, n_regions, &r) != 0) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(gin_signal_apply_kernel, dim3((n + 255u) / 256u), dim3(256), 0, as_stream(stream),
			   d_work, n, r, d_rejected);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

extern "C" int ofi_amd_gin_signal_apply_post(const ofi_amd_gin_signal_work_t *d_work, uint32_t n,
					     const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
					     uint32_t *d_rejected, const void *d_flush_buf, void *slots_dev,
					     uint32_t num_rails, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!d_flush_buf || !slots_dev || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS ||
	    (reinterpret_cast<uintptr_t>(d_flush_buf) & 7u) || (reinterpret_cast<uintptr_t>(slots_dev) & 7u)) {
		return -EINVAL;
	}
	if (n > kMaxApplyPost) {
		return -E2BIG;
	}
	regions_t r = {};
	if (n != 0 && (!d_work || pack_regions(regions, n_regions, &r) != 0)) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(gin_signal_apply_post_kernel, dim3(1), dim3(256), 0, as_stream(stream), d_work, n, r,
			   d_rejected, static_cast<const uint64_t *>(d_flush_buf), static_cast<uint64_t *>(slots_dev),
			   num_rails);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

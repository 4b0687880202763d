/*
 * Batched bounce / eager copy and read-back flush for gfx950.
 *
 * The reference copies every eager payload with its own loop-back fi_read from
 * the bounce buffer into the receive buffer
 * (rdma_eager_copy_req::post, src/nccl_ofi_rdma.cpp:2729-2776) and forces
 * visibility with a small read-back (rdma_flush_req::post, :2664-2713).  Here
 * one launch moves a whole batch.
 *
 * Work mapping: one 64-lane wavefront per buffer.  Destinations are 64-byte
 * aligned, so every lane stores whole 16-byte words.  A wavefront covers up to
 * 8 KiB (the eager limit) per trip: all eight loads of a lane are issued before
 * its first store, so the whole buffer is in flight at once whatever its length.
 * The table entry of the buffer is wave-uniform and is read through the scalar
 * cache.
 *
 * The packed source can start at any byte.  16-byte loads from a 4-byte-aligned
 * address run at full rate on gfx950, loads from an odd byte address do not
 * (measured: about 15 % slower), so a source that is not 4-byte aligned is read
 * as aligned dwords -- four plus the one that follows -- and each output dword
 * is cut out of two neighbours with v_alignbyte_b32.  The fifth dword always
 * contains at least one byte of the buffer, so nothing beyond the dword that
 * holds the last source byte is read.  The sub-16-byte tail goes out as single
 * bytes so that nothing outside [dst, dst+len) is written.
 *
 * Flush: the wave waits until its own stores have left the CU (they are
 * write-through to the L2 of its XCD), then lane 0 re-reads the first 4 bytes
 * of the destination from that L2 and writes them to d_flush[i].  No wider
 * fence is used: on a multi-XCD part a device-scope release per buffer would
 * write back the whole L2 each time; device-wide visibility of the copied
 * bytes comes with the end of the kernel, as for any other kernel output.
 */
#include "common.hpp"
#include "ofi_amd_hotpath.h"

#ifndef OFI_BOUNCE_WAVES
#define OFI_BOUNCE_WAVES 1 /* 64-thread workgroups measured fastest: finer-grained slot reuse */
#endif

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
/* 16 bytes at a 4-byte-aligned address */
struct __attribute__((packed, aligned(4))) dword_aligned_u32x4 {
	u32x4 v;
};

constexpr int kWavesPerBlock = OFI_BOUNCE_WAVES;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr uint32_t kXcds = 8;
#ifndef OFI_BOUNCE_DEPTH
#define OFI_BOUNCE_DEPTH 8
#endif
constexpr uint32_t kVecPerTrip = OFI_BOUNCE_DEPTH; /* 16-byte words per lane per trip: 8 KiB per wave */

__device__ __forceinline__ u32x4 load16_dword_aligned(const uint8_t *p)
{
	return reinterpret_cast<const dword_aligned_u32x4 *>(p)->v;
}

/* Copies nvec 16-byte words from s (4-byte aligned) + shift bytes to d (16-byte aligned).
 * SHIFTED = false: shift is 0 and the source words are used as they are. */
template <bool SHIFTED>
__device__ __forceinline__ void copy_words(const uint8_t *__restrict__ s, uint8_t *__restrict__ d,
					   uint32_t nvec, uint32_t shift, uint32_t lane)
{
	for (uint32_t base = 0; base < nvec; base += kVecPerTrip * 64u) {
		u32x4 v[kVecPerTrip];
		uint32_t x[kVecPerTrip];
#pragma unroll
		for (uint32_t k = 0; k < kVecPerTrip; k++) {
			const uint32_t j = base + k * 64u + lane;
			if (j < nvec) {
				v[k] = load16_dword_aligned(s + ((uint64_t)j << 4));
				if (SHIFTED) {
					x[k] = *reinterpret_cast<const uint32_t *>(s + ((uint64_t)j << 4) + 16);
				}
			}
		}
#pragma unroll
		for (uint32_t k = 0; k < kVecPerTrip; k++) {
			const uint32_t j = base + k * 64u + lane;
			if (j < nvec) {
				u32x4 o = v[k];
				if (SHIFTED) {
					o.x = __builtin_amdgcn_alignbyte(v[k].y, v[k].x, shift);
					o.y = __builtin_amdgcn_alignbyte(v[k].z, v[k].y, shift);
					o.z = __builtin_amdgcn_alignbyte(v[k].w, v[k].z, shift);
					o.w = __builtin_amdgcn_alignbyte(x[k], v[k].w, shift);
				}
				__builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(d + ((uint64_t)j << 4)));
			}
		}
	}
}

__global__ __launch_bounds__(kBlock) void bounce_scatter_kernel(
	const uint8_t *__restrict__ src, uint8_t *__restrict__ arena, uint64_t arena_bytes,
	const uint64_t *__restrict__ src_off, const uint64_t *__restrict__ dst_off,
	const uint32_t *__restrict__ len, uint32_t n, uint32_t *__restrict__ flush,
	uint32_t *__restrict__ err)
{
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	/* Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every
	 * XCD one contiguous eighth of the batch, so that neighbouring buffers -- which share
	 * a cache line of the packed source at their boundary -- meet in the same L2. */
	const uint32_t per_xcd = gridDim.x / kXcds;
	const uint32_t wg = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
	const uint32_t buf = wg * kWavesPerBlock + wave;
	if (buf >= n) {
		return;
	}

	const uint64_t doff = dst_off[buf];
	const uint32_t bytes = len[buf];
	const uint64_t soff = src_off[buf];
	/* precondition check: skip (and report) instead of writing out of range */
	if ((doff & 63u) != 0 || doff > arena_bytes || bytes > arena_bytes - doff) {
		if (lane == 0) {
			atomicOr(err, ofi_amd::ASYNC_ERR_BOUNCE_RANGE);
		}
		return;
	}

	const uint8_t *s = src + soff;
	uint8_t *d = arena + doff;
	const uint32_t nvec = bytes >> 4;
	const uint32_t tail = bytes & 15u;

	/* tail bytes first, so their latency overlaps the body */
	uint8_t tail_byte = 0;
	const uint64_t tail_at = ((uint64_t)nvec << 4) + lane;
	if (lane < tail) {
		tail_byte = s[tail_at];
	}

	const uint32_t shift = (uint32_t)(reinterpret_cast<uintptr_t>(s) & 3u);
	if (shift == 0) {
		copy_words<false>(s, d, nvec, 0, lane);
	} else {
		copy_words<true>(s - shift, d, nvec, shift, lane);
	}
	if (lane < tail) {
		d[tail_at] = tail_byte;
	}

	if (flush != nullptr) {
		__builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
		if (lane == 0) {
			flush[buf] = __hip_atomic_load(reinterpret_cast<const uint32_t *>(d),
						       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
		}
	}
}

__global__ __launch_bounds__(256) void flush_read_kernel(const uint8_t *__restrict__ arena,
							 const uint64_t *__restrict__ dst_off,
							 uint32_t n, uint32_t *__restrict__ flush)
{
	const uint32_t i = blockIdx.x * 256u + threadIdx.x;
	if (i < n) {
		flush[i] = __hip_atomic_load(reinterpret_cast<const uint32_t *>(arena + dst_off[i]),
					     __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
	}
}

} // namespace

struct ofi_amd_devcopy_region {
	uint8_t *base;
	size_t size;
};

using namespace ofi_amd;

extern "C" {

int ofi_amd_bounce_scatter(const void *d_src, void *d_arena, uint64_t arena_bytes,
			   const uint64_t *d_src_off, const uint64_t *d_dst_off,
			   const uint32_t *d_len, uint32_t n, uint32_t *d_flush, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!d_src || !d_arena || !d_src_off || !d_dst_off || !d_len) {
		return -EINVAL;
	}
	uint32_t *err = async_error_word();
	if (!err) {
		return -ENOMEM;
	}
	uint32_t blocks = (n + kWavesPerBlock - 1) / kWavesPerBlock;
	blocks = (blocks + kXcds - 1) / kXcds * kXcds; /* whole rounds over the XCDs */
	hipLaunchKernelGGL(bounce_scatter_kernel, dim3(blocks), dim3(kBlock), 0, as_stream(stream),
			   static_cast<const uint8_t *>(d_src), static_cast<uint8_t *>(d_arena),
			   arena_bytes, d_src_off, d_dst_off, d_len, n, d_flush, err);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_flush_read(const void *d_arena, const uint64_t *d_dst_off, uint32_t n,
		       uint32_t *d_flush, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!d_arena || !d_dst_off || !d_flush) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(flush_read_kernel, dim3((n + 255u) / 256u), dim3(256), 0,
			   as_stream(stream), static_cast<const uint8_t *>(d_arena), d_dst_off, n,
			   d_flush);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

/* ---- nccl_ofi_device_copy (include/nccl_ofi_device_copy.h:14-69) ---- */

int ofi_amd_devcopy_register(void *device_ptr, size_t size, ofi_amd_devcopy_region_t **out)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!device_ptr || size == 0 || !out) {
		return -EINVAL;
	}
	hipPointerAttribute_t attr;
	if (hipPointerGetAttributes(&attr, device_ptr) != hipSuccess) {
		(void)hipGetLastError();
		return -EINVAL;
	}
	if (attr.type != hipMemoryTypeDevice) {
		return -EINVAL;
	}
	auto *h = new (std::nothrow) ofi_amd_devcopy_region;
	if (!h) {
		return -ENOMEM;
	}
	h->base = static_cast<uint8_t *>(device_ptr);
	h->size = size;
	*out = h;
	return 0;
}

int ofi_amd_devcopy_to_device(const void *host_ptr, ofi_amd_devcopy_region_t *h, size_t offset,
			      size_t size)
{
	if (!h || !host_ptr || offset > h->size || size > h->size - offset) {
		return -EINVAL;
	}
	OFI_AMD_HIP_TRY(hipMemcpy(h->base + offset, host_ptr, size, hipMemcpyHostToDevice));
	return 0;
}

int ofi_amd_devcopy_from_device(ofi_amd_devcopy_region_t *h, size_t offset, void *host_ptr,
				size_t size)
{
	if (!h || !host_ptr || offset > h->size || size > h->size - offset) {
		return -EINVAL;
	}
	OFI_AMD_HIP_TRY(hipMemcpy(host_ptr, h->base + offset, size, hipMemcpyDeviceToHost));
	return 0;
}

int ofi_amd_devcopy_forced_pcie_copy(void)
{
	return 0;
}

int ofi_amd_devcopy_deregister(ofi_amd_devcopy_region_t *h)
{
	if (!h) {
		return -EINVAL;
	}
	delete h;
	return 0;
}

} /* extern "C" */

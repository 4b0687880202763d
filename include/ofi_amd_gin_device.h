/*
 * Device side of the GIN descriptor rings: what a HIP kernel calls to initiate a put, a
 * put-signal or a get (a descriptor of kind OFI_AMD_GIN_KIND_GET travels the same way).
 * Compile with hipcc for gfx950; host code only needs ofi_amd_hotpath.h.
 *
 * The reference has no such call on AMD or in proxy mode -- NCCL's own GPU-to-CPU queue
 * feeds its proxy thread, which calls iputSignal (src/rdma/gin/nccl_ofi_gin_api.cpp:370-419);
 * its GPU-initiated build posts NIC work queue entries from device code instead
 * (include/rdma/gin/nccl_ofi_gin_gdaki_dev.h:131-336).  Here the device hands the host proxy
 * the iputSignal argument tuple through a ring with the slot protocol of
 * include/nccl_ofi_mpsc_ring.h:79-143: a slot's sequence word equals its position when free,
 * position + 1 when published; the consumer frees it with position + capacity.
 */
#ifndef OFI_AMD_GIN_DEVICE_H_
#define OFI_AMD_GIN_DEVICE_H_

#include <hip/hip_runtime.h>

#include "ofi_amd_hotpath.h"

#define OFI_AMD_GIN_DEV_TIMEOUT_BIT 2u /* the bit ofi_amd_gin_producer_status() reports */

/*
 * Wave-collective: all 64 lanes of the wavefront call it together (no divergence around
 * the call); lanes with active == true each put *desc.  Returns 0, or -1 when the ring
 * stayed full for spin_limit polls -- the timeout bit is then set in the ring's status word
 * and the reserved slots are never published, so the ring must not be used any further
 * until the host has reset it (ofi_amd_gin_rings_reset, once the kernel has ended).
 *
 * The wave's descriptors take consecutive positions in lane order: one atomic add on the
 * device-resident cursor per call (not per descriptor, and nothing atomic over the host
 * link), positions from a ballot and a prefix popcount.  The single consumer frees slots
 * in position order, so one lane checking one slot is enough, and what it learns is kept
 * in a device-resident horizon so that most calls read nothing over the host link.  Records go out
 * as four 16-byte stores per lane, then a system-scope release fence, then the sequence
 * words: the host proxy that sees a published sequence word sees the record.
 */
__device__ __forceinline__ int ofi_amd_gin_dev_put(const ofi_amd_gin_dev_ring_t ring,
						    const ofi_amd_gin_desc_t *desc, bool active,
						    uint64_t spin_limit)
{
	typedef uint32_t ofi_amd_u32x4 __attribute__((ext_vector_type(4)));
	const uint32_t lane = __lane_id();
	const uint64_t ballot = __ballot(active);
	if (ballot == 0) {
		return 0;
	}
	const uint32_t count = (uint32_t)__popcll(ballot);
	const uint32_t rank = (uint32_t)__popcll(ballot & ((1ull << lane) - 1ull));
	const uint32_t leader = (uint32_t)__ffsll((unsigned long long)ballot) - 1u;
	const uint32_t mask = ring.capacity - 1u;

	/* ring.reserve[0] is the cursor; ring.reserve[1] a horizon: every position below it is
	 * known to have been freed by the consumer.  That is a fact that stays true (a freed
	 * slot stays free until the one producer that reserved it publishes), so a stale or
	 * smaller value is merely conservative and plain loads and stores suffice for it. */
	uint32_t base = 0, horizon = 0;
	if (lane == leader) {
		horizon = __hip_atomic_load(ring.reserve + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
		base = __hip_atomic_fetch_add(ring.reserve, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	base = __shfl(base, (int)leader, 64);
	const uint32_t pos = base + rank;

	int timed_out = 0;
	if (lane == leader) {
		const uint32_t last_pos = base + count - 1u;
		if ((int32_t)(last_pos - horizon) >= 0) {
			/* Not known to be free.  The consumer frees slots in position order, so the
			 * slot of a position being free implies it for every position before it:
			 * look half a lap ahead first -- when the consumer keeps up, one read over
			 * the host link then covers the next capacity / 2 descriptors of all the
			 * ring's producers -- and fall back to waiting for the wave's own last slot. */
			const uint32_t far_pos = last_pos + (ring.capacity >> 1);
			uint32_t known = 0;
			if (__hip_atomic_load(&ring.sequences[far_pos & mask], __ATOMIC_RELAXED,
					      __HIP_MEMORY_SCOPE_SYSTEM) == far_pos) {
				known = far_pos + 1u;
			} else {
				uint64_t spins = 0;
				while (__hip_atomic_load(&ring.sequences[last_pos & mask], __ATOMIC_RELAXED,
							 __HIP_MEMORY_SCOPE_SYSTEM) != last_pos) {
					if (++spins > spin_limit) {
						timed_out = 1;
						break;
					}
					__builtin_amdgcn_s_sleep(16);
				}
				known = last_pos + 1u;
			}
			if (timed_out) {
				__hip_atomic_fetch_or(ring.status, OFI_AMD_GIN_DEV_TIMEOUT_BIT, __ATOMIC_RELAXED,
						      __HIP_MEMORY_SCOPE_SYSTEM);
			} else if ((int32_t)(known - horizon) > 0) {
				__hip_atomic_store(ring.reserve + 1, known, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
	}
	if (__shfl(timed_out, (int)leader, 64)) {
		return -1;
	}
	__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");

	ofi_amd_u32x4 part[4]; /* the descriptor is only 8-byte aligned: copy, do not cast */
	__builtin_memcpy(&part[0], reinterpret_cast<const char *>(desc), 16);
	__builtin_memcpy(&part[1], reinterpret_cast<const char *>(desc) + 16, 16);
	__builtin_memcpy(&part[2], reinterpret_cast<const char *>(desc) + 32, 16);
	__builtin_memcpy(&part[3], reinterpret_cast<const char *>(desc) + 48, 16);
	ofi_amd_u32x4 *records = static_cast<ofi_amd_u32x4 *>(ring.records);
	if (ballot == ~0ull) {
		/* Full wavefront: lanes 4g..4g+3 hold records 4g..4g+3.  Each of the four store
		 * instructions writes one whole record per group of four lanes -- lane 4g+p the
		 * p-th 16 bytes of record 4g+k -- so the host link carries complete 64-byte lines
		 * instead of four 16-byte pieces per record scattered over four instructions.
		 * The parts travel between the four lanes through DPP quad broadcasts. */
		const uint32_t p = lane & 3u;
#define OFI_AMD_GIN_QUAD_BCAST(v, ctrl) \
	((uint32_t)__builtin_amdgcn_mov_dpp((int)(v), (ctrl), 0xf, 0xf, true))
#define OFI_AMD_GIN_STORE_COLUMN(k, ctrl)                                                              \
	do {                                                                                           \
		ofi_amd_u32x4 out;                                                                     \
		ofi_amd_u32x4 q0, q1, q2, q3;                                                          \
		q0.x = OFI_AMD_GIN_QUAD_BCAST(part[0].x, ctrl); q0.y = OFI_AMD_GIN_QUAD_BCAST(part[0].y, ctrl); \
		q0.z = OFI_AMD_GIN_QUAD_BCAST(part[0].z, ctrl); q0.w = OFI_AMD_GIN_QUAD_BCAST(part[0].w, ctrl); \
		q1.x = OFI_AMD_GIN_QUAD_BCAST(part[1].x, ctrl); q1.y = OFI_AMD_GIN_QUAD_BCAST(part[1].y, ctrl); \
		q1.z = OFI_AMD_GIN_QUAD_BCAST(part[1].z, ctrl); q1.w = OFI_AMD_GIN_QUAD_BCAST(part[1].w, ctrl); \
		q2.x = OFI_AMD_GIN_QUAD_BCAST(part[2].x, ctrl); q2.y = OFI_AMD_GIN_QUAD_BCAST(part[2].y, ctrl); \
		q2.z = OFI_AMD_GIN_QUAD_BCAST(part[2].z, ctrl); q2.w = OFI_AMD_GIN_QUAD_BCAST(part[2].w, ctrl); \
		q3.x = OFI_AMD_GIN_QUAD_BCAST(part[3].x, ctrl); q3.y = OFI_AMD_GIN_QUAD_BCAST(part[3].y, ctrl); \
		q3.z = OFI_AMD_GIN_QUAD_BCAST(part[3].z, ctrl); q3.w = OFI_AMD_GIN_QUAD_BCAST(part[3].w, ctrl); \
		out = p == 0u ? q0 : (p == 1u ? q1 : (p == 2u ? q2 : q3));                             \
		const uint32_t rec_pos = base + (lane & ~3u) + (k);                                    \
		records[(uint64_t)(rec_pos & mask) * 4u + p] = out;                                    \
	} while (0)
		OFI_AMD_GIN_STORE_COLUMN(0u, 0x00);
		OFI_AMD_GIN_STORE_COLUMN(1u, 0x55);
		OFI_AMD_GIN_STORE_COLUMN(2u, 0xAA);
		OFI_AMD_GIN_STORE_COLUMN(3u, 0xFF);
#undef OFI_AMD_GIN_STORE_COLUMN
#undef OFI_AMD_GIN_QUAD_BCAST
	} else if (active) {
		ofi_amd_u32x4 *dst = records + (uint64_t)(pos & mask) * 4u;
		dst[0] = part[0];
		dst[1] = part[1];
		dst[2] = part[2];
		dst[3] = part[3];
	}
	__builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
	if (active) {
		__hip_atomic_store(&ring.sequences[pos & mask], pos + 1u, __ATOMIC_RELAXED,
				   __HIP_MEMORY_SCOPE_SYSTEM);
	}
	return 0;
}

#endif /* OFI_AMD_GIN_DEVICE_H_ */

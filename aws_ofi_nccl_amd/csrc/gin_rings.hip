/*
 * GIN put / put-signal descriptor production on the GPU (gfx950) into
 * pinned-host rings drained by the host proxy.
 *
 * In the reference the GPU never talks to the plugin: NCCL owns a GPU->CPU
 * queue and its proxy thread calls iputSignal per op
 * (src/rdma/gin/nccl_ofi_gin_api.cpp:370-419).  Here device code emits the op
 * descriptors itself -- the argument tuple of iputSignal
 * (include/nccl_ofi_gin_base.h:83-91) as a 64-byte record -- into one ring per
 * context that follows the slot protocol of include/nccl_ofi_mpsc_ring.h:56-163.
 *
 * Per 256-op round of a workgroup (= one context):
 *   1. every lane decides whether it has an op; slot positions come from a
 *      wavefront ballot + popcount prefix and a workgroup prefix over the four
 *      wave counts, added to the ring cursor -- no atomic per op;
 *   2. each lane waits until its slot is free (sequence == position), bounded
 *      by spin_limit polls;
 *   3. the wave stages its 64 records in LDS and writes them as 16-byte stores,
 *      1 KiB contiguous per instruction, to the pinned ring;
 *   4. system-scope fence, then each lane publishes sequence = position + 1
 *      with a release store (64 lanes = one contiguous 256-byte write).
 * The ring cursor (device memory, shared with ofi_amd_gin_dev_put) stays in a register for
 * the whole launch and is written back once at the end: this generator owns its context
 * for the duration of a launch.
 */
#include <cstring>
#include <new>

#include "common.hpp"
#include "gin_rings.hpp"
#include "ofi_amd_gin_device.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kThreads = 256;
constexpr uint32_t kWaves = kThreads / 64;
constexpr uint64_t kDefaultSpinLimit = 1ull << 22;
static_assert(OFI_AMD_GIN_DEV_TIMEOUT_BIT == ofi_amd::ASYNC_ERR_GIN_TIMEOUT,
	      "the device header and the status reader agree on the timeout bit");

__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
	z ^= z >> 30;
	z *= 0xBF58476D1CE4E5B9ull;
	z ^= z >> 27;
	z *= 0x94D049BB133111EBull;
	z ^= z >> 31;
	return z;
}

__device__ __forceinline__ uint64_t stream_rnd(uint64_t seed, uint32_t ctx, uint64_t i, uint32_t j)
{
	uint64_t ctr = ((((uint64_t)ctx << 40) + i) * 4u) + j + 1u;
	return mix64(seed + 0x9E3779B97F4A7C15ull * ctr);
}

/* The synthetic op stream: descriptor i of context ctx.  Sizes are log-uniform
 * in [8 B, 1 MiB) (uniform octave, uniform inside it), offsets 8-byte aligned
 * inside a 1 GiB window, a put-signal every signal_every-th op. */
__device__ __forceinline__ void make_desc(uint64_t seed, uint32_t ctx, uint64_t i, uint32_t peer_rank,
					  uint32_t signal_every, uint32_t signal_op,
					  uint32_t aggregate_mask, uint64_t w[8])
{
	const uint64_t span = (1ull << 30) - (1ull << 20);
	const uint64_t r0 = stream_rnd(seed, ctx, i, 0);
	const uint64_t r1 = stream_rnd(seed, ctx, i, 1);
	const uint64_t r2 = stream_rnd(seed, ctx, i, 2);
	const uint32_t e = 3u + (uint32_t)((r0 & 0xffu) % 17u);

	const uint64_t size = (1ull << e) | ((r0 >> 8) & ((1ull << e) - 1));
	const uint64_t src_off = ((r1 & 0xffffffffull) % span) & ~7ull;
	const uint64_t dst_off = ((r1 >> 32) % span) & ~7ull;
	const uint32_t opt_flags = (uint32_t)(r2 & aggregate_mask);
	uint64_t signal_off = 0, signal_value = 0;
	uint32_t sig_op = 0, sig_mr = 0xffffu, kind = 1;
	if (signal_every != 0 && (i % signal_every) == signal_every - 1) {
		sig_op = signal_op;
		signal_off = 8ull * ((i / signal_every) % 512u);
		signal_value = (signal_op == 2u) ? (((r2 >> 8) & 0xffffu) + 1u) : 0;
		sig_mr = 2;
		kind = 2;
	}
	/* ofi_amd_gin_desc_t, little endian */
	w[0] = src_off;
	w[1] = dst_off;
	w[2] = size;
	w[3] = signal_off;
	w[4] = signal_value;
	w[5] = (uint64_t)peer_rank | ((uint64_t)sig_op << 32);
	w[6] = (uint64_t)opt_flags | ((uint64_t)ctx << 32);
	w[7] = 0ull /* src_mr */ | (1ull << 16) /* dst_mr */ | ((uint64_t)sig_mr << 32) |
	       ((uint64_t)kind << 48);
}

__global__ __launch_bounds__(kThreads) void gin_produce_seeded_kernel(
	u32x4 *__restrict__ records, uint32_t *__restrict__ sequences,
	uint32_t *__restrict__ enqueue_pos, uint32_t *__restrict__ status, uint32_t capacity,
	uint64_t seed, uint64_t ops, uint32_t peer_rank, uint32_t signal_every, uint32_t signal_op,
	uint32_t aggregate_mask, uint64_t spin_limit)
{
	__shared__ u32x4 stage[kWaves][64 * 4];
	__shared__ uint32_t wave_count[kWaves];

	const uint32_t ctx = blockIdx.x;
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	const uint32_t mask = capacity - 1;
	u32x4 *ring = records + (uint64_t)ctx * capacity * 4;
	uint32_t *seq = sequences + (uint64_t)ctx * capacity;

	uint32_t cursor = __hip_atomic_load(&enqueue_pos[ctx * kGinReserveStride], __ATOMIC_RELAXED,
					    __HIP_MEMORY_SCOPE_AGENT);

	for (uint64_t round = 0; round < ops; round += kThreads) {
		const uint64_t i = round + threadIdx.x;
		const bool active = i < ops;

		/* slot reservation: ballot + prefix popcount, then a prefix over the waves */
		const uint64_t ballot = __ballot(active);
		const uint32_t lane_prefix = __popcll(ballot & ((1ull << lane) - 1ull));
		if (lane == 0) {
			wave_count[wave] = __popcll(ballot);
		}
		__syncthreads();
		uint32_t wave_base = 0, total = 0;
#pragma unroll
		for (uint32_t w = 0; w < kWaves; w++) {
			const uint32_t c = wave_count[w];
			wave_base += (w < wave) ? c : 0;
			total += c;
		}
		const uint32_t pos = cursor + wave_base + lane_prefix;
		const uint32_t slot = pos & mask;

		uint64_t w[8];
		if (active) {
			make_desc(seed, ctx, i, peer_rank, signal_every, signal_op, aggregate_mask, w);
		}

		/* Wait for the consumer to have freed the wave's slots one lap ago.  The
		 * single consumer frees slots in position order, so the slot of the
		 * wave's highest position being free implies the others are: one lane
		 * polls one word instead of 64 lanes polling over the host link. */
		bool timed_out = false;
		if (ballot != 0) {
			const uint32_t last = 63u - (uint32_t)__clzll((long long)ballot);
			const uint32_t last_pos = __shfl(pos, last, 64);
			if (lane == 0) {
				uint64_t spins = 0;
				while (__hip_atomic_load(&seq[last_pos & mask], __ATOMIC_RELAXED,
							 __HIP_MEMORY_SCOPE_SYSTEM) != last_pos) {
					if (++spins > spin_limit) {
						timed_out = true;
						break;
					}
					__builtin_amdgcn_s_sleep(16);
				}
			}
		}
		if (__syncthreads_or(timed_out ? 1 : 0)) {
			if (threadIdx.x == 0) {
				atomicOr(status, ofi_amd::ASYNC_ERR_GIN_TIMEOUT);
			}
			return; /* every wave leaves here: the grid always drains */
		}
		__builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");

		/* stage: lane l holds record l of this wave */
		if (active) {
#pragma unroll
			for (uint32_t q = 0; q < 4; q++) {
				u32x4 v;
				v.x = (uint32_t)w[2 * q];
				v.y = (uint32_t)(w[2 * q] >> 32);
				v.z = (uint32_t)w[2 * q + 1];
				v.w = (uint32_t)(w[2 * q + 1] >> 32);
				stage[wave][lane * 4 + q] = v;
			}
		}
		__syncthreads();

		/* write-out: instruction q covers records 16q..16q+15 of the wave, 16 B per lane */
#pragma unroll
		for (uint32_t q = 0; q < 4; q++) {
			const uint32_t rec = q * 16 + (lane >> 2);
			const uint32_t part = lane & 3u;
			const uint32_t rec_pos = __shfl(pos, rec, 64);
			if ((ballot >> rec) & 1ull) {
				ring[(uint64_t)(rec_pos & mask) * 4 + part] = stage[wave][rec * 4 + part];
			}
		}

		/* publish */
		__builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
		if (active) {
			__hip_atomic_store(&seq[slot], pos + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
		}
		cursor += total;
		__syncthreads();
	}

	if (threadIdx.x == 0) {
		/* the free-slot horizon of the device-side put follows the cursor: every position
		 * this kernel filled was seen free first */
		__hip_atomic_store(&enqueue_pos[ctx * kGinReserveStride + 1], cursor, __ATOMIC_RELAXED,
				   __HIP_MEMORY_SCOPE_AGENT);
		__hip_atomic_store(&enqueue_pos[ctx * kGinReserveStride], cursor, __ATOMIC_RELEASE,
				   __HIP_MEMORY_SCOPE_AGENT);
	}
}

/* Multi-producer form: one wavefront per workgroup, `waves` of them per context, each putting
 * its share of a descriptor table through the device-side put. */
__global__ __launch_bounds__(64) void gin_produce_table_kernel(
	ofi_amd_gin_dev_ring_t first, const ofi_amd_gin_desc_t *__restrict__ table, uint64_t ops,
	uint32_t waves, uint64_t spin_limit)
{
	const uint32_t ctx = blockIdx.x / waves, g = blockIdx.x % waves;
	ofi_amd_gin_dev_ring_t ring = first; /* context 0; the arrays of context c follow at fixed strides */
	ring.records = static_cast<uint8_t *>(first.records) + (uint64_t)ctx * first.capacity * 64u;
	ring.sequences = first.sequences + (uint64_t)ctx * first.capacity;
	ring.reserve = first.reserve + (uint64_t)ctx * kGinReserveStride;
	ring.context = ctx;
	const ofi_amd_gin_desc_t *mine = table + (uint64_t)ctx * ops;
	for (uint64_t group = g; group * 64u < ops; group += waves) {
		const uint64_t i = group * 64u + threadIdx.x;
		const bool active = i < ops;
		const ofi_amd_gin_desc_t d = mine[active ? i : ops - 1];
		if (ofi_amd_gin_dev_put(ring, &d, active, spin_limit) != 0) {
			return; /* wave-uniform: the whole wave leaves */
		}
	}
}

} // namespace

using namespace ofi_amd;

extern "C" {

int ofi_amd_gin_rings_destroy(ofi_amd_gin_rings_t *r)
{
	if (!r) {
		return -EINVAL;
	}
	if (r->records) (void)hipHostFree(r->records);
	if (r->sequences) (void)hipHostFree(r->sequences);
	if (r->enqueue_pos) (void)hipHostFree(r->enqueue_pos);
	if (r->status) (void)hipHostFree(r->status);
	if (r->d_reserve) (void)hipFree(r->d_reserve);
	delete[] r->dequeue_pos;
	delete r;
	return 0;
}

int ofi_amd_gin_rings_create(uint32_t n_contexts, uint32_t capacity, ofi_amd_gin_rings_t **out)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!out || n_contexts == 0 || n_contexts > 65535 || capacity < 256 ||
	    (capacity & (capacity - 1)) != 0 || capacity > (1u << 24)) {
		return -EINVAL;
	}
	auto *r = new (std::nothrow) ofi_amd_gin_rings();
	if (!r) {
		return -ENOMEM;
	}
	std::memset(r, 0, sizeof(*r));
	r->n_contexts = n_contexts;
	r->capacity = capacity;
	const size_t slots = (size_t)n_contexts * capacity;
	const unsigned flags = hipHostMallocMapped | hipHostMallocCoherent;
	hipError_t e = hipHostMalloc((void **)&r->records, slots * sizeof(ofi_amd_gin_desc_t), flags);
	if (e == hipSuccess) e = hipHostMalloc((void **)&r->sequences, slots * sizeof(uint32_t), flags);
	if (e == hipSuccess) e = hipHostMalloc((void **)&r->enqueue_pos, (size_t)n_contexts * 64, flags);
	if (e == hipSuccess) e = hipHostMalloc((void **)&r->status, 64, flags);
	if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&r->d_records, r->records, 0);
	if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&r->d_sequences, r->sequences, 0);
	if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&r->d_enqueue_pos, r->enqueue_pos, 0);
	if (e == hipSuccess) e = hipHostGetDevicePointer((void **)&r->d_status, r->status, 0);
	const size_t reserve_bytes = (size_t)n_contexts * kGinReserveStride * sizeof(uint32_t);
	if (e == hipSuccess) e = hipMalloc((void **)&r->d_reserve, reserve_bytes);
	if (e == hipSuccess) e = hipMemset(r->d_reserve, 0, reserve_bytes);
	r->dequeue_pos = new (std::nothrow) uint32_t[n_contexts]();
	if (e != hipSuccess || !r->dequeue_pos) {
		ofi_amd_gin_rings_destroy(r);
		return e != hipSuccess ? errno_of(e) : -ENOMEM;
	}
	std::memset(r->records, 0, slots * sizeof(ofi_amd_gin_desc_t));
	std::memset(r->enqueue_pos, 0, (size_t)n_contexts * 64);
	std::memset(r->status, 0, 64);
	/* sequence of slot i starts at i (nccl_ofi_mpsc_ring ctor, :64-69) */
	for (uint32_t c = 0; c < n_contexts; c++) {
		for (uint32_t i = 0; i < capacity; i++) {
			r->sequences[(size_t)c * capacity + i] = i;
		}
	}
	__atomic_thread_fence(__ATOMIC_SEQ_CST);
	*out = r;
	return 0;
}

int ofi_amd_gin_rings_reset(ofi_amd_gin_rings_t *r, uint32_t context, uint64_t *dropped)
{
	if (!r || (context != OFI_AMD_GIN_ALL_CONTEXTS && context >= r->n_contexts)) {
		return -EINVAL;
	}
	const uint32_t first = context == OFI_AMD_GIN_ALL_CONTEXTS ? 0 : context;
	const uint32_t last = context == OFI_AMD_GIN_ALL_CONTEXTS ? r->n_contexts : context + 1;
	const uint32_t cap = r->capacity, mask = cap - 1;
	uint64_t lost = 0;
	for (uint32_t c = first; c < last; c++) {
		/* everything from the consumer's position on is handed back to the producers: slot of
		 * position p free for p, whatever a producer that gave up left in it */
		const uint32_t base = r->dequeue_pos[c];
		uint32_t *seq = r->sequences + (size_t)c * cap;
		for (uint32_t k = 0; k < cap; k++) {
			const uint32_t pos = base + k;
			if (seq[pos & mask] == pos + 1u) {
				lost++; /* published, never popped */
			}
			seq[pos & mask] = pos;
		}
		__atomic_store_n(&r->enqueue_pos[c * 16], base, __ATOMIC_RELAXED);
		/* cursor back to the consumer's position; every slot is free, so the horizon is a
		 * whole lap ahead and the next producers need not look over the host link */
		const uint32_t cursor[2] = { base, base + cap };
		OFI_AMD_HIP_TRY(hipMemcpy(r->d_reserve + (size_t)c * kGinReserveStride, cursor, sizeof(cursor),
					  hipMemcpyHostToDevice));
	}
	if (context == OFI_AMD_GIN_ALL_CONTEXTS) {
		__atomic_store_n(r->status, 0u, __ATOMIC_RELAXED);
	}
	__atomic_thread_fence(__ATOMIC_SEQ_CST);
	if (dropped) {
		*dropped = lost;
	}
	return 0;
}

int ofi_amd_gin_rings_view(ofi_amd_gin_rings_t *r, void **records, uint32_t **sequences,
			   uint32_t *n_contexts, uint32_t *capacity)
{
	if (!r) {
		return -EINVAL;
	}
	if (records) *records = r->records;
	if (sequences) *sequences = r->sequences;
	if (n_contexts) *n_contexts = r->n_contexts;
	if (capacity) *capacity = r->capacity;
	return 0;
}

int ofi_amd_gin_produce_seeded(ofi_amd_gin_rings_t *r, uint64_t seed, uint64_t ops_per_context,
			       uint32_t peer_rank, uint32_t signal_every, uint32_t signal_op,
			       uint32_t aggregate_mask, uint64_t spin_limit, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!r || signal_op > 2 || ops_per_context > (1ull << 38)) {
		return -EINVAL;
	}
	if (ops_per_context == 0) {
		return 0;
	}
	hipLaunchKernelGGL(gin_produce_seeded_kernel, dim3(r->n_contexts), dim3(kThreads), 0,
			   as_stream(stream), reinterpret_cast<u32x4 *>(r->d_records), r->d_sequences,
			   r->d_reserve, r->d_status, r->capacity, seed, ops_per_context, peer_rank,
			   signal_every, signal_op, aggregate_mask,
			   spin_limit ? spin_limit : kDefaultSpinLimit);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_gin_rings_device_view(ofi_amd_gin_rings_t *r, uint32_t context, ofi_amd_gin_dev_ring_t *out)
{
	if (!r || !out || context >= r->n_contexts) {
		return -EINVAL;
	}
	out->records = r->d_records + (size_t)context * r->capacity;
	out->sequences = r->d_sequences + (size_t)context * r->capacity;
	out->reserve = r->d_reserve + (size_t)context * kGinReserveStride;
	out->status = r->d_status;
	out->capacity = r->capacity;
	out->context = context;
	return 0;
}

int ofi_amd_gin_produce_table(ofi_amd_gin_rings_t *r, const ofi_amd_gin_desc_t *d_table,
			      uint64_t ops_per_context, uint32_t waves_per_context, uint64_t spin_limit,
			      void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!r || !d_table || waves_per_context < 1 || waves_per_context > 1024 ||
	    ops_per_context > (1ull << 38) || (uint64_t)r->n_contexts * waves_per_context > (1u << 30)) {
		return -EINVAL;
	}
	if (ops_per_context == 0) {
		return 0;
	}
	ofi_amd_gin_dev_ring_t first;
	rc = ofi_amd_gin_rings_device_view(r, 0, &first);
	if (rc != 0) {
		return rc;
	}
	hipLaunchKernelGGL(gin_produce_table_kernel, dim3(r->n_contexts * waves_per_context), dim3(64), 0,
			   as_stream(stream), first, d_table, ops_per_context, waves_per_context,
			   spin_limit ? spin_limit : kDefaultSpinLimit);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_gin_producer_status(ofi_amd_gin_rings_t *r)
{
	if (!r) {
		return -EINVAL;
	}
	uint32_t bits = __atomic_load_n(r->status, __ATOMIC_ACQUIRE);
	return (bits & ASYNC_ERR_GIN_TIMEOUT) ? -ETIMEDOUT : 0;
}

} /* extern "C" */

/*
 * Batched rail striping (threshold scheduler) for gfx950.
 *
 * The reference schedules one message per call on a stateful object: messages
 * below max_small_msg_size take one rail from rr_small_counter, larger ones take
 * get_num_stripes(size) consecutive rails starting at rr_counter; both counters
 * advance modulo num_rails (src/nccl_ofi_scheduler.cpp:47-133).  For a batch in
 * index order that is two exclusive prefix sums:
 *
 *   small_rail_i = (rr_small + #{j < i : size_j <  max_small}) mod R
 *   start_rail_i = (rr      + sum{j < i : size_j >= max_small} n_j) mod R
 *
 * Launches on one stream:
 *   1. stripe_count_kernel  per-tile totals of (small count, stripe count), each
 *                           reduced mod R (only the residues matter); snapshots the
 *                           two counters of *state as the batch's seed
 *   2. stripe_scan_kernel   (batches of more than kInlineTiles tiles only) one
 *                           workgroup scans the tile totals and writes the new
 *                           counters back
 *   3. stripe_emit_kernel   re-reads the tile, scans inside the workgroup with
 *                           wavefront shuffles, builds the 96-byte stripe rows in
 *                           LDS and writes them out as coalesced 16-byte stores.
 *                           Up to kInlineTiles tiles every workgroup sums the
 *                           totals of the tiles before it by itself (at most 16 KiB
 *                           from L2) instead of waiting for a scan launch, and the
 *                           last workgroup writes the new counters back.
 * A tile is 512 messages for batches up to 2^21 messages and 1024 beyond.
 *
 * HBM traffic per message: 8 B read twice + 4 B + 96 B written.
 */
#include <mutex>
#include <unordered_map>

#include "common.hpp"
#include "ofi_amd_hotpath.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kThreads = 256;
/* Messages per workgroup = kThreads * PASSES.  Small batches want many small tiles (the
 * launch is short, so ramp-up and tail dominate: 1,000,000 messages take 22.2 us with two
 * passes per workgroup against 24.4 with four); large ones want somewhat longer workgroups
 * (16,000,000: 322-325 us with three or four passes, 332-334 with two, six or eight). */
#ifndef OFI_STRIPE_PASSES_SMALL
#define OFI_STRIPE_PASSES_SMALL 2
#endif
#ifndef OFI_STRIPE_PASSES_LARGE
#define OFI_STRIPE_PASSES_LARGE 4
#endif
constexpr uint32_t kPassesSmall = OFI_STRIPE_PASSES_SMALL, kPassesLarge = OFI_STRIPE_PASSES_LARGE;
constexpr uint64_t kSmallBatch = 1ull << 21;
constexpr uint32_t kScanThreads = 1024;
constexpr uint32_t kScanPer = 8; /* tiles per thread and round of the scan kernel */
constexpr uint64_t kMaxBatch = 1ull << 28;
/* residues are < 4, so packed 16-bit sums over this many tiles cannot overflow */
#ifndef OFI_STRIPE_INLINE_TILES
#define OFI_STRIPE_INLINE_TILES 4096
#endif
constexpr uint32_t kInlineTiles = OFI_STRIPE_INLINE_TILES;
#ifndef OFI_STRIPE_NT_STORES
#define OFI_STRIPE_NT_STORES 1
#endif

struct params_t {
	uint64_t max_small;
	uint64_t min_stripe;
	uint64_t align;
	int32_t min_stripe_shift; /* log2 when a power of two, else -1 */
	int32_t align_shift;
	uint32_t num_rails;
	uint32_t stripe_counts; /* get_num_stripes for this rail count, 4 bits per requested count 1..4 */
	uint32_t mod_magic;     /* 65536 / num_rails + 1, see mod_rails */
};

__device__ __forceinline__ uint64_t div_by(uint64_t x, uint64_t d, int32_t shift)
{
	return shift >= 0 ? (x >> shift) : (x / d);
}

/* NCCL_OFI_DIV_CEIL, include/nccl_ofi_math.h:23-26 */
__device__ __forceinline__ uint64_t div_ceil_by(uint64_t x, uint64_t d, int32_t shift)
{
	return x == 0 ? 0 : 1 + div_by(x - 1, d, shift);
}

/* get_num_stripes, src/nccl_ofi_scheduler.cpp:47-64: the request, capped to the rail count,
 * goes down to the largest count >= 2 that divides the rail count and stays as it is when there
 * is none (3 rails: 2 stays 2).  At most 4 rails, so the loop is a 16-entry table. */
constexpr uint64_t kStripeCounts = 0x4221332122211111ull; /* 16 bits per rail count, 4 per request */

__device__ __forceinline__ uint32_t num_stripes(uint64_t size, const params_t &p)
{
	uint64_t want = div_ceil_by(size, p.min_stripe, p.min_stripe_shift);
	uint32_t n = (uint32_t)(want < p.num_rails ? want : p.num_rails);
	n = n > 1 ? n : 1;
	return (p.stripe_counts >> (4u * (n - 1u))) & 7u;
}

/* x mod num_rails for x < 16384, by multiply and shift (checked exhaustively for 1..4 rails) */
__device__ __forceinline__ uint32_t mod_rails(uint32_t x, const params_t &p)
{
	return x - p.num_rails * ((x * p.mod_magic) >> 16);
}

/* Thresholds come from the device-resident state; a power-of-two divisor becomes a
 * shift.  False when the state is unusable (rails outside 1..4, zero stripe size). */
__device__ __forceinline__ int32_t log2_if_pow2_dev(uint64_t v)
{
	return (v != 0 && (v & (v - 1)) == 0) ? (int32_t)(__ffsll((unsigned long long)v) - 1) : -1;
}

__device__ __forceinline__ bool load_params(const ofi_amd_sched_state_t *st, uint64_t align,
					    params_t &p)
{
	p.max_small = st->max_small_msg_size;
	p.min_stripe = st->min_stripe_size;
	p.align = align;
	p.min_stripe_shift = log2_if_pow2_dev(p.min_stripe);
	p.align_shift = log2_if_pow2_dev(align);
	p.num_rails = (uint32_t)st->num_rails;
	p.stripe_counts = (uint32_t)(kStripeCounts >> (16u * ((p.num_rails - 1u) & 3u))) & 0xffffu;
	p.mod_magic = 65536u / (p.num_rails ? p.num_rails : 1u) + 1u;
	return st->num_rails >= 1 && st->num_rails <= OFI_AMD_MAX_NUM_RAILS && p.min_stripe != 0;
}

/* packed (small count << 16 | stripe count) contribution of one message */
__device__ __forceinline__ uint32_t contribution(uint64_t size, const params_t &p, uint32_t &n_out)
{
	if (size < p.max_small) {
		n_out = 1;
		return 1u << 16;
	}
	n_out = num_stripes(size, p);
	return n_out;
}

/* Inclusive sum over the 64 lanes with lane-to-lane moves inside the vector unit: shifts by 1,
 * 2, 4 and 8 lanes within each row of 16 (a lane shifted in from outside the row reads 0), then
 * lane 15 of rows 0 and 2 added to rows 1 and 3, then lane 31 added to rows 2 and 3. */
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v, uint32_t)
{
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false); /* row_shr:1 */
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false); /* row_shr:2 */
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false); /* row_shr:4 */
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false); /* row_shr:8 */
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false); /* row_bcast:15 */
	v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false); /* row_bcast:31 */
	return v;
}

/* Which tile a workgroup takes.  Workgroups are dealt to the 8 XCDs in turn; with tile =
 * workgroup number every XCD writes one tile's rows (96 KiB) out of every eight, with runs of
 * 16 consecutive tiles per XCD each of them writes 1.5 MiB at a stretch.  Once the output no
 * longer fits the last-level cache the longer stretches are faster (5,000,000 messages: 110.6 ->
 * 102.9 us, 16,000,000: 324.6 -> 305.9 us; runs of 4, 64, 256 or an eighth of the batch per XCD:
 * 307-312 us), below that they are slower (1,000,000: 22.4 -> 24.1 us, 4,200,000: 91.3 -> 97.0
 * us), so they are used from 4.5 Mi messages on.  The grid is rounded up to whole rounds; a
 * workgroup whose tile does not exist leaves at once. */
constexpr uint32_t kXcdRunShift = 4;
constexpr uint64_t kXcdRunBatch = 9ull << 19;
__device__ __forceinline__ uint32_t tile_of_workgroup(uint32_t wg, uint32_t run_shift)
{
	/* XCDs take runs of 2^run_shift consecutive tiles in turn */
	const uint32_t x = wg & 7u, t = wg >> 3;
	return ((((t >> run_shift) << 3) + x) << run_shift) + (t & ((1u << run_shift) - 1u));
}

template <uint32_t PASSES>
__global__ __launch_bounds__(kThreads) void stripe_count_kernel(
	const uint64_t *__restrict__ sizes, uint32_t n, const ofi_amd_sched_state_t *__restrict__ state,
	uint64_t align, uint32_t *__restrict__ tile_totals, uint32_t *__restrict__ seed0,
	uint32_t *__restrict__ err)
{
	__shared__ uint32_t wave_sum[kThreads / 64];
	/* the tile's sizes are requested before anything waits for the state, so a workgroup pays
	 * one memory latency, not two */
	const uint32_t base = blockIdx.x * (kThreads * PASSES);
	uint64_t size_of[PASSES];
#pragma unroll
	for (uint32_t pass = 0; pass < PASSES; pass++) {
		const uint32_t i = base + pass * kThreads + threadIdx.x;
		size_of[pass] = i < n ? sizes[i] : 0;
	}
	params_t p;
	if (!load_params(state, align, p)) {
		if (blockIdx.x == 0 && threadIdx.x == 0) {
			atomicOr(err, ofi_amd::ASYNC_ERR_SCHED_STATE);
		}
		return;
	}
	if (blockIdx.x == 0 && threadIdx.x == 0) {
		*seed0 = ((state->rr_small_counter % p.num_rails) << 16) | (state->rr_counter % p.num_rails);
	}
	uint32_t acc = 0;
#pragma unroll
	for (uint32_t pass = 0; pass < PASSES; pass++) {
		uint32_t k;
		const uint32_t c = contribution(size_of[pass], p, k);
		acc += base + pass * kThreads + threadIdx.x < n ? c : 0u;
	}
#pragma unroll
	for (uint32_t d = 32; d > 0; d >>= 1) {
		acc += __shfl_xor(acc, d, 64);
	}
	if ((threadIdx.x & 63u) == 0) {
		wave_sum[threadIdx.x >> 6] = acc;
	}
	__syncthreads();
	if (threadIdx.x == 0) {
		const uint32_t t = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
		tile_totals[blockIdx.x] = (((t >> 16) % p.num_rails) << 16) | ((t & 0xffffu) % p.num_rails);
	}
}

/* One workgroup: exclusive scan of the tile totals.  tile_prefix[t] holds the two
 * rail seeds of tile t (already reduced mod R); *state gets the final counters. */
__global__ __launch_bounds__(kScanThreads) void stripe_scan_kernel(
	const uint32_t *__restrict__ tile_totals, uint32_t num_tiles,
	ofi_amd_sched_state_t *__restrict__ state, uint32_t *__restrict__ tile_prefix,
	uint32_t *__restrict__ err)
{
	__shared__ uint32_t wave_small[kScanThreads / 64];
	__shared__ uint32_t wave_big[kScanThreads / 64];
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	if (state->num_rails < 1 || state->num_rails > OFI_AMD_MAX_NUM_RAILS ||
	    state->min_stripe_size == 0) {
		if (threadIdx.x == 0) {
			atomicOr(err, ofi_amd::ASYNC_ERR_SCHED_STATE);
		}
		return;
	}
	const uint32_t num_rails = (uint32_t)state->num_rails;
	/* totals can reach 2^28 each, so the two sums are scanned unpacked */
	uint32_t carry_small = state->rr_small_counter % num_rails;
	uint32_t carry_big = state->rr_counter % num_rails;

	/* eight consecutive tiles per thread and round: 16 M messages are one round, so the kernel
	 * waits for memory once */
	for (uint32_t start = 0; start < num_tiles; start += kScanThreads * kScanPer) {
		const uint32_t t0 = start + threadIdx.x * kScanPer;
		const bool whole = t0 + kScanPer <= num_tiles;
		uint32_t v[kScanPer];
		if (whole) {
			const u32x4 lo = *reinterpret_cast<const u32x4 *>(tile_totals + t0);
			const u32x4 hi = *reinterpret_cast<const u32x4 *>(tile_totals + t0 + 4);
			v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
			v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
		} else {
#pragma unroll
			for (uint32_t j = 0; j < kScanPer; j++) {
				v[j] = t0 + j < num_tiles ? tile_totals[t0 + j] : 0;
			}
		}
		uint32_t s = 0, b = 0;
#pragma unroll
		for (uint32_t j = 0; j < kScanPer; j++) {
			s += v[j] >> 16;
			b += v[j] & 0xffffu;
		}
		uint32_t inc_s = wave_inclusive_scan(s, lane);
		uint32_t inc_b = wave_inclusive_scan(b, lane);
		if (lane == 63) {
			wave_small[wave] = inc_s;
			wave_big[wave] = inc_b;
		}
		__syncthreads();
		uint32_t off_s = 0, off_b = 0, tot_s = 0, tot_b = 0;
		for (uint32_t w = 0; w < kScanThreads / 64; w++) {
			uint32_t ws = wave_small[w], wb = wave_big[w];
			if (w < wave) {
				off_s += ws;
				off_b += wb;
			}
			tot_s += ws;
			tot_b += wb;
		}
		uint32_t run_s = carry_small + off_s + inc_s - s;
		uint32_t run_b = carry_big + off_b + inc_b - b;
		uint32_t out[kScanPer];
#pragma unroll
		for (uint32_t j = 0; j < kScanPer; j++) {
			out[j] = ((run_s % num_rails) << 16) | (run_b % num_rails);
			run_s += v[j] >> 16;
			run_b += v[j] & 0xffffu;
		}
		if (whole) {
			*reinterpret_cast<u32x4 *>(tile_prefix + t0) = u32x4{ out[0], out[1], out[2], out[3] };
			*reinterpret_cast<u32x4 *>(tile_prefix + t0 + 4) = u32x4{ out[4], out[5], out[6], out[7] };
		} else {
#pragma unroll
			for (uint32_t j = 0; j < kScanPer; j++) {
				if (t0 + j < num_tiles) {
					tile_prefix[t0 + j] = out[j];
				}
			}
		}
		carry_small = (carry_small + tot_s) % num_rails;
		carry_big = (carry_big + tot_b) % num_rails;
		__syncthreads();
	}
	if (threadIdx.x == 0) {
		state->rr_small_counter = carry_small;
		state->rr_counter = carry_big;
	}
}

/* INLINE: tile_prefix holds the per-tile totals (residues) and *seed0 the batch's seed;
 * otherwise tile_prefix holds each tile's finished seed. */
template <bool INLINE, uint32_t PASSES>
__global__ __launch_bounds__(kThreads) void stripe_emit_kernel(
	const uint64_t *__restrict__ sizes, uint32_t n, ofi_amd_sched_state_t *__restrict__ state,
	uint64_t align, const uint32_t *__restrict__ tile_prefix, const uint32_t *__restrict__ seed0,
	uint32_t num_tiles, uint32_t xcd_run_shift, uint32_t *__restrict__ num_xfers, u32x4 *__restrict__ xfers)
{
	/* 256 rows of 96 bytes = 6 x 16 B each */
	__shared__ u32x4 rows[kThreads * 6];
	__shared__ uint32_t wave_sum[kThreads / 64];
	const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
	const uint32_t tile = tile_of_workgroup(blockIdx.x, xcd_run_shift);
	if (tile >= num_tiles) {
		return;
	}
	const uint32_t base = tile * (kThreads * PASSES);
	/* every pass's size is requested up front: the passes below then run out of registers
	 * instead of each waiting for its own load */
	uint64_t size_of[PASSES];
#pragma unroll
	for (uint32_t pass = 0; pass < PASSES; pass++) {
		const uint32_t i = base + pass * kThreads + threadIdx.x;
		size_of[pass] = i < n ? __builtin_nontemporal_load(&sizes[i]) : 0;
	}
	params_t p;
	if (!load_params(state, align, p)) {
		return;
	}
	const uint32_t R = p.num_rails;

	uint32_t seed;
	if (INLINE) {
		/* sum of the totals of the tiles before this one (packed halves, no overflow) */
		uint32_t acc = 0;
		for (uint32_t t = threadIdx.x; t < tile; t += kThreads) {
			acc += tile_prefix[t];
		}
#pragma unroll
		for (uint32_t d = 32; d > 0; d >>= 1) {
			acc += __shfl_xor(acc, d, 64);
		}
		if (lane == 0) {
			wave_sum[wave] = acc;
		}
		__syncthreads();
		acc = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3] + *seed0;
		__syncthreads();
		seed = (((acc >> 16) % R) << 16) | ((acc & 0xffffu) % R);
	} else {
		seed = tile_prefix[tile];
	}
	uint32_t carry_small = seed >> 16, carry_big = seed & 0xffffu; /* both < R */

#pragma unroll
	for (uint32_t pass = 0; pass < PASSES; pass++) {
		const uint32_t first = base + pass * kThreads;
		if (first >= n) {
			break;
		}
		const uint32_t i = first + threadIdx.x;
		const bool live = i < n;
		const uint64_t size = size_of[pass];
		uint32_t k = 0;
		const uint32_t c = live ? contribution(size, p, k) : 0;

		uint32_t inc = wave_inclusive_scan(c, lane);
		if (lane == 63) {
			wave_sum[wave] = inc;
		}
		__syncthreads();
		uint32_t off = 0, tot = 0;
#pragma unroll
		for (uint32_t w = 0; w < kThreads / 64; w++) {
			uint32_t ws = wave_sum[w];
			off += (w < wave) ? ws : 0;
			tot += ws;
		}
		const uint32_t excl = off + inc - c;

		/* set_schedule_by_threshold, src/nccl_ofi_scheduler.cpp:77-133 */
		const bool small = (c >> 16) != 0;
		uint32_t rail = mod_rails(small ? carry_small + (excl >> 16) : carry_big + (excl & 0xffffu), p);
		uint64_t max_stripe = size;
		if (!small) {
			/* (size - 1) / k: k is 1, 2 or 4 unless there are three rails */
			uint64_t whole = size == 0 ? 0 : (size - 1) >> (k >> 1);
			if (R == 3) {
				whole = k == 3 ? (size == 0 ? 0 : (size - 1) / 3) : whole;
			}
			const uint64_t per = size == 0 ? 0 : 1 + whole;
			max_stripe = div_ceil_by(per, p.align, p.align_shift) * p.align;
		}
		/* k stripes of max_stripe cover the message, so `left` is 0 from stripe k on and the
		 * length of an unused entry comes out as 0 by itself; lanes past the end have k = 0 */
		uint64_t left = size, offset = 0;
		u32x4 *row = &rows[threadIdx.x * 6];
		uint64_t f[12]; /* 4 x {rail word, offset, msg_size} */
#pragma unroll
		for (uint32_t s = 0; s < 4; s++) {
			const bool used = s < k;
			const uint64_t stripe = left < max_stripe ? left : max_stripe;
			f[3 * s + 0] = used ? rail : 0; /* rail_id in the low 16 bits, padding zero */
			f[3 * s + 1] = used ? offset : 0;
			f[3 * s + 2] = stripe;
			offset += stripe;
			left -= stripe;
			rail = rail + 1 == R ? 0 : rail + 1;
		}
#pragma unroll
		for (uint32_t q = 0; q < 6; q++) {
			u32x4 v;
			v.x = (uint32_t)f[2 * q];
			v.y = (uint32_t)(f[2 * q] >> 32);
			v.z = (uint32_t)f[2 * q + 1];
			v.w = (uint32_t)(f[2 * q + 1] >> 32);
			row[q] = v;
		}
		if (live) {
			num_xfers[i] = k;
		}
		__syncthreads();

		/* coalesced write-out of the tile's rows */
		const uint32_t valid = (n - first) < kThreads ? (n - first) : kThreads;
		u32x4 *out = xfers + (uint64_t)first * 6;
		for (uint32_t v = threadIdx.x; v < valid * 6; v += kThreads) {
#if OFI_STRIPE_NT_STORES
			__builtin_nontemporal_store(rows[v], &out[v]);
#else
			out[v] = rows[v];
#endif
		}

		carry_small = mod_rails(carry_small + (tot >> 16), p);
		carry_big = mod_rails(carry_big + (tot & 0xffffu), p);
		__syncthreads();
	}
	if (INLINE && tile == num_tiles - 1 && threadIdx.x == 0) {
		/* the carries after the last tile are the counters the next batch starts from;
		 * nobody reads them any more in this launch (the seed was snapshotted) */
		state->rr_small_counter = carry_small;
		state->rr_counter = carry_big;
	}
}

/* Scratch for tile totals / prefixes, one per stream (launches on one stream are ordered, so
 * they can share; launches on different streams may overlap and must not), grown on demand. */
struct workspace_t {
	uint32_t *totals = nullptr;
	uint32_t *prefix = nullptr; /* prefix[capacity] is the seed word */
	uint32_t tiles = 0;
};
std::mutex g_ws_lock;
std::unordered_map<void *, workspace_t> g_ws_by_stream;

/*
 * The same scratch for callers that may not allocate: one array per GPU, part of the loaded
 * code object, held until the process ends.  Layout in 32-bit words:
 * [0, kNoAllocTiles) tile totals, [kNoAllocTiles, 2 * kNoAllocTiles) tile prefixes, then the
 * seed word.  kNoAllocMaxBatch messages need kNoAllocTiles tiles of 1024.  In host code the
 * array's name is only a handle for hipGetSymbolAddress; kernels get the address it returns.
 */
constexpr uint64_t kNoAllocMaxBatch = 1ull << 26;
constexpr uint32_t kNoAllocTiles = (uint32_t)(kNoAllocMaxBatch / (kThreads * kPassesLarge));
static_assert(kNoAllocTiles >= kInlineTiles, "small batches use up to kInlineTiles tiles of 512");
static __device__ __align__(256) __attribute__((used)) uint32_t scratch[2 * kNoAllocTiles + 64];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
uint32_t *g_scratch_ptr[kMaxDevices]; /* device address of `scratch` on each GPU, once looked up */

/* Device address of the current GPU's copy of `scratch` as ofi_amd_gpu_init() has recorded it;
 * no runtime call that could allocate.  -ENXIO when the address has not been looked up. */
int cached_scratch_of_current_device(uint32_t **out)
{
	int dev = -1;
	OFI_AMD_HIP_TRY(hipGetDevice(&dev));
	if (dev < 0 || dev >= kMaxDevices) {
		return -ENODEV;
	}
	std::lock_guard<std::mutex> g(g_scratch_lock);
	if (!g_scratch_ptr[dev]) {
		return -ENXIO;
	}
	*out = g_scratch_ptr[dev];
	return 0;
}

/* Device address of the current GPU's copy of `scratch` (each GPU has its own), looked up on
 * first use: set-up only. */
int scratch_of_current_device(uint32_t **out)
{
	int dev = -1;
	OFI_AMD_HIP_TRY(hipGetDevice(&dev));
	if (dev < 0 || dev >= kMaxDevices) {
		return -ENODEV;
	}
	std::lock_guard<std::mutex> g(g_scratch_lock);
	if (!g_scratch_ptr[dev]) {
		void *p = nullptr;
		OFI_AMD_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
		if (!p) {
			return -EIO;
		}
		g_scratch_ptr[dev] = static_cast<uint32_t *>(p);
	}
	*out = g_scratch_ptr[dev];
	return 0;
}

uint32_t pick_passes(uint64_t n)
{
	return n <= kSmallBatch ? kPassesSmall : kPassesLarge;
}

template <uint32_t PASSES>
void launch_batch(hipStream_t s, uint32_t tiles, const uint64_t *d_sizes, uint32_t n,
		  ofi_amd_sched_state_t *d_state, uint64_t align, uint32_t *totals, uint32_t *prefix,
		  uint32_t *seed0, uint32_t *d_num_xfers, u32x4 *d_xfers, uint32_t *err)
{
	hipLaunchKernelGGL(stripe_count_kernel<PASSES>, dim3(tiles), dim3(kThreads), 0, s, d_sizes, n, d_state,
			   align, totals, seed0, err);
	const uint32_t xcd_run_shift = n >= kXcdRunBatch ? kXcdRunShift : 0u;
	const uint32_t xcd_run = 1u << xcd_run_shift;
	const uint32_t emit_grid = (tiles + 8u * xcd_run - 1u) / (8u * xcd_run) * (8u * xcd_run);
	if (tiles <= kInlineTiles) {
		hipLaunchKernelGGL((stripe_emit_kernel<true, PASSES>), dim3(emit_grid), dim3(kThreads), 0, s, d_sizes, n,
				   d_state, align, totals, seed0, tiles, xcd_run_shift, d_num_xfers, d_xfers);
	} else {
		hipLaunchKernelGGL(stripe_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, totals, tiles, d_state,
				   prefix, err);
		hipLaunchKernelGGL((stripe_emit_kernel<false, PASSES>), dim3(emit_grid), dim3(kThreads), 0, s, d_sizes, n,
				   d_state, align, prefix, seed0, tiles, xcd_run_shift, d_num_xfers, d_xfers);
	}
}

} // namespace

namespace ofi_amd {

int sched_noalloc_setup()
{
	int count = 0, before = -1;
	OFI_AMD_HIP_TRY(hipGetDeviceCount(&count));
	OFI_AMD_HIP_TRY(hipGetDevice(&before));
	int rc = 0;
	for (int dev = 0; dev < count && dev < kMaxDevices && rc == 0; dev++) {
		uint32_t *p = nullptr;
		if (hipSetDevice(dev) != hipSuccess) {
			rc = -ENODEV;
			break;
		}
		rc = scratch_of_current_device(&p);
	}
	(void)hipSetDevice(before);
	return rc;
}

} // namespace ofi_amd

using namespace ofi_amd;

extern "C" {

int ofi_amd_sched_batch(ofi_amd_sched_state_t *d_state, const uint64_t *d_sizes, uint64_t n,
			uint64_t align, uint32_t *d_num_xfers, ofi_amd_xfer_info_t *d_xfers,
			void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!d_state || align == 0 || n > kMaxBatch) {
		return -EINVAL;
	}
	if (n == 0) {
		return 0;
	}
	if (!d_sizes || !d_num_xfers || !d_xfers) {
		return -EINVAL;
	}

	uint32_t *err = async_error_word();
	if (!err) {
		return -ENOMEM;
	}

	const uint32_t passes = pick_passes(n);
	const uint32_t tiles = (uint32_t)((n + kThreads * passes - 1) / (kThreads * passes));
	hipStream_t s = as_stream(stream);
	try {
		/* held until the launches are queued: two threads submitting to one stream share its
		 * scratch, and their count/emit pairs must not interleave */
		std::lock_guard<std::mutex> g(g_ws_lock);
		workspace_t &ws = g_ws_by_stream[stream];
		if (tiles > ws.tiles) {
			uint32_t want = tiles < 4096 ? 4096 : tiles;
			uint32_t *a = nullptr, *b = nullptr;
			OFI_AMD_HIP_TRY(hipMalloc((void **)&a, sizeof(uint32_t) * want));
			if (hipMalloc((void **)&b, sizeof(uint32_t) * (want + 1)) != hipSuccess) {
				(void)hipFree(a);
				return -ENOMEM;
			}
			/* the older buffers may still be in use by launches queued on this stream */
			(void)hipStreamSynchronize(s);
			(void)hipFree(ws.totals);
			(void)hipFree(ws.prefix);
			ws.totals = a;
			ws.prefix = b;
			ws.tiles = want;
		}
		uint32_t *seed0 = ws.prefix + ws.tiles;
		if (passes == kPassesSmall) {
			launch_batch<kPassesSmall>(s, tiles, d_sizes, (uint32_t)n, d_state, align, ws.totals, ws.prefix,
						   seed0, d_num_xfers, reinterpret_cast<u32x4 *>(d_xfers), err);
		} else {
			launch_batch<kPassesLarge>(s, tiles, d_sizes, (uint32_t)n, d_state, align, ws.totals, ws.prefix,
						   seed0, d_num_xfers, reinterpret_cast<u32x4 *>(d_xfers), err);
		}
	} catch (...) {
		return -ENOMEM;
	}
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_sched_stream_release(void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	workspace_t ws;
	{
		std::lock_guard<std::mutex> g(g_ws_lock);
		auto it = g_ws_by_stream.find(stream);
		if (it == g_ws_by_stream.end()) {
			return 0; /* nothing was ever allocated for it */
		}
		ws = it->second;
		g_ws_by_stream.erase(it);
	}
	/* launches queued on the stream may still read the scratch */
	OFI_AMD_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
	(void)hipFree(ws.totals);
	(void)hipFree(ws.prefix);
	return 0;
}

int ofi_amd_sched_batch_noalloc(ofi_amd_sched_state_t *d_state, const uint64_t *d_sizes, uint64_t n,
				uint64_t align, uint32_t *d_num_xfers, ofi_amd_xfer_info_t *d_xfers,
				void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!d_state || align == 0) {
		return -EINVAL;
	}
	if (n > kNoAllocMaxBatch) {
		return -E2BIG; /* more messages than the fixed scratch has tiles for */
	}
	if (n == 0) {
		return 0;
	}
	if (!d_sizes || !d_num_xfers || !d_xfers) {
		return -EINVAL;
	}
	uint32_t *err = async_error_word_if_ready();
	if (!err) {
		return -ENXIO; /* ofi_amd_gpu_init() allocates it; this call must not */
	}
	uint32_t *base = nullptr;
	rc = cached_scratch_of_current_device(&base); /* -ENXIO: ofi_amd_gpu_init() looks the address up; this call must not */
	if (rc != 0) {
		return rc;
	}
	uint32_t *totals = base, *prefix = base + kNoAllocTiles, *seed0 = base + 2 * kNoAllocTiles;

	const uint32_t passes = pick_passes(n);
	const uint32_t tiles = (uint32_t)((n + kThreads * passes - 1) / (kThreads * passes));
	hipStream_t s = as_stream(stream);
	if (passes == kPassesSmall) {
		launch_batch<kPassesSmall>(s, tiles, d_sizes, (uint32_t)n, d_state, align, totals, prefix, seed0,
					   d_num_xfers, reinterpret_cast<u32x4 *>(d_xfers), err);
	} else {
		launch_batch<kPassesLarge>(s, tiles, d_sizes, (uint32_t)n, d_state, align, totals, prefix, seed0,
					   d_num_xfers, reinterpret_cast<u32x4 *>(d_xfers), err);
	}
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

} /* extern "C" */

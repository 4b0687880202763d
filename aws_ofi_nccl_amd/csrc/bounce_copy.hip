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
 * 8 KiB (the eager limit) per trip as rows of 1 KiB: all loads of a trip are
 * issued before its first store, so the whole buffer is in flight at once
 * whatever its length.  The table entry of the buffer is wave-uniform and is
 * read through the scalar cache.
 *
 * Every trip is straight-line code.  The number of rows a buffer needs is
 * wave-uniform, so the body is picked by a scalar switch over 1..8 rows, the
 * lanes past the end of the (possibly partial) last row are clamped to the last
 * valid word instead of being predicated: they copy that word again, the same
 * bytes to the same place, and likewise for the sub-16-byte tail.
 * Loads and stores share one in-order counter (vmcnt) on this ISA; with
 * per-load predication the compiler cannot count across the branches and falls
 * back to waiting for *everything* before each store, which serialises the
 * stores of a wave (measured: 5.2 TB/s against 7.1 TB/s for the same traffic).
 *
 * The packed source can start at any byte.  16-byte loads from a 4-byte-aligned
 * address run at full rate on gfx950, loads from an odd byte address do not
 * (measured: about 15 % slower), so a source that is not 4-byte aligned is read
 * as aligned dwords -- four plus the one that follows -- and each output dword
 * is cut out of two neighbours with v_alignbyte_b32.  The fifth dword is the
 * next lane's first, so it travels between lanes (one wave-wide DPP shift per
 * row; lane 63 takes lane 0 of the next row) rather than through a second load
 * instruction over the same cache lines; only the last row of a trip, whose
 * lanes may be clamped, loads it (94.4 -> 91.8 us on the configured batch: the
 * texture-address unit is busy 74 % of the kernel's time).  That dword always
 * contains at least one byte of the buffer, so nothing beyond the dword that
 * holds the last source byte is read.  The rows cover whole 64-byte units of the
 * destination; what is left of the buffer (up to 63 bytes) goes out as single
 * bytes, one per lane, so that nothing outside [dst, dst+len) is written and the
 * last, partial unit is written by one instruction.
 *
 * Flush: the wave waits until its own stores have left the CU (they are
 * write-through to the L2 of its XCD), then lane 0 re-reads the first 4 bytes
 * of the destination from that L2 and writes them to d_flush[i].  No wider
 * fence is used: on a multi-XCD part a device-scope release per buffer would
 * write back the whole L2 each time; device-wide visibility of the copied
 * bytes comes with the end of the kernel, as for any other kernel output.
 */
#include <cstring>
#include <new>

#include <immintrin.h>
#include <sys/mman.h>
#include <unistd.h>

#include "common.hpp"
#include "ofi_amd_hotpath.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
/* 16 bytes at a 4-byte-aligned address */
struct __attribute__((packed, aligned(4))) dword_aligned_u32x4 {
	u32x4 v;
};

/* Buffers (= wavefronts) per workgroup and consecutive workgroups that share an XCD, swept over
 * thousands of launches in a row on 65,536 buffers.  Bounce copy: 8 wavefronts per workgroup with
 * runs of 4 workgroups (32 buffers) per XCD was the fastest (91.1 us per launch; 4 x 8: 91.8,
 * 2 x 16: 92.5, 16 x 2: 92.6, 8 x 8: 91.7).  The eager copy, whose sources are rx buffers in
 * arrival order, prefers single-wavefront workgroups (1 x 32: 97.8 us, 4 x 8: 98.4, 8 x 4: 101.6,
 * 16 x 2: 108.6), and so does the table copy (1: 419.9 us per GiB, 4: 439.5, 8: 430.3). */
constexpr int kWavesPerBlock = 8;
constexpr int kBlock = 64 * kWavesPerBlock;
constexpr uint32_t kGroup = 4;
constexpr int kEagerWaves = 1;
constexpr uint32_t kEagerGroup = 32;
constexpr int kTableWaves = 1;
constexpr uint32_t kXcds = 8;
constexpr uint32_t kRows = 8;              /* rows of 64 x 16 bytes per trip: 8 KiB per wave */
constexpr uint32_t kTripVec = kRows * 64u; /* 16-byte words per trip */

__device__ __forceinline__ u32x4 load16_dword_aligned(const uint8_t *p)
{
	return reinterpret_cast<const dword_aligned_u32x4 *>(p)->v;
}

/*
 * Every access to a destination carries the same cache policy, the streaming one: the 16-byte
 * stores of the rows, the single head and tail bytes and the read-back of the flush.  With the
 * rows streaming and the tail bytes and the read-back as ordinary accesses, the same batch
 * launched over and over on the same buffers slowed down by 6 % within 2,000 launches (91 ->
 * 97 us; fewer and fewer of those ordinary lines leave the L2 between launches, and a read
 * sweep of 16 MiB of other memory brought the first rate back); with one policy the rate does
 * not move (91 us from the first launch to the 20,000th).
 */
__device__ __forceinline__ void store_byte_streaming(uint8_t *p, uint8_t v)
{
	__builtin_nontemporal_store(v, p);
}

/*
 * One trip: R rows from s (4-byte aligned; the data starts `shift` bytes in) to d (16-byte
 * aligned).  nvec = 16-byte words left, 64*(R-1) < nvec <= 64*R unless FULL, where all R rows
 * are complete.  SHIFTED = false: shift is 0 and the source words are used as they are.
 */
template <int R, bool SHIFTED, bool FULL>
__device__ __forceinline__ void copy_rows(const uint8_t *__restrict__ s, uint8_t *__restrict__ d,
					  uint32_t nvec, uint32_t shift, uint32_t lane)
{
	u32x4 v[R];
	uint32_t x[R];
#pragma unroll
	for (int k = 0; k < R; k++) {
		uint32_t j = (uint32_t)k * 64u + lane;
		if (!FULL && k == R - 1) {
			j = min(j, nvec - 1u); /* lanes past the end re-read the last word */
		}
		const uint8_t *p = s + ((uint64_t)j << 4);
		v[k] = load16_dword_aligned(p);
		if (SHIFTED && k == R - 1) {
			x[k] = *reinterpret_cast<const uint32_t *>(p + 16);
		}
	}
	if (SHIFTED) {
		/* The dword that follows a lane's 16 bytes is the first dword of the next lane's: it
		 * comes over from the neighbour (one wave-wide DPP shift; lane 63 takes lane 0 of the
		 * next row) instead of through a second load instruction over the same cache lines.
		 * Only the last row, whose lanes may be clamped, loads it. */
#pragma unroll
		for (int k = 0; k < R - 1; k++) {
			const uint32_t from_next = (uint32_t)__builtin_amdgcn_update_dpp(
				0, (int)v[k].x, 0x130 /* wave_shl:1 */, 0xf, 0xf, false);
			const uint32_t wrap = (uint32_t)__builtin_amdgcn_readfirstlane((int)v[k + 1].x);
			x[k] = lane == 63u ? wrap : from_next;
		}
	}
#pragma unroll
	for (int k = 0; k < R; k++) {
		uint32_t j = (uint32_t)k * 64u + lane;
		if (!FULL && k == R - 1) {
			j = min(j, nvec - 1u); /* ... and re-write it: same bytes, same place */
		}
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

template <bool SHIFTED>
__device__ __forceinline__ void copy_words(const uint8_t *__restrict__ s, uint8_t *__restrict__ d,
					   uint32_t nvec, uint32_t shift, uint32_t lane)
{
	while (nvec > kTripVec) { /* buffers beyond 8 KiB: whole trips first */
		copy_rows<kRows, SHIFTED, true>(s, d, kTripVec, shift, lane);
		s += (uint64_t)kTripVec << 4;
		d += (uint64_t)kTripVec << 4;
		nvec -= kTripVec;
	}
	switch ((nvec + 63u) >> 6) { /* wave-uniform */
	case 1: copy_rows<1, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 2: copy_rows<2, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 3: copy_rows<3, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 4: copy_rows<4, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 5: copy_rows<5, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 6: copy_rows<6, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 7: copy_rows<7, SHIFTED, false>(s, d, nvec, shift, lane); break;
	case 8: copy_rows<8, SHIFTED, false>(s, d, nvec, shift, lane); break;
	default: break; /* nvec == 0 */
	}
}

__global__ __launch_bounds__(kBlock) void bounce_scatter_kernel(
	const uint8_t *__restrict__ src, uint64_t src_bytes, uint8_t *__restrict__ arena, uint64_t arena_bytes,
	const uint64_t *__restrict__ src_off, const uint64_t *__restrict__ dst_off,
	const uint32_t *__restrict__ len, uint32_t n, uint32_t *__restrict__ flush,
	uint32_t *__restrict__ err)
{
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	/* Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Runs of kGroup
	 * consecutive workgroups' worth of buffers go to one XCD, so that neighbouring buffers
	 * -- which share a cache line of the packed source at their boundary -- mostly meet in
	 * the same L2, while every XCD still sees an even sample of the whole batch whatever
	 * order the lengths come in. */
	const uint32_t xcd = blockIdx.x % kXcds;
	const uint32_t turn = blockIdx.x / kXcds;
	const uint32_t wg = ((turn / kGroup) * kXcds + xcd) * kGroup + turn % kGroup;
	const uint32_t buf = wg * kWavesPerBlock + wave;
	if (buf >= n) {
		return;
	}

	const uint64_t doff = dst_off[buf];
	const uint32_t bytes = len[buf];
	const uint64_t soff = src_off[buf];
	/* precondition check: skip (and report) instead of reading or writing out of range; the
	 * read-back takes four bytes at the destination whatever the length */
	const uint64_t need = (flush != nullptr && bytes < 4u) ? 4u : bytes;
	if ((doff & 63u) != 0 || doff > arena_bytes || need > arena_bytes - doff || soff > src_bytes ||
	    bytes > src_bytes - soff) {
		if (lane == 0) {
			atomicOr(err, ofi_amd::ASYNC_ERR_BOUNCE_RANGE);
		}
		return;
	}

	const uint8_t *s = src + soff;
	uint8_t *d = arena + doff;

	if (bytes != 0) {
		/* whole 64-byte units as 16-byte words, the rest (up to 63 bytes) singly, one per
		 * lane: the last, partial unit of memory is then written by one instruction rather
		 * than by the end of a row and by the tail.  Tail bytes first, so their latency
		 * overlaps the body; unpredicated (lanes without a tail byte re-copy the buffer's
		 * last byte) to stay branch-free */
		const uint32_t nvec = (bytes >> 6) << 2;
		const uint32_t tail_at = min((nvec << 4) + lane, bytes - 1u);
		const uint8_t tail_byte = s[tail_at];

		const uint32_t shift = (uint32_t)(reinterpret_cast<uintptr_t>(s) & 3u);
		if (shift == 0) {
			copy_words<false>(s, d, nvec, 0, lane);
		} else {
			copy_words<true>(s - shift, d, nvec, shift, lane);
		}
		store_byte_streaming(d + tail_at, tail_byte);
	}

	if (flush != nullptr) {
		__builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
		if (lane == 0) {
			flush[buf] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(d));
		}
	}
}

/*
 * bytes from s to d, neither aligned: the bytes in front of the first 64-byte boundary of the
 * destination go out singly, one per lane; from there on it is the aligned-destination copy
 * above, with whatever source alignment that leaves.  Stopping at the first 16-byte boundary
 * would do for the 16-byte stores, but then every 1 KiB row of a trip begins and ends inside a
 * 64-byte unit of memory that the neighbouring row completes with a second, partial write
 * (measured on 65,536 buffers: 99.7 us with rows on 16-byte boundaries, 95.7 us on 64- or
 * 128-byte ones).  Wave-collective.
 */
__device__ __forceinline__ void copy_any(const uint8_t *__restrict__ s, uint8_t *__restrict__ d,
					 uint32_t bytes, uint32_t lane)
{
	if (bytes == 0) {
		return;
	}
	const uint32_t head = min(bytes, (64u - (uint32_t)(reinterpret_cast<uintptr_t>(d) & 63u)) & 63u);
	/* lanes without a head byte re-copy byte 0: same value, same place */
	const uint32_t head_at = min(lane, max(head, 1u) - 1u);
	const uint8_t head_byte = s[head_at];
	const uint32_t rem = bytes - head;
	if (rem != 0) {
		const uint8_t *s2 = s + head;
		uint8_t *d2 = d + head;
		const uint32_t nvec = (rem >> 6) << 2; /* as in the bounce copy */
		const uint32_t tail_at = min((nvec << 4) + lane, rem - 1u);
		const uint8_t tail_byte = s2[tail_at];
		const uint32_t shift = (uint32_t)(reinterpret_cast<uintptr_t>(s2) & 3u);
		if (shift == 0) {
			copy_words<false>(s2, d2, nvec, 0, lane);
		} else {
			copy_words<true>(s2 - shift, d2, nvec, shift, lane);
		}
		store_byte_streaming(d2 + tail_at, tail_byte);
	}
	store_byte_streaming(d + head_at, head_byte);
}

/*
 * The same copy for eager arrivals as they sit in rx buffers: an 8-byte header, then the
 * payload, which goes to a receive buffer at any alignment, truncated to that buffer's
 * length (rdma_eager_copy_req::post, src/nccl_ofi_rdma.cpp:2729-2776).
 */
__global__ __launch_bounds__(64 * kEagerWaves) void eager_copy_kernel(
	const uint8_t *__restrict__ rx_base, const uint64_t *__restrict__ rx_off,
	const uint32_t *__restrict__ recv_len, uint8_t *__restrict__ dst_base,
	const uint64_t *__restrict__ dst_off, const uint32_t *__restrict__ dst_len, uint32_t n,
	uint32_t *__restrict__ copied, uint32_t *__restrict__ flush)
{
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const uint32_t xcd = blockIdx.x % kXcds;
	const uint32_t turn = blockIdx.x / kXcds;
	const uint32_t wg = ((turn / kEagerGroup) * kXcds + xcd) * kEagerGroup + turn % kEagerGroup;
	const uint32_t buf = wg * kEagerWaves + wave;
	if (buf >= n) {
		return;
	}
	const uint8_t *s = rx_base + rx_off[buf] + 8u; /* skip nccl_ofi_eager_msg_header_t */
	uint8_t *d = dst_base + dst_off[buf];
	const uint32_t bytes = min(recv_len[buf], dst_len[buf]);
	if (copied != nullptr && lane == 0) {
		copied[buf] = bytes;
	}

	copy_any(s, d, bytes, lane);

	if (flush != nullptr) {
		__builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
		/* the first min(4, bytes) destination bytes, little-endian: lanes 0..3 read one byte
		 * each in one instruction (the destination has no alignment to read a word from),
		 * then the four are combined inside the quad */
		uint32_t word = 0;
		if (lane < min(bytes, 4u)) {
			word = (uint32_t)__builtin_nontemporal_load(d + lane) << (8u * lane);
		}
		word |= __shfl_xor(word, 1, 64);
		word |= __shfl_xor(word, 2, 64);
		if (lane == 0) {
			flush[buf] = word;
		}
	}
}

/* One wavefront per (source address, destination address, length) entry. */
__global__ __launch_bounds__(64 * kTableWaves) void copy_table_kernel(const uint64_t *__restrict__ src_addr,
							     const uint64_t *__restrict__ dst_addr,
							     const uint32_t *__restrict__ len, uint32_t n)
{
	const uint32_t lane = threadIdx.x & 63u;
	const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const uint32_t i = blockIdx.x * kTableWaves + wave;
	if (i >= n) {
		return;
	}
	copy_any(reinterpret_cast<const uint8_t *>(src_addr[i]), reinterpret_cast<uint8_t *>(dst_addr[i]), len[i],
		 lane);
}

/*
 * The same table with one wavefront per 8 KiB piece of an entry instead of per entry: entry e is
 * pieces [e * pieces_per_entry, (e + 1) * pieces_per_entry), and a wavefront whose piece lies
 * beyond its entry's length leaves at once.  Consecutive wavefronts then sweep long entries
 * densely, 8 KiB each, instead of each streaming through its own entry (1 GiB copied 8 KiB per
 * wavefront: 5.65 TB/s read + written, 256 KiB per wavefront: 5.17), and the XCDs take runs of
 * 128 consecutive pieces (1 MiB) in turn (5.82 TB/s; runs of 4 or 16: 5.5-5.7).
 */
constexpr uint32_t kPieceBytes = kRows * 1024u;
constexpr uint32_t kPieceRunShift = 7;
__global__ __launch_bounds__(64) void copy_table_pieces_kernel(const uint64_t *__restrict__ src_addr,
							       const uint64_t *__restrict__ dst_addr,
							       const uint32_t *__restrict__ len, uint32_t n,
							       uint32_t pieces_per_entry, uint32_t max_len,
							       uint32_t *__restrict__ err)
{
	const uint32_t lane = threadIdx.x;
	const uint32_t xcd = blockIdx.x % kXcds, turn = blockIdx.x / kXcds;
	const uint32_t g = ((((turn >> kPieceRunShift) * kXcds) + xcd) << kPieceRunShift) +
			   (turn & ((1u << kPieceRunShift) - 1u));
	const uint32_t e = g / pieces_per_entry, piece = g - e * pieces_per_entry;
	if (e >= n) {
		return;
	}
	const uint32_t stated = len[e];
	if (piece == 0 && stated > max_len && lane == 0) {
		atomicOr(err, ofi_amd::ASYNC_ERR_COPY_LENGTH); /* longer than the caller said: the rest stays uncopied */
	}
	const uint32_t bytes = min(stated, max_len);
	const uint64_t off = (uint64_t)piece * kPieceBytes;
	if (off >= bytes) {
		return;
	}
	const uint32_t here = bytes - off < kPieceBytes ? (uint32_t)(bytes - off) : kPieceBytes;
	copy_any(reinterpret_cast<const uint8_t *>(src_addr[e] + off), reinterpret_cast<uint8_t *>(dst_addr[e] + off),
		 here, lane);
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

__global__ __launch_bounds__(64) void flush_fill_kernel(uint64_t *__restrict__ flush_buf, uint64_t sentinel)
{
	if (threadIdx.x < 8) {
		flush_buf[threadIdx.x] = sentinel;
	}
}

__global__ __launch_bounds__(64) void flush_post_kernel(const uint64_t *__restrict__ flush_buf,
							uint64_t *__restrict__ slots, uint32_t num_rails)
{
	ofi_amd::flush_post_lanes(flush_buf, slots, num_rails, threadIdx.x);
}

} // namespace

/* A registered region: on a large-BAR system the whole of device memory is mapped into the
 * process at its device address, so the CPU mapping that GDRCopy creates by pinning and
 * mmap-ing (gdrcopy_RegHandle::mapped_ptr, include/nccl_ofi_gdrcopy.h:54-74) is the device
 * pointer itself. */
struct ofi_amd_devcopy_region {
	uint8_t *base;   /* device address (= CPU-visible mapping where cpu_mapped) */
	size_t size;
	bool cpu_mapped; /* the CPU can store to and load from `base`: large BAR and the range is in the
			  * process's address space; otherwise every copy goes through the copy engine */
};

/* CPU stores into the mapping are write-combined: 0.2-0.4 us for anything up to a page and
 * about 20 GB/s up to 1 MiB, against 11-14 us for the smallest hipMemcpy; from 16 MiB on the
 * copy engine is faster.  CPU loads from it are uncached round trips over PCIe: 2.5 us per
 * 64 bytes, so only a read of a few words beats the 12 us of a hipMemcpy. */
constexpr size_t kCpuStoreMax = 2u << 20;
constexpr size_t kCpuLoadMax = 256;

using namespace ofi_amd;

extern "C" {

int ofi_amd_bounce_scatter(const void *d_src, uint64_t src_bytes, void *d_arena, uint64_t arena_bytes,
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
	if (!d_src || !d_arena || !d_src_off || !d_dst_off || !d_len || n > (1u << 30)) {
		return -EINVAL;
	}
	uint32_t *err = async_error_word();
	if (!err) {
		return -ENOMEM;
	}
	uint32_t blocks = (n + kWavesPerBlock - 1) / kWavesPerBlock;
	const uint32_t round = kXcds * kGroup; /* whole rounds over the XCDs */
	blocks = (blocks + round - 1) / round * round;
	hipLaunchKernelGGL(bounce_scatter_kernel, dim3(blocks), dim3(kBlock), 0, as_stream(stream),
			   static_cast<const uint8_t *>(d_src), src_bytes, static_cast<uint8_t *>(d_arena),
			   arena_bytes, d_src_off, d_dst_off, d_len, n, d_flush, err);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_eager_copy_batch(const void *rx_base, const uint64_t *d_rx_off, const uint32_t *d_recv_len,
			     void *dst_base, const uint64_t *d_dst_off, const uint32_t *d_dst_len,
			     uint32_t n, uint32_t *d_copied, uint32_t *d_flush, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!rx_base || !d_rx_off || !d_recv_len || !d_dst_off || !d_dst_len || n > (1u << 30)) {
		return -EINVAL;
	}
	uint32_t blocks = (n + kEagerWaves - 1) / kEagerWaves;
	const uint32_t round = kXcds * kEagerGroup;
	blocks = (blocks + round - 1) / round * round;
	hipLaunchKernelGGL(eager_copy_kernel, dim3(blocks), dim3(64 * kEagerWaves), 0, as_stream(stream),
			   static_cast<const uint8_t *>(rx_base), d_rx_off, d_recv_len,
			   static_cast<uint8_t *>(dst_base), d_dst_off, d_dst_len, n, d_copied, d_flush);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_copy_table(const uint64_t *d_src_addr, const uint64_t *d_dst_addr, const uint32_t *d_len,
		       uint32_t n, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!d_src_addr || !d_dst_addr || !d_len || n > (1u << 30)) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(copy_table_kernel, dim3((n + kTableWaves - 1) / kTableWaves), dim3(64 * kTableWaves), 0,
			   as_stream(stream), d_src_addr, d_dst_addr, d_len, n);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_copy_table_pieces(const uint64_t *d_src_addr, const uint64_t *d_dst_addr, const uint32_t *d_len,
			      uint32_t n, uint32_t max_len, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (n == 0) {
		return 0;
	}
	if (!d_src_addr || !d_dst_addr || !d_len || n > (1u << 30)) {
		return -EINVAL;
	}
	const uint64_t pieces_per_entry = max_len == 0 ? 1 : ((uint64_t)max_len + kPieceBytes - 1) / kPieceBytes;
	const uint64_t round = (uint64_t)kXcds << kPieceRunShift; /* whole rounds over the XCDs */
	const uint64_t blocks = ((uint64_t)n * pieces_per_entry + round - 1) / round * round;
	if (blocks > 0x7fffffffull) {
		return -E2BIG; /* more pieces than one launch has workgroups: split the table */
	}
	uint32_t *err = async_error_word();
	if (!err) {
		return -ENOMEM;
	}
	hipLaunchKernelGGL(copy_table_pieces_kernel, dim3((uint32_t)blocks), dim3(64), 0, as_stream(stream), d_src_addr,
			   d_dst_addr, d_len, n, (uint32_t)pieces_per_entry, max_len, err);
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

int ofi_amd_flush_buffer_fill(void *d_flush_buf, uint64_t sentinel, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!d_flush_buf || (reinterpret_cast<uintptr_t>(d_flush_buf) & 7u)) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(flush_fill_kernel, dim3(1), dim3(64), 0, as_stream(stream),
			   static_cast<uint64_t *>(d_flush_buf), sentinel);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

int ofi_amd_flush_post(const void *d_flush_buf, void *slots_dev, uint32_t num_rails, void *stream)
{
	int rc = require_device();
	if (rc != 0) {
		return rc;
	}
	if (!d_flush_buf || !slots_dev || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS ||
	    (reinterpret_cast<uintptr_t>(d_flush_buf) & 7u) || (reinterpret_cast<uintptr_t>(slots_dev) & 7u)) {
		return -EINVAL;
	}
	hipLaunchKernelGGL(flush_post_kernel, dim3(1), dim3(64), 0, as_stream(stream),
			   static_cast<const uint64_t *>(d_flush_buf), static_cast<uint64_t *>(slots_dev),
			   num_rails);
	OFI_AMD_HIP_TRY(hipGetLastError());
	return 0;
}

/* ofi_amd_flush_test, the host side of the flush, lives with the other host-only wire code
 * (wire_codec.cpp). */

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
	/* The CPU reaches device memory only where the whole of it sits behind the PCIe BAR, and
	 * then only allocations that the runtime has mapped into the process at their device
	 * address (hipMalloc memory is; an imported or virtual-memory allocation need not be):
	 * the first and the last page of the range are asked of the kernel.  Without either,
	 * the region still registers and its copies take the copy engine at every size, as the
	 * interface promises nothing about the path. */
	int large_bar = 0;
	if (hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, attr.device) != hipSuccess) {
		(void)hipGetLastError();
		large_bar = 0;
	}
	bool mapped = large_bar != 0;
	if (mapped) {
		const long page = sysconf(_SC_PAGESIZE);
		const uintptr_t first = reinterpret_cast<uintptr_t>(device_ptr) & ~(uintptr_t)(page - 1);
		const uintptr_t last = (reinterpret_cast<uintptr_t>(device_ptr) + size - 1) & ~(uintptr_t)(page - 1);
		unsigned char vec = 0;
		mapped = mincore(reinterpret_cast<void *>(first), (size_t)page, &vec) == 0 &&
			 mincore(reinterpret_cast<void *>(last), (size_t)page, &vec) == 0;
	}
	auto *h = new (std::nothrow) ofi_amd_devcopy_region;
	if (!h) {
		return -ENOMEM;
	}
	h->base = static_cast<uint8_t *>(device_ptr);
	h->size = size;
	h->cpu_mapped = mapped;
	*out = h;
	return 0;
}

int ofi_amd_devcopy_to_device(const void *host_ptr, ofi_amd_devcopy_region_t *h, size_t offset,
			      size_t size)
{
	if (!h || !host_ptr || offset > h->size || size > h->size - offset) {
		return -EINVAL;
	}
	if (h->cpu_mapped && size <= kCpuStoreMax) {
		/* gdr_copy_to_mapping: CPU stores through the mapping, then drain the
		 * write-combining buffers so that the bytes are on their way before the caller
		 * rings any doorbell */
		std::memcpy(h->base + offset, host_ptr, size);
		_mm_sfence();
		return 0;
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
	if (h->cpu_mapped && size <= kCpuLoadMax) {
		/* gdr_copy_from_mapping: CPU loads through the mapping */
		std::memcpy(host_ptr, h->base + offset, size);
		_mm_lfence();
		return 0;
	}
	OFI_AMD_HIP_TRY(hipMemcpy(host_ptr, h->base + offset, size, hipMemcpyDeviceToHost));
	return 0;
}

int ofi_amd_devcopy_cpu_mapped(const ofi_amd_devcopy_region_t *h)
{
	return h ? (h->cpu_mapped ? 1 : 0) : -EINVAL;
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

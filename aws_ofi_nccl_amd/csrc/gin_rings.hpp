/*
 * Layout of the GIN descriptor rings shared by the GPU producers
 * (gin_rings.hip) and the host proxy (gin_proxy.cpp).
 *
 * One ring per GIN context, all in pinned host memory.  The protocol is the
 * bounded-slot scheme of include/nccl_ofi_mpsc_ring.h:56-163 in the reference:
 * slot s carries a 32-bit sequence word that says whose turn it is --
 * sequence == pos: free for the producer of position pos; == pos + 1: published
 * for the consumer; the consumer frees it with pos + capacity.  Unlike the
 * reference's array of {sequence, payload} cells, payloads (64 B) and sequence
 * words are kept in two arrays, so a wavefront writes 64 descriptors as 4 KiB
 * of contiguous 16-byte stores and publishes them with one contiguous 256-byte
 * store, and the consumer sees 16 sequence words per cache line.
 */
#ifndef OFI_AMD_GIN_RINGS_HPP_
#define OFI_AMD_GIN_RINGS_HPP_

#include <cstdint>

#include "ofi_amd_hotpath.h"

struct ofi_amd_gin_rings {
	uint32_t n_contexts;
	uint32_t capacity;          /* power of two */
	ofi_amd_gin_desc_t *records; /* [n_contexts][capacity], pinned host */
	uint32_t *sequences;        /* [n_contexts][capacity], pinned host */
	uint32_t *enqueue_pos;      /* [n_contexts * 16] one cursor per 64-byte line, pinned host */
	uint32_t *dequeue_pos;      /* [n_contexts], ordinary host memory (single consumer) */
	uint32_t *status;           /* pinned host: producers OR error bits in */
	/* device-side addresses of the pinned arrays */
	ofi_amd_gin_desc_t *d_records;
	uint32_t *d_sequences;
	uint32_t *d_enqueue_pos;
	uint32_t *d_status;
	/* device memory: reservation cursor of the GPU producers, one per 128-byte line */
	uint32_t *d_reserve;
};

constexpr uint32_t kGinReserveStride = 32; /* u32 words between two contexts' cursors */

#endif

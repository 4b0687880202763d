/*
 * CPU oracle (test infrastructure): batched eager/bounce copy + flush read.
 *
 * The reference moves each eager payload with one loop-back fi_read from the
 * bounce buffer into the user buffer (src/nccl_ofi_rdma.cpp:2729-2776;
 * zero-length payloads are skipped, :753-762) and makes it visible with a
 * small read-back (flush, :2664-2713; NCCL_OFI_FLUSH_SIZE = 4,
 * include/nccl_ofi.h:74).  Its observable result is plain byte-copy semantics,
 * restated here as one memcpy per buffer.
 */
#include <string.h>

#include "oracle.h"

void oracle_bounce_scatter(const uint8_t *src, uint8_t *arena, const uint64_t *src_off,
			   const uint64_t *dst_off, const uint32_t *len, uint32_t n,
			   uint32_t *flush)
{
	for (uint32_t i = 0; i < n; i++) {
		if (len[i] != 0) {
			memcpy(arena + dst_off[i], src + src_off[i], len[i]);
		}
	}
	if (flush) {
		for (uint32_t i = 0; i < n; i++) {
			uint32_t w;
			memcpy(&w, arena + dst_off[i], sizeof(w));
			flush[i] = w;
		}
	}
}

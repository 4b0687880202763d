/*
 * Test infrastructure: C entry points onto the parts of the aws-ofi-nccl
 * reference that are self-contained headers and therefore compile here
 * straight from the reference tree (no generated config.h, no libfabric):
 *
 *   include/nccl_ofi_mpsc_ring.h, include/nccl_ofi_spsc_ring.h  (ring protocol)
 *   include/rdma/gin/nccl_ofi_gin_types.h   (immediate-data macros, bit-field
 *                                            message structs, window constants)
 *   include/nccl_ofi_math.h                 (DIV_CEIL, ROUND_UP, ...)
 *
 * The headers are included where they lie (-I <reference>/include); nothing of
 * them is copied.  The resulting library (oracle/_ref/libref.so) is used only
 * by tests to cross-check the oracle's restatement of the same items.
 */
#include <cstdint>
#include <cstring>

#include "nccl_ofi_math.h"
#include "nccl_ofi_mpsc_ring.h"
#include "nccl_ofi_spsc_ring.h"
#include "rdma/gin/nccl_ofi_gin_types.h"

namespace {
struct rec64 {
	uint8_t b[64];
};
using mpsc_rec_4096 = nccl_ofi_mpsc_ring<rec64, 4096>;
using mpsc_u64_8 = nccl_ofi_mpsc_ring<uint64_t, 8>;
using mpsc_u64_1024 = nccl_ofi_mpsc_ring<uint64_t, 1024>;
using spsc_u64_8 = nccl_ofi_spsc_ring<uint64_t, 8>;
} // namespace

extern "C" {

/* kind: 0 = <64-byte record, 4096>, 1 = <u64, 8>, 2 = <u64, 1024> */
void *ref_mpsc_create(int kind)
{
	switch (kind) {
	case 0: return new mpsc_rec_4096();
	case 1: return new mpsc_u64_8();
	case 2: return new mpsc_u64_1024();
	default: return nullptr;
	}
}

void ref_mpsc_destroy(int kind, void *r)
{
	switch (kind) {
	case 0: delete static_cast<mpsc_rec_4096 *>(r); break;
	case 1: delete static_cast<mpsc_u64_8 *>(r); break;
	case 2: delete static_cast<mpsc_u64_1024 *>(r); break;
	}
}

int ref_mpsc_push(int kind, void *r, const void *entry)
{
	switch (kind) {
	case 0: return static_cast<mpsc_rec_4096 *>(r)->push(*static_cast<const rec64 *>(entry));
	case 1: return static_cast<mpsc_u64_8 *>(r)->push(*static_cast<const uint64_t *>(entry));
	case 2: return static_cast<mpsc_u64_1024 *>(r)->push(*static_cast<const uint64_t *>(entry));
	default: return -1;
	}
}

int ref_mpsc_pop(int kind, void *r, void *entry)
{
	switch (kind) {
	case 0: return static_cast<mpsc_rec_4096 *>(r)->pop(*static_cast<rec64 *>(entry));
	case 1: return static_cast<mpsc_u64_8 *>(r)->pop(*static_cast<uint64_t *>(entry));
	case 2: return static_cast<mpsc_u64_1024 *>(r)->pop(*static_cast<uint64_t *>(entry));
	default: return -1;
	}
}

void *ref_spsc_create(void) { return new spsc_u64_8(); }
void ref_spsc_destroy(void *r) { delete static_cast<spsc_u64_8 *>(r); }
int ref_spsc_push(void *r, uint64_t v) { return static_cast<spsc_u64_8 *>(r)->push(v); }
int ref_spsc_pop(void *r, uint64_t *v) { return static_cast<spsc_u64_8 *>(r)->pop(*v); }

uint32_t ref_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return (uint32_t)GIN_IMM_SEG_DATA(comm_id, seq, nseg, ack_req);
}

void ref_gin_imm_decode(uint32_t imm, uint32_t *comm_id, uint32_t *seq, uint32_t *nseg,
			uint32_t *ack_req)
{
	*comm_id = GIN_IMM_GET_COMM_ID(imm);
	*seq = GIN_IMM_GET_SEQ_NUM(imm);
	*nseg = GIN_IMM_GET_SEG_CNT(imm);
	*ack_req = GIN_IMM_GET_ACK_REQUESTED(imm);
}

/* Fill the 32-byte metadata message through the reference's bit-field struct. */
void ref_gin_meta(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req,
		  uint64_t base, uint64_t off, uint64_t value, void *out32)
{
	nccl_net_ofi_gin_signal_metadata_msg_t m;
	std::memset(&m, 0, sizeof(m));
	m.header.msg_type = GIN_MSG_TYPE_METADATA;
	m.header.remote_comm_id = comm_id;
	m.header.seq_num = seq;
	m.header.seq_seg_cnt = nseg;
	m.header.ack_req = ack_req;
	m.signal_base_address = base;
	m.signal_offset = off;
	m.signal_value = value;
	std::memcpy(out32, &m, sizeof(m));
}

uint64_t ref_gin_ack(uint32_t comm_id, uint32_t rx_consumed)
{
	gin_ack_msg_t a;
	std::memset(&a, 0, sizeof(a));
	a.msg_type = GIN_MSG_TYPE_ACK;
	a.ack_comm_id = comm_id;
	a.rx_consumed = rx_consumed;
	uint64_t v;
	std::memcpy(&v, &a, sizeof(v));
	return v;
}

/* index: 0 seq mask, 1 rx-consumed mask, 2 rx-consumed half, 3 ack interval,
 * 4 reqs per doorbell, 5 ack-request threshold, 6 max comms, 7 max rails */
uint64_t ref_gin_const(int index)
{
	switch (index) {
	case 0: return GIN_IMM_SEQ_MASK;
	case 1: return GIN_RX_CONSUMED_MASK;
	case 2: return GIN_RX_CONSUMED_HALF;
	case 3: return GIN_ACK_INTERVAL;
	case 4: return GIN_REQS_PER_DOORBELL;
	case 5: return GIN_ACK_REQ_THRESHOLD;
	case 6: return NCCL_GIN_MAX_COMMS;
	case 7: return MAX_NUM_RAILS;
	default: return ~0ull;
	}
}

uint64_t ref_div_ceil(uint64_t x, uint64_t y) { return NCCL_OFI_DIV_CEIL(x, y); }
uint64_t ref_round_up(uint64_t x, uint64_t y) { return NCCL_OFI_ROUND_UP(x, y); }
uint64_t ref_round_down(uint64_t x, uint64_t y) { return NCCL_OFI_ROUND_DOWN(x, y); }

} /* extern "C" */

/*
 * The glue a maintainer of the reference would add on top of the C ABI, compiled for real:
 * the replacement of src/nccl_ofi_rocm.cpp and an nccl_ofi_device_copy implementation, both
 * as they are printed in sections 1 and 2 of the integration guide at the repository root
 * (tests/test_integration_glue.py checks that the text between the markers below is the text
 * printed there), built against
 * the reference's own headers where they lie (include/nccl_ofi_rocm.h,
 * include/nccl_ofi_device_copy.h) and linked against libofi_amd_hotpath.so.
 *
 *   integration_glue link   the forwards that answer without a GPU
 *   integration_glue gpu    the patterns of the reference's tests/unit/gdrcopy.cpp:15-133 (a
 *                           2 MiB buffer written and read back whole, a 10-byte buffer written
 *                           and read back byte by byte) through the C++ class, plus offsets
 *                           and sizes around the class's CPU-store / copy-engine switch; a message
 *                           each way through the net table and a put-signal through the RMA table
 *   integration_glue rate   messages and put-signals per second through the two tables, 64 in
 *                           flight, as one JSON line
 */
#include <cerrno>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <ctime>
#include <vector>

// [section 1]
// src/nccl_ofi_rocm.cpp (replacement)
#include <cstddef>
#include "nccl_ofi_rocm.h"
#include "ofi_amd_hotpath.h"

int nccl_net_ofi_gpu_init(void)                                   { return ofi_amd_gpu_init(); }
int nccl_net_ofi_get_gpu_device_for_addr(void *p, int *dev)       { return ofi_amd_gpu_get_device_for_addr(p, dev); }
int nccl_net_ofi_gpu_flush_gpudirect_rdma_writes(void)            { return ofi_amd_gpu_flush_gpudirect_rdma_writes(); } // -EPERM, as today
int nccl_net_ofi_gpu_mem_alloc(void **p, size_t n)                { return ofi_amd_gpu_mem_alloc(p, n); }
int nccl_net_ofi_gpu_mem_free(void *p)                            { return ofi_amd_gpu_mem_free(p); }
int nccl_net_ofi_gpu_mem_copy_host_to_device(void *d, void *s, size_t n) { return ofi_amd_gpu_mem_copy_host_to_device(d, s, n); }
int nccl_net_ofi_gpu_get_dma_buf_fd(void *p, size_t n, int *fd, size_t *off) { return ofi_amd_gpu_get_dma_buf_fd(p, n, fd, off); }
bool nccl_net_ofi_gpu_have_dma_buf_attr(void)                     { return ofi_amd_gpu_have_dma_buf_attr() != 0; }
bool nccl_net_ofi_gpu_have_gdr_support_attr(void)                 { return ofi_amd_gpu_have_gdr_support_attr() != 0; }
// [end of section 1]

// [section 2]
#include "nccl_ofi_device_copy.h"

class nccl_ofi_device_copy_amd : public nccl_ofi_device_copy {
	struct Handle : RegHandle { ofi_amd_devcopy_region_t *r; };
public:
	int register_region(void *ptr, size_t size, RegHandle *&out) override {
		auto *h = new Handle;
		int rc = ofi_amd_devcopy_register(ptr, size, &h->r);
		if (rc) { delete h; return rc; }
		out = h; return 0;
	}
	int copy_to_device(const void *host, const RegHandle &h, size_t off, size_t n) override {
		return ofi_amd_devcopy_to_device(host, static_cast<const Handle &>(h).r, off, n);
	}
	int copy_from_device(const RegHandle &h, size_t off, void *host, size_t n) override {
		return ofi_amd_devcopy_from_device(static_cast<const Handle &>(h).r, off, host, n);
	}
	bool forced_pcie_copy() override { return ofi_amd_devcopy_forced_pcie_copy() != 0; }
	int deregister_region(RegHandle *h) override {
		int rc = ofi_amd_devcopy_deregister(static_cast<Handle *>(h)->r); delete static_cast<Handle *>(h); return rc;
	}
};
// [end of section 2]

/* The data-path members of the reference's ncclRma_v15_t take this library's functions as they
 * are: a mismatch in any parameter list is a compile error here. */
#include "nccl/net.h"
#include "nccl/rma_v15.h"
#include "ofi_amd_rma_abi.h"

static ncclRma_v15_t rma_table_with_this_librarys_data_path()
{
	ncclRma_v15_t t = {};
	t.name = "Libfabric";
	t.iput = ofi_amd_rma_iput;
	t.iputSignal = ofi_amd_rma_iputSignal;
	t.iget = ofi_amd_rma_iget;
	t.iflush = ofi_amd_rma_iflush;
	t.test = ofi_amd_rma_test;
	t.rmaProgress = ofi_amd_rma_rmaProgress;
	return t;
}

/* ... and the older tables the reference exports beside it (ncclRmaPlugin_v14, ncclGinPlugin_v13,
 * ncclGinPlugin_v11: src/rdma/gin/nccl_ofi_gin_api.cpp:566-617, 666-688) */
#include "nccl/rma_v14.h"
#include "nccl/gin_v13.h"

static ncclRma_v14_t rma_v14_table_with_this_librarys_data_path()
{
	ncclRma_v14_t t = {};
	t.iput = ofi_amd_rma_iput_v14;
	t.iputSignal = ofi_amd_rma_iputSignal_v14;
	t.iget = ofi_amd_rma_iget_v14;
	t.iflush = ofi_amd_rma_iflush;
	t.test = ofi_amd_rma_test;
	t.rmaProgress = ofi_amd_rma_rmaProgress;
	return t;
}

static ncclGin_v13_t gin_v13_table_with_this_librarys_data_path()
{
	ncclGin_v13_t t = {};
	t.iput = ofi_amd_rma_iput_v14;
	t.iputSignal = ofi_amd_gin_iputSignal_v13;
	t.iget = ofi_amd_rma_iget_v14;
	t.iflush = ofi_amd_rma_iflush;
	t.test = ofi_amd_rma_test;
	t.ginProgress = ofi_amd_rma_rmaProgress;
	return t;
}

static ncclGin_v11_t gin_v11_table_with_this_librarys_data_path()
{
	ncclGin_v11_t t = {};
	t.iput = ofi_amd_gin_iput_v11;
	t.iputSignal = ofi_amd_gin_iputSignal_v11;
	t.test = ofi_amd_rma_test;
	t.ginProgress = ofi_amd_rma_rmaProgress;
	return t;
}

/* The data-path members of the reference's ncclNet tables (ncclNetPlugin_v6 .. v12,
 * src/nccl_ofi_interface_nvidia.cpp:661-825): the three spellings the reference's shims cover */
#include "ofi_amd_net_abi.h"

static ncclNet_v12_t net_v12_table_with_this_librarys_data_path()
{
	ncclNet_v12_t t = {};
	t.name = "Libfabric";
	t.isend = ofi_amd_net_isend;
	t.irecv = ofi_amd_net_irecv;
	t.iflush = ofi_amd_net_iflush;
	t.test = ofi_amd_net_test;
	return t;
}

template <typename Table> static Table net_table_v10_or_v11()
{
	Table t = {};
	t.isend = ofi_amd_net_isend;
	t.irecv = ofi_amd_net_irecv;
	t.iflush = ofi_amd_net_iflush;
	t.test = ofi_amd_net_test;
	return t;
}

static ncclNet_v9_t net_v9_table_with_this_librarys_data_path()
{
	ncclNet_v9_t t = {};
	t.isend = ofi_amd_net_isend_v9;
	t.irecv = ofi_amd_net_irecv_v9;
	t.iflush = ofi_amd_net_iflush;
	t.test = ofi_amd_net_test;
	return t;
}

template <typename Table> static Table net_table_v6_to_v8()
{
	Table t = {};
	t.isend = ofi_amd_net_isend_v5;
	t.irecv = ofi_amd_net_irecv_v5;
	t.iflush = ofi_amd_net_iflush;
	t.test = ofi_amd_net_test;
	return t;
}

#define CHECK(cond)                                                                       \
	do {                                                                              \
		if (!(cond)) {                                                            \
			fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
			return 1;                                                         \
		}                                                                         \
	} while (0)

static int link_checks()
{
	/* answers that do not depend on a device */
	CHECK(nccl_net_ofi_gpu_flush_gpudirect_rdma_writes() == -EPERM); /* src/nccl_ofi_rocm.cpp:53-56 */
	CHECK(nccl_net_ofi_gpu_have_gdr_support_attr() == false);        /* :78-81 */
	nccl_ofi_device_copy_amd copy;
	nccl_ofi_device_copy &iface = copy;
	CHECK(iface.forced_pcie_copy() == false);
	/* one put through the table's pointers over the in-process fabric, polled to completion */
	{
		const ncclRma_v15_t table = rma_table_with_this_librarys_data_path();
		ofi_amd_loopfab_t *fab = nullptr;
		ofi_amd_gin_fabric_ops_t ops;
		CHECK(ofi_amd_loopfab_create(4, 64, &fab) == 0 && ofi_amd_loopfab_ops(fab, &ops) == 0);
		ofi_amd_rma_ctx_t *rma = nullptr;
		CHECK(ofi_amd_rma_ctx_create(2, 4, 131072, 64, &ops, 256, 0, &rma) == 0);
		const uint64_t addr[2] = {0x7e0000000000ull, 0x7e0100000000ull}, keys[8] = {1, 2, 3, 4, 5, 6, 7, 8};
		ofi_amd_rma_mr_t *mr = nullptr;
		CHECK(ofi_amd_rma_mr_create(rma, 0x7f0000000000ull, addr, addr, keys, &mr) == 0);
		void *request = nullptr;
		CHECK(table.iput(rma, 0, 16, mr, 5000, 32, mr, 1, ncclRmaOptFlagsDefault, &request) == ncclSuccess && request);
		ofi_amd_gin_post_t sent[4];
		CHECK(ofi_amd_loopfab_take_transmitted(fab, sent, 4) == 1);
		CHECK(sent[0].kind == OFI_AMD_GIN_POST_WRITE && sent[0].len == 5000 && sent[0].src == 0x7f0000000010ull &&
		      sent[0].dest == addr[1] + 32 && sent[0].key == keys[4 + sent[0].rail]);
		int done = 0;
		CHECK(table.test(rma, request, &done) == ncclSuccess && done == 0);
		CHECK(table.rmaProgress(rma) == ncclSuccess);
		CHECK(table.test(rma, request, &done) == ncclSuccess && done == 1);
		CHECK(table.iput(rma, 0, 0, mr, 8, 0, mr, 7, 0, &request) == ncclInternalError); /* no such rank */
		/* the older tables reach the same context: one put-signal through each, the sequence
		 * number in the immediate data counts on (GIN_IMM_SEQ, bits 11..23) */
		const ncclRma_v14_t t14 = rma_v14_table_with_this_librarys_data_path();
		const ncclGin_v13_t t13 = gin_v13_table_with_this_librarys_data_path();
		const ncclGin_v11_t t11 = gin_v11_table_with_this_librarys_data_path();
		void *r14 = nullptr, *r13 = nullptr, *r11 = nullptr;
		CHECK(t14.iputSignal(rma, 0, 0, mr, 5000, 0, mr, 1, 8, mr, 1, 1, true, &r14) == ncclSuccess && r14);
		CHECK(t13.iputSignal(rma, 0, 0, mr, 5000, 0, mr, 1, 8, mr, 1, 1, &r13) == ncclSuccess && r13);
		CHECK(t11.iputSignal(rma, 0, mr, 5000, 0, mr, 1, 8, mr, 1, 1, &r11) == ncclSuccess && r11);
		ofi_amd_gin_post_t later[8];
		CHECK(ofi_amd_loopfab_take_transmitted(fab, later, 8) == 6); /* a write and a metadata message each */
		for (int k = 0; k < 3; k++) {
			CHECK(later[2 * k].kind == OFI_AMD_GIN_POST_WRITE && later[2 * k + 1].kind == OFI_AMD_GIN_POST_META);
			CHECK(((later[2 * k].imm >> 11) & 0x1fffu) == 1u + (uint32_t)k);
		}
		CHECK(t13.ginProgress(rma) == ncclSuccess);
		CHECK(t14.test(rma, r14, &done) == ncclSuccess && done == 1);
		CHECK(t13.test(rma, r13, &done) == ncclSuccess && done == 1);
		CHECK(t11.test(rma, r11, &done) == ncclSuccess && done == 1);
		void *g = nullptr;
		CHECK(t13.iget(rma, 0, 0, mr, 64, 0, mr, 1, &g) == ncclSuccess && g);
		CHECK(t11.iput(rma, 0, mr, 8, 0, mr, 1, &g) == ncclSuccess && g);
		CHECK(ofi_amd_rma_mr_destroy(mr) == 0 && ofi_amd_rma_ctx_destroy(rma) == 0 && ofi_amd_loopfab_destroy(fab) == 0);
	}
	{ /* every net table takes the functions; without a comm they answer as the reference's checks do */
		const ncclNet_v12_t n12 = net_v12_table_with_this_librarys_data_path();
		const ncclNet_v11_t n11 = net_table_v10_or_v11<ncclNet_v11_t>();
		const ncclNet_v10_t n10 = net_table_v10_or_v11<ncclNet_v10_t>();
		const ncclNet_v9_t n9 = net_v9_table_with_this_librarys_data_path();
		const ncclNet_v8_t n8 = net_table_v6_to_v8<ncclNet_v8_t>();
		const ncclNet_v7_t n7 = net_table_v6_to_v8<ncclNet_v7_t>();
		const ncclNet_v6_t n6 = net_table_v6_to_v8<ncclNet_v6_t>();
		void *request = &request;
		int done = 0;
		CHECK(n12.isend(nullptr, nullptr, 8, 1, nullptr, nullptr, &request) == ncclInternalError && !request);
		CHECK(n11.test(nullptr, &done, nullptr) == ncclInternalError);
		CHECK(n10.iflush(nullptr, 1, nullptr, nullptr, nullptr, &request) == ncclInternalError);
		CHECK(n9.isend(nullptr, nullptr, 8, 1, nullptr, &request) == ncclInternalError);
		CHECK(n8.irecv(nullptr, 1, nullptr, nullptr, nullptr, nullptr, &request) == ncclInvalidArgument);
		CHECK(n7.isend(nullptr, nullptr, 8, 1, nullptr, &request) == ncclInternalError);
		CHECK(n6.test(nullptr, &done, nullptr) == ncclInternalError);
	}
	const int init = nccl_net_ofi_gpu_init();
	if (init == -ENODEV) {
		/* no GPU here: every device call says so, through the glue as through the C ABI */
		void *p = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&p, 64) == -ENODEV);
		nccl_ofi_device_copy::RegHandle *h = nullptr;
		char byte = 0;
		CHECK(iface.register_region(&byte, 1, h) == -ENODEV && h == nullptr);
		printf("link: ok (no device)\n");
		return 0;
	}
	CHECK(init == 0);
	printf("link: ok (device present)\n");
	return 0;
}

static int gpu_checks()
{
	CHECK(nccl_net_ofi_gpu_init() == 0);
	nccl_ofi_device_copy_amd amd;
	nccl_ofi_device_copy &gdr = amd;

	{ /* test_large_buffer, tests/unit/gdrcopy.cpp:15-74 */
		constexpr size_t buff_size = 2 * 1024 * 1024UL;
		void *ptr = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&ptr, buff_size) == 0);
		int dev = -1;
		CHECK(nccl_net_ofi_get_gpu_device_for_addr(ptr, &dev) == 0 && dev >= 0);
		nccl_ofi_device_copy::RegHandle *handle = nullptr;
		CHECK(gdr.register_region(ptr, buff_size, handle) == 0);
		std::vector<char> host_buff(buff_size, 'A'), dst_host_buff(buff_size, 0);
		CHECK(gdr.copy_to_device(host_buff.data(), *handle, 0, buff_size) == 0);
		CHECK(gdr.copy_from_device(*handle, 0, dst_host_buff.data(), buff_size) == 0);
		CHECK(memcmp(host_buff.data(), dst_host_buff.data(), buff_size) == 0);
		CHECK(gdr.deregister_region(handle) == 0);
		CHECK(nccl_net_ofi_gpu_mem_free(ptr) == 0);
	}
	{ /* test_small_buffer, :76-133 */
		constexpr size_t buff_size = 10;
		void *ptr = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&ptr, buff_size) == 0);
		nccl_ofi_device_copy::RegHandle *handle = nullptr;
		CHECK(gdr.register_region(ptr, buff_size, handle) == 0);
		for (size_t i = 0; i < buff_size; ++i) {
			uint8_t v = (uint8_t)i;
			CHECK(gdr.copy_to_device(&v, *handle, i, 1) == 0);
		}
		for (size_t i = 0; i < buff_size; ++i) {
			uint8_t v = 0xff;
			CHECK(gdr.copy_from_device(*handle, i, &v, 1) == 0);
			CHECK(v == i);
		}
		CHECK(gdr.deregister_region(handle) == 0);
		CHECK(nccl_net_ofi_gpu_mem_free(ptr) == 0);
	}
	{ /* either side of the switch between CPU stores / loads and the copy engine, at odd offsets,
	   * against a host-to-device copy through the other path of the glue */
		constexpr size_t buff_size = 16u << 20;
		void *ptr = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&ptr, buff_size) == 0);
		nccl_ofi_device_copy::RegHandle *handle = nullptr;
		CHECK(gdr.register_region(ptr, buff_size, handle) == 0);
		std::vector<uint8_t> pattern(buff_size), back(buff_size);
		for (size_t i = 0; i < buff_size; i++) {
			pattern[i] = (uint8_t)(i * 2654435761u >> 24);
		}
		std::vector<uint8_t> zero(buff_size, 0);
		CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(ptr, zero.data(), buff_size) == 0);
		const size_t sizes[] = {1, 255, 256, 257, 4096, (2u << 20) - 1, 2u << 20, (2u << 20) + 1, 3u << 20};
		size_t at = 3;
		for (size_t n : sizes) {
			CHECK(at + n <= buff_size);
			CHECK(gdr.copy_to_device(pattern.data() + at, *handle, at, n) == 0);
			CHECK(gdr.copy_from_device(*handle, at, back.data() + at, n) == 0);
			CHECK(memcmp(pattern.data() + at, back.data() + at, n) == 0);
			at += n + 5;
		}
		/* out of range: refused, nothing written */
		CHECK(gdr.copy_to_device(pattern.data(), *handle, buff_size - 4, 8) == -EINVAL);
		CHECK(gdr.copy_from_device(*handle, buff_size, back.data(), 1) == -EINVAL);
		CHECK(gdr.deregister_region(handle) == 0);
		CHECK(nccl_net_ofi_gpu_mem_free(ptr) == 0);
	}
	{ /* the dma-buf forward, called as the reference calls it for a registration */
		void *ptr = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&ptr, 1u << 20) == 0);
		if (nccl_net_ofi_gpu_have_dma_buf_attr()) {
			int fd = -1;
			size_t off = 99;
			CHECK(nccl_net_ofi_gpu_get_dma_buf_fd(ptr, 1u << 20, &fd, &off) == 0 && fd >= 0 && off == 0);
		}
		CHECK(nccl_net_ofi_gpu_mem_free(ptr) == 0);
	}
	{ /* one eager and one rendezvous message through the v12 table's pointers: post_send /
	   * post_recv / poll as in tests/functional/functional_test.cpp:242-294, 592-640 */
		const ncclNet_v12_t net = net_v12_table_with_this_librarys_data_path();
		ofi_amd_net_link_t *link = nullptr;
		CHECK(ofi_amd_net_link_create(4, 8192, 0, 0, 0, nullptr, &link) == 0);
		void *sComm = ofi_amd_net_link_send_comm(link), *rComm = ofi_amd_net_link_recv_comm(link);
		const size_t sizes_to_try[2] = {4096, 1u << 20};
		for (size_t bytes : sizes_to_try) {
			void *src = nullptr, *dst = nullptr;
			CHECK(nccl_net_ofi_gpu_mem_alloc(&src, bytes) == 0 && nccl_net_ofi_gpu_mem_alloc(&dst, bytes) == 0);
			std::vector<uint8_t> pattern(bytes), back(bytes, 0);
			for (size_t i = 0; i < bytes; i++) {
				pattern[i] = (uint8_t)((i + bytes) * 2654435761u >> 24);
			}
			CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(src, pattern.data(), bytes) == 0);
			CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(dst, back.data(), bytes) == 0);
			void *sreq = nullptr, *rreq = nullptr, *mh = nullptr;
			size_t rsize = bytes;
			int tag = 1;
			CHECK(net.isend(sComm, src, bytes, tag, mh, nullptr, &sreq) == ncclSuccess);
			CHECK((sreq != nullptr) == (bytes + 8 <= 8192)); /* eager goes ahead of its receive */
			CHECK(net.irecv(rComm, 1, &dst, &rsize, &tag, &mh, nullptr, &rreq) == ncclSuccess && rreq);
			for (int tries = 0; !sreq && tries < 1000; tries++) {
				CHECK(net.isend(sComm, src, bytes, tag, mh, nullptr, &sreq) == ncclSuccess);
			}
			CHECK(sreq);
			int sdone = 0, rdone = 0, ssize = -1, got = -1;
			for (long spins = 0; (!sdone || !rdone) && spins < 100000000L; spins++) {
				if (!sdone) CHECK(net.test(sreq, &sdone, &ssize) == ncclSuccess);
				if (!rdone) CHECK(net.test(rreq, &rdone, &got) == ncclSuccess);
			}
			CHECK(sdone && rdone && ssize == (int)bytes && got == (int)bytes);
			void *freq = nullptr;
			int isize = (int)bytes;
			CHECK(net.iflush(rComm, 1, &dst, &isize, &mh, &freq) == ncclSuccess && freq);
			int fdone = 0;
			for (long spins = 0; !fdone && spins < 100000000L; spins++) {
				CHECK(net.test(freq, &fdone, nullptr) == ncclSuccess);
			}
			CHECK(fdone);
			CHECK(ofi_amd_gpu_mem_copy_device_to_host(back.data(), dst, bytes) == 0);
			CHECK(memcmp(back.data(), pattern.data(), bytes) == 0);
			CHECK(nccl_net_ofi_gpu_mem_free(src) == 0 && nccl_net_ofi_gpu_mem_free(dst) == 0);
		}
		CHECK(ofi_amd_net_link_destroy(link) == 0);
	}
	{ /* a put-signal through the RMA v15 table over the fabric that moves the bytes: the data is at the
	   * peer, the request completes, and the peer's signal counts one once progress has run on */
		const ncclRma_v15_t table = rma_table_with_this_librarys_data_path();
		constexpr size_t bytes = 300000;
		void *src = nullptr, *dst = nullptr, *counters = nullptr;
		CHECK(nccl_net_ofi_gpu_mem_alloc(&src, bytes) == 0 && nccl_net_ofi_gpu_mem_alloc(&dst, bytes) == 0 &&
		      nccl_net_ofi_gpu_mem_alloc(&counters, 4096) == 0);
		std::vector<uint8_t> pattern(bytes), back(bytes, 0), zero(4096, 0);
		for (size_t i = 0; i < bytes; i++) {
			pattern[i] = (uint8_t)((i * 7 + 3) * 2654435761u >> 24);
		}
		CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(src, pattern.data(), bytes) == 0);
		CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(dst, back.data(), bytes) == 0);
		CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(counters, zero.data(), 4096) == 0);
		const uint64_t signal_base = 0x7f5500000000ull;
		const ofi_amd_gin_signal_region_t region = {signal_base, 4096, counters};
		const uint32_t ids[2] = {0, 1};
		ofi_amd_devfab_t *fab = nullptr;
		ofi_amd_gin_fabric_ops_t ops;
		CHECK(ofi_amd_devfab_create(4, 64, 2, ids, &region, 1, nullptr, &fab) == 0 && ofi_amd_devfab_ops(fab, &ops) == 0);
		ofi_amd_rma_ctx_t *rma = nullptr;
		CHECK(ofi_amd_rma_ctx_create(2, 4, 131072, 64, &ops, 256, 0, &rma) == 0);
		CHECK(ofi_amd_devfab_on_ack(fab, [](void *ctx, uint32_t peer, uint64_t msg) {
			      return ofi_amd_rma_ack_received(static_cast<ofi_amd_rma_ctx_t *>(ctx), peer, msg);
		      }, rma) == 0);
		const uint64_t keys[8] = {1, 2, 3, 4, 5, 6, 7, 8};
		const uint64_t src_addr[2] = {(uint64_t)(uintptr_t)src, (uint64_t)(uintptr_t)src};
		const uint64_t dst_addr[2] = {(uint64_t)(uintptr_t)dst, (uint64_t)(uintptr_t)dst};
		const uint64_t sig_addr[2] = {signal_base, signal_base};
		ofi_amd_rma_mr_t *mr_src = nullptr, *mr_dst = nullptr, *mr_sig = nullptr;
		CHECK(ofi_amd_rma_mr_create(rma, src_addr[0], src_addr, src_addr, keys, &mr_src) == 0);
		CHECK(ofi_amd_rma_mr_create(rma, dst_addr[0], dst_addr, dst_addr, keys, &mr_dst) == 0);
		CHECK(ofi_amd_rma_mr_create(rma, signal_base, sig_addr, sig_addr, keys, &mr_sig) == 0);
		void *request = nullptr;
		CHECK(table.iputSignal(rma, 0, 0, mr_src, bytes, 0, mr_dst, 1, 16, mr_sig, 1, 1 /* increment */, true,
				       ncclRmaOptFlagsDefault, &request) == ncclSuccess && request);
		int done = 0;
		for (long spins = 0; !done && spins < 100000000L; spins++) {
			CHECK(table.test(rma, request, &done) == ncclSuccess);
			if (!done) CHECK(table.rmaProgress(rma) == ncclSuccess);
		}
		CHECK(done);
		CHECK(ofi_amd_devfab_quiesce(fab, 0) == 0);
		CHECK(ofi_amd_gpu_mem_copy_device_to_host(back.data(), dst, bytes) == 0);
		CHECK(memcmp(back.data(), pattern.data(), bytes) == 0);
		uint64_t slots[4] = {9, 9, 9, 9};
		CHECK(ofi_amd_gpu_mem_copy_device_to_host(slots, counters, sizeof(slots)) == 0);
		CHECK(slots[0] == 0 && slots[1] == 0 && slots[2] == 1 && slots[3] == 0);
		CHECK(ofi_amd_rma_mr_destroy(mr_src) == 0 && ofi_amd_rma_mr_destroy(mr_dst) == 0 && ofi_amd_rma_mr_destroy(mr_sig) == 0);
		CHECK(ofi_amd_rma_ctx_destroy(rma) == 0 && ofi_amd_devfab_destroy(fab) == 0);
		CHECK(nccl_net_ofi_gpu_mem_free(src) == 0 && nccl_net_ofi_gpu_mem_free(dst) == 0 && nccl_net_ofi_gpu_mem_free(counters) == 0);
	}
	printf("gpu: ok\n");
	return 0;
}

/* The two entry-point families driven from compiled code at NCCL's depth of 64 requests, through
 * the reference's own structs: messages per second and payload rate of the in-process link and of
 * the device fabric, without an interpreter between the calls.  One JSON line. */
static double now_s()
{
	struct timespec t;
	clock_gettime(CLOCK_MONOTONIC, &t);
	return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

static int rate_checks()
{
	CHECK(nccl_net_ofi_gpu_init() == 0);
	const ncclNet_v12_t net = net_v12_table_with_this_librarys_data_path();
	const ncclRma_v15_t rma_table = rma_table_with_this_librarys_data_path();
	constexpr int kInFlight = 64;
	printf("{");
	{
		ofi_amd_net_link_t *link = nullptr;
		CHECK(ofi_amd_net_link_create(4, 8192, 0, 0, 0, nullptr, &link) == 0);
		void *sComm = ofi_amd_net_link_send_comm(link), *rComm = ofi_amd_net_link_recv_comm(link);
		const size_t sizes[3] = {4096, 1u << 20, 64u << 20};
		printf("\"net_v12\": [");
		for (int which = 0; which < 3; which++) {
			const size_t bytes = sizes[which];
			const int rounds = bytes <= 4096 ? 256 : (bytes <= (1u << 20) ? 32 : 2);
			void *src = nullptr, *dst = nullptr;
			CHECK(nccl_net_ofi_gpu_mem_alloc(&src, bytes * kInFlight) == 0);
			CHECK(nccl_net_ofi_gpu_mem_alloc(&dst, bytes * kInFlight) == 0);
			double best = 1e30;
			for (int pass = 0; pass < 3; pass++) {
				const double t0 = now_s();
				for (int r = 0; r < rounds; r++) {
					void *sreq[kInFlight] = {}, *rreq[kInFlight] = {}, *freq[kInFlight] = {};
					void *mh = nullptr;
					int tag = 1;
					/* the sender is ahead, as in NCCL's pipelines: small messages go eager */
					for (int k = 0; k < kInFlight; k++) {
						CHECK(net.isend(sComm, (char *)src + k * bytes, bytes, tag, mh, nullptr, &sreq[k]) == ncclSuccess);
					}
					for (int k = 0; k < kInFlight; k++) {
						void *d = (char *)dst + k * bytes;
						size_t sz = bytes;
						CHECK(net.irecv(rComm, 1, &d, &sz, &tag, &mh, nullptr, &rreq[k]) == ncclSuccess && rreq[k]);
					}
					for (int k = 0; k < kInFlight; k++) {
						for (long spins = 0; !sreq[k] && spins < 100000000L; spins++) {
							CHECK(net.isend(sComm, (char *)src + k * bytes, bytes, tag, mh, nullptr, &sreq[k]) == ncclSuccess);
						}
						CHECK(sreq[k]);
					}
					int open = 3 * kInFlight; /* a send, a receive and a flush per message */
					for (long spins = 0; open > 0 && spins < 100000000L; spins++) {
						for (int k = 0; k < kInFlight; k++) {
							int done = 0;
							if (sreq[k]) {
								CHECK(net.test(sreq[k], &done, nullptr) == ncclSuccess);
								if (done) { sreq[k] = nullptr; open--; }
							}
							if (rreq[k]) {
								CHECK(net.test(rreq[k], &done, nullptr) == ncclSuccess);
								if (done) {
									rreq[k] = nullptr;
									open--;
									void *d = (char *)dst + k * bytes;
									int isz = (int)bytes;
									CHECK(net.iflush(rComm, 1, &d, &isz, &mh, &freq[k]) == ncclSuccess && freq[k]);
								}
							}
							if (freq[k]) {
								CHECK(net.test(freq[k], &done, nullptr) == ncclSuccess);
								if (done) { freq[k] = nullptr; open--; }
							}
						}
					}
					CHECK(open == 0);
				}
				const double dt = now_s() - t0;
				best = dt < best ? dt : best;
			}
			const double n = (double)rounds * kInFlight;
			printf("%s{\"bytes\": %zu, \"messages\": %.0f, \"msgs_per_s\": %.1f, \"payload_gbs\": %.2f}", which ? ", " : "",
			       bytes, n, n / best, n * (double)bytes / best / 1e9);
			CHECK(nccl_net_ofi_gpu_mem_free(src) == 0 && nccl_net_ofi_gpu_mem_free(dst) == 0);
		}
		printf("], ");
		CHECK(ofi_amd_net_link_destroy(link) == 0);
	}
	{
		const size_t sizes[2] = {4096, 1u << 20};
		printf("\"rma_v15\": [");
		for (int which = 0; which < 2; which++) {
			const size_t bytes = sizes[which];
			const int n_ops = bytes <= 4096 ? 65536 : 8192;
			void *src = nullptr, *dst = nullptr, *counters = nullptr;
			CHECK(nccl_net_ofi_gpu_mem_alloc(&src, bytes * kInFlight) == 0 && nccl_net_ofi_gpu_mem_alloc(&dst, bytes * kInFlight) == 0 &&
			      nccl_net_ofi_gpu_mem_alloc(&counters, 4096) == 0);
			std::vector<uint8_t> zero(4096, 0);
			CHECK(nccl_net_ofi_gpu_mem_copy_host_to_device(counters, zero.data(), 4096) == 0);
			const uint64_t signal_base = 0x7f5500000000ull;
			const ofi_amd_gin_signal_region_t region = {signal_base, 4096, counters};
			const uint32_t ids[2] = {0, 1};
			ofi_amd_devfab_t *fab = nullptr;
			ofi_amd_gin_fabric_ops_t ops;
			CHECK(ofi_amd_devfab_create(4, 256, 2, ids, &region, 1, nullptr, &fab) == 0 && ofi_amd_devfab_ops(fab, &ops) == 0);
			ofi_amd_rma_ctx_t *rma = nullptr;
			CHECK(ofi_amd_rma_ctx_create(2, 4, 131072, 64, &ops, 4096, 0, &rma) == 0);
			CHECK(ofi_amd_devfab_on_ack(fab, [](void *ctx, uint32_t peer, uint64_t msg) {
				      return ofi_amd_rma_ack_received(static_cast<ofi_amd_rma_ctx_t *>(ctx), peer, msg);
			      }, rma) == 0);
			const uint64_t keys[8] = {1, 2, 3, 4, 5, 6, 7, 8};
			const uint64_t a_src[2] = {(uint64_t)(uintptr_t)src, (uint64_t)(uintptr_t)src};
			const uint64_t a_dst[2] = {(uint64_t)(uintptr_t)dst, (uint64_t)(uintptr_t)dst};
			const uint64_t a_sig[2] = {signal_base, signal_base};
			ofi_amd_rma_mr_t *mr_src = nullptr, *mr_dst = nullptr, *mr_sig = nullptr;
			CHECK(ofi_amd_rma_mr_create(rma, a_src[0], a_src, a_src, keys, &mr_src) == 0);
			CHECK(ofi_amd_rma_mr_create(rma, a_dst[0], a_dst, a_dst, keys, &mr_dst) == 0);
			CHECK(ofi_amd_rma_mr_create(rma, signal_base, a_sig, a_sig, keys, &mr_sig) == 0);
			void *open_reqs[kInFlight] = {};
			int head = 0, count = 0;
			const double t0 = now_s();
			for (int i = 0; i < n_ops; i++) {
				const uint64_t off = (uint64_t)(i % kInFlight) * bytes;
				void *req = nullptr;
				CHECK(rma_table.iputSignal(rma, 0, off, mr_src, bytes, off, mr_dst, 1, 8 * (uint64_t)(i % 4), mr_sig, 1, 1,
							   true, ncclRmaOptFlagsDefault, &req) == ncclSuccess && req);
				open_reqs[(head + count++) % kInFlight] = req;
				/* "test the oldest request; if it is not done, progress" (tests/functional/rma.cpp:316-330) */
				for (long spins = 0; (count == kInFlight || (i == n_ops - 1 && count > 0)) && spins < 100000000L; spins++) {
					int done = 0;
					CHECK(rma_table.test(rma, open_reqs[head], &done) == ncclSuccess);
					if (done) {
						head = (head + 1) % kInFlight;
						count--;
					} else {
						CHECK(rma_table.rmaProgress(rma) == ncclSuccess);
					}
				}
			}
			CHECK(count == 0 && ofi_amd_devfab_quiesce(fab, 0) == 0);
			const double dt = now_s() - t0;
			uint64_t slots[4] = {};
			CHECK(ofi_amd_gpu_mem_copy_device_to_host(slots, counters, sizeof(slots)) == 0);
			CHECK(slots[0] + slots[1] + slots[2] + slots[3] == (uint64_t)n_ops);
			printf("%s{\"bytes\": %zu, \"operations\": %d, \"puts_per_s\": %.1f, \"payload_gbs\": %.2f}", which ? ", " : "", bytes,
			       n_ops, n_ops / dt, (double)n_ops * (double)bytes / dt / 1e9);
			CHECK(ofi_amd_rma_mr_destroy(mr_src) == 0 && ofi_amd_rma_mr_destroy(mr_dst) == 0 && ofi_amd_rma_mr_destroy(mr_sig) == 0);
			CHECK(ofi_amd_rma_ctx_destroy(rma) == 0 && ofi_amd_devfab_destroy(fab) == 0);
			CHECK(nccl_net_ofi_gpu_mem_free(src) == 0 && nccl_net_ofi_gpu_mem_free(dst) == 0 && nccl_net_ofi_gpu_mem_free(counters) == 0);
		}
		printf("]");
	}
	printf("}\n");
	return 0;
}

int main(int argc, char **argv)
{
	if (argc == 2 && strcmp(argv[1], "link") == 0) {
		return link_checks();
	}
	if (argc == 2 && strcmp(argv[1], "gpu") == 0) {
		return gpu_checks();
	}
	if (argc == 2 && strcmp(argv[1], "rate") == 0) {
		return rate_checks();
	}
	fprintf(stderr, "usage: %s link|gpu|rate\n", argv[0]);
	return 2;
}

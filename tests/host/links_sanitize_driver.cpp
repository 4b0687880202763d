/*
 * The in-process fabrics and the entry points over them (net_abi.cpp + net_fabric.cpp,
 * rma_abi.cpp + gin_devfab.cpp) and the GIN loop-back run (gin_loopback.cpp) on the CPU under
 * AddressSanitizer + UndefinedBehaviorSanitizer, and under ThreadSanitizer: the device side of
 * the library is replaced, in this test program only, by stand-ins that keep a queue of
 * "launches" and execute them later (host memory plays device memory) -- when this thread
 * ticks the device, or, in the "threaded" mode, on a device thread -- so that tables, sentinels
 * and buffers are used when a GPU would use them, some time after they were handed over.  A
 * table freed or reused too early is then a sanitizer finding, a data race or a wrong byte.
 * Random programs; every byte, reported size and counter is checked.  Test infrastructure:
 * built and run by tests/test_host_sanitizers.py.
 */
#include <algorithm>
#include <atomic>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <thread>
#include <vector>

#include "gin_rings.hpp"
#include "ofi_amd_hotpath.h"
#include "ofi_amd_net_abi.h"
#include "ofi_amd_rma_abi.h"
#include "ofi_amd_sendrecv.h"

namespace {

struct rng_t {
	uint64_t s;
	uint64_t next()
	{
		s += 0x9E3779B97F4A7C15ull;
		uint64_t z = s;
		z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
		z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
		return z ^ (z >> 31);
	}
	uint32_t below(uint32_t n) { return (uint32_t)(next() % n); }
	bool chance(uint32_t pct) { return below(100) < pct; }
};

[[noreturn]] void fail(const char *what, uint64_t a = 0, uint64_t b = 0)
{
	std::fprintf(stderr, "FAILED: %s (%llu, %llu)\n", what, (unsigned long long)a, (unsigned long long)b);
	std::exit(1);
}

#define CHECK(cond)                                  \
	do {                                         \
		if (!(cond)) {                       \
			fail(#cond, __LINE__, 0);    \
		}                                    \
	} while (0)

/* ---- the stand-in device: a queue of launches, executed some calls later ---- */
std::deque<std::function<void()>> g_stream;
std::mutex g_stream_mu;
std::atomic<uint64_t> g_queued{0}; /* launches queued or running */
std::atomic<bool> g_device_thread{false}; /* the launches run on a thread of their own, as a GPU's do */
uint64_t g_launches;

void launch(std::function<void()> f)
{
	std::lock_guard<std::mutex> lock(g_stream_mu);
	g_stream.push_back(std::move(f));
	g_queued.fetch_add(1);
}

/* the oldest queued launch, run outside the lock: one executor at a time, so stream order holds */
bool run_one()
{
	std::function<void()> f;
	{
		std::lock_guard<std::mutex> lock(g_stream_mu);
		if (g_stream.empty()) {
			return false;
		}
		f = std::move(g_stream.front());
		g_stream.pop_front();
	}
	f();
	g_queued.fetch_sub(1);
	return true;
}

void device_tick(uint32_t n)
{
	if (g_device_thread.load()) {
		return;
	}
	while (n-- && run_one()) {
	}
}

bool stream_empty()
{
	return g_queued.load() == 0;
}

std::thread g_device;
std::atomic<bool> g_device_stop{false};
std::atomic<bool> g_device_hold{false}; /* the device thread leaves the queue alone: launches that cannot start yet */

void start_device_thread()
{
	g_device_stop.store(false);
	g_device_thread.store(true);
	g_device = std::thread([]() {
		while (!g_device_stop.load()) {
			if (g_device_hold.load() || !run_one()) {
				std::this_thread::yield();
			}
		}
	});
}

void stop_device_thread()
{
	while (g_queued.load() != 0) {
		std::this_thread::yield();
	}
	g_device_stop.store(true);
	g_device.join();
	g_device_thread.store(false);
}

} // namespace

extern "C" {

int ofi_amd_gpu_init(void) { return 0; }
int ofi_amd_gpu_host_alloc(void **ptr, size_t size)
{
	*ptr = std::aligned_alloc(64, (size + 63) / 64 * 64);
	return *ptr ? 0 : -ENOMEM;
}
int ofi_amd_gpu_host_free(void *ptr)
{
	std::free(ptr);
	return 0;
}
int ofi_amd_gpu_host_get_device_pointer(void **dev_ptr, void *host_ptr)
{
	*dev_ptr = host_ptr;
	return 0;
}
int ofi_amd_gpu_mem_alloc(void **ptr, size_t size) { return ofi_amd_gpu_host_alloc(ptr, size); }
int ofi_amd_gpu_mem_free(void *ptr) { return ofi_amd_gpu_host_free(ptr); }
int ofi_amd_gpu_stream_synchronize(void *)
{
	if (g_device_thread.load()) {
		while (g_queued.load() != 0) {
			std::this_thread::yield();
		}
		return 0;
	}
	device_tick(~0u);
	return 0;
}
int ofi_amd_flush_buffer_fill(void *d_flush_buf, uint64_t sentinel, void *)
{
	launch([=]() {
		for (int w = 0; w < 8; w++) {
			static_cast<uint64_t *>(d_flush_buf)[w] = sentinel;
		}
	});
	return 0;
}
int ofi_amd_flush_post(const void *d_flush_buf, void *slots_dev, uint32_t num_rails, void *)
{
	g_launches++;
	launch([=]() {
		for (uint32_t r = 0; r < num_rails; r++) {
			for (int w = 7; w >= 0; w--) {
				__atomic_store_n(&static_cast<uint64_t *>(slots_dev)[r * 8 + w],
						 static_cast<const uint64_t *>(d_flush_buf)[w], __ATOMIC_RELEASE);
			}
		}
	});
	return 0;
}
int ofi_amd_copy_table_pieces(const uint64_t *d_src, const uint64_t *d_dst, const uint32_t *d_len, uint32_t n,
			      uint32_t max_len, void *)
{
	g_launches++;
	launch([=]() { /* the tables are read when the launch runs, as on the device */
		for (uint32_t i = 0; i < n; i++) {
			const uint32_t bytes = d_len[i] < max_len ? d_len[i] : max_len;
			if (bytes == 64 && d_dst[i] % 8 == 0 && d_src[i] % 8 == 0) {
				/* the shape of a flush read: its landing slots are polled by the host while the
				 * copy is on its way, word by word as a device writes them */
				for (int w = 7; w >= 0; w--) {
					const uint64_t v = reinterpret_cast<const uint64_t *>(static_cast<uintptr_t>(d_src[i]))[w];
					__atomic_store_n(&reinterpret_cast<uint64_t *>(static_cast<uintptr_t>(d_dst[i]))[w], v, __ATOMIC_RELEASE);
				}
				continue;
			}
			std::memmove(reinterpret_cast<void *>(static_cast<uintptr_t>(d_dst[i])),
				     reinterpret_cast<const void *>(static_cast<uintptr_t>(d_src[i])), bytes);
		}
	});
	return 0;
}
int ofi_amd_eager_copy_batch(const void *rx_base, const uint64_t *d_rx_off, const uint32_t *d_recv_len, void *dst_base,
			     const uint64_t *d_dst_off, const uint32_t *d_dst_len, uint32_t n, uint32_t *d_copied,
			     uint32_t *, void *)
{
	g_launches++;
	launch([=]() {
		for (uint32_t i = 0; i < n; i++) {
			const uint32_t bytes = d_recv_len[i] < d_dst_len[i] ? d_recv_len[i] : d_dst_len[i];
			std::memcpy(reinterpret_cast<void *>(reinterpret_cast<uintptr_t>(dst_base) + d_dst_off[i]),
				    static_cast<const uint8_t *>(rx_base) + d_rx_off[i] + OFI_AMD_EAGER_HEADER_SIZE, bytes);
			if (d_copied) {
				d_copied[i] = bytes;
			}
		}
	});
	return 0;
}
int ofi_amd_gin_signal_apply(const ofi_amd_gin_signal_work_t *d_work, uint32_t n, const ofi_amd_gin_signal_region_t *regions,
			     uint32_t n_regions, uint32_t *, void *)
{
	g_launches++;
	std::vector<ofi_amd_gin_signal_region_t> regs(regions, regions + n_regions); /* passed by value to a kernel */
	launch([=]() {
		for (uint32_t i = 0; i < n; i++) {
			for (const ofi_amd_gin_signal_region_t &r : regs) {
				if (d_work[i].base == r.base && d_work[i].offset + 8 <= r.size) {
					static_cast<uint64_t *>(r.d_counters)[d_work[i].offset / 8] += d_work[i].value;
					break;
				}
			}
		}
	});
	return 0;
}

int ofi_amd_gin_signal_apply_post(const ofi_amd_gin_signal_work_t *d_work, uint32_t n, const ofi_amd_gin_signal_region_t *regions,
				  uint32_t n_regions, uint32_t *d_rejected, const void *d_flush_buf, void *slots_dev,
				  uint32_t num_rails, void *stream)
{
	if (n > 65536) {
		return -E2BIG;
	}
	if (n != 0) {
		const int rc = ofi_amd_gin_signal_apply(d_work, n, regions, n_regions, d_rejected, stream);
		if (rc != 0) {
			return rc;
		}
		g_launches--; /* one launch on the device, two entries in this queue */
	}
	return ofi_amd_flush_post(d_flush_buf, slots_dev, num_rails, stream);
}

} /* extern "C" */

namespace {

constexpr int kOk = ncclSuccess;

/* ------------------------------------------------------------------ net entry points */

struct message_t {
	size_t size;
	int tag;
	std::vector<uint8_t> bytes;
	void *req = nullptr;
	int reported = -1;
};

struct receive_t {
	std::vector<int> tags;
	std::vector<size_t> caps;
	std::vector<std::vector<uint8_t>> bufs;
	void *req = nullptr, *flush = nullptr;
	bool done = false;
	int sizes[8];
};

void run_net(uint64_t seed, int rounds)
{
	rng_t rng{ seed };
	ofi_amd_net_link_t *link = nullptr;
	const uint32_t rails = 1 + rng.below(4), rx_buffers = rng.chance(50) ? 4 + rng.below(8) : 0;
	CHECK(ofi_amd_net_link_create(rails, rng.chance(85) ? 8192 : -1, 0, 0, rx_buffers, nullptr, &link) == 0);
	void *sComm = ofi_amd_net_link_send_comm(link), *rComm = ofi_amd_net_link_recv_comm(link);
	const size_t choices[] = { 0, 1, 7, 8, 1000, 8184, 8185, 65536, 131072, 131073, 300000 };
	for (int round = 0; round < rounds; round++) {
		/* receives of 1..8 sub-receives; one message per sub-receive */
		std::vector<receive_t> recvs(1 + rng.below(6));
		std::vector<message_t> msgs;
		for (receive_t &r : recvs) {
			const int n = 1 + (int)rng.below(8);
			std::vector<int> pool = { 1, 2, 3, 4, 5, 6, 7, 8 };
			for (int i = 0; i < n; i++) {
				const size_t size = choices[rng.below(sizeof(choices) / sizeof(choices[0]))];
				const size_t cap = rng.chance(75) ? size : choices[rng.below(sizeof(choices) / sizeof(choices[0]))];
				const size_t pick = rng.below((uint32_t)pool.size());
				r.tags.push_back(pool[pick]); /* distinct within a request, shared between requests */
				pool.erase(pool.begin() + (long)pick);
				r.caps.push_back(cap);
				r.bufs.emplace_back(cap + 16, (uint8_t)0xCD);
				message_t m;
				m.size = size;
				m.tag = r.tags.back();
				m.bytes.resize(size ? size : 1);
				for (uint8_t &b : m.bytes) {
					b = (uint8_t)rng.next();
				}
				msgs.push_back(std::move(m));
			}
		}
		/* The sends of one receive go out in any order, receive after receive: once a sender has
		 * begun a grouped receive's control message, every send up to the group's count must find
		 * its tag there (update_send_data_from_remote, src/nccl_ofi_rdma.cpp:574-640). */
		std::deque<size_t> sendq;
		for (size_t r = 0, first = 0; r < recvs.size(); first += recvs[r].tags.size(), r++) {
			std::vector<size_t> idx(recvs[r].tags.size());
			for (size_t i = 0; i < idx.size(); i++) {
				idx[i] = first + i;
			}
			for (size_t i = idx.size(); i > 1; i--) {
				std::swap(idx[i - 1], idx[rng.below((uint32_t)i)]);
			}
			sendq.insert(sendq.end(), idx.begin(), idx.end());
		}
		const bool late = rng.chance(60);
		size_t posted = 0;
		auto post_some_receives = [&](size_t upto) {
			for (; posted < upto && posted < recvs.size(); posted++) {
				receive_t &r = recvs[posted];
				void *data[8], *mh[8];
				size_t caps[8];
				int tags[8];
				for (size_t i = 0; i < r.tags.size(); i++) {
					data[i] = r.bufs[i].data();
					mh[i] = reinterpret_cast<void *>(0x1000 + i);
					caps[i] = r.caps[i];
					tags[i] = r.tags[i];
				}
				for (int tries = 0; !r.req; tries++) {
					CHECK(tries < 100000);
					CHECK(ofi_amd_net_irecv(rComm, (int)r.tags.size(), data, caps, tags, mh, nullptr, &r.req) == kOk);
					device_tick(rng.below(4));
				}
			}
		};
		if (!late) {
			post_some_receives(recvs.size());
		}
		/* post_sends_interleaved with polling in between */
		for (int spins = 0; !sendq.empty() || std::any_of(msgs.begin(), msgs.end(), [](const message_t &m) { return m.req; }) ||
				    std::any_of(recvs.begin(), recvs.end(), [](const receive_t &r) { return !r.done || r.flush; });
		     spins++) {
			CHECK(spins < 2000000);
			while (!sendq.empty()) {
				message_t &m = msgs[sendq.front()];
				CHECK(ofi_amd_net_isend(sComm, m.bytes.data(), m.size, m.tag, nullptr, nullptr, &m.req) == kOk);
				if (!m.req) {
					break; /* call again later: nothing overtakes it */
				}
				sendq.pop_front();
				if (rng.chance(30)) {
					break;
				}
			}
			post_some_receives(late ? posted + 1 + rng.below(3) : recvs.size());
			device_tick(rng.below(6));
			for (message_t &m : msgs) {
				int done = 0, size = -1;
				if (m.req) {
					CHECK(ofi_amd_net_test(m.req, &done, &size) == kOk);
					if (done) {
						m.req = nullptr;
						m.reported = size;
					}
				}
			}
			for (size_t k = 0; k < posted; k++) {
				receive_t &r = recvs[k];
				int done = 0;
				if (!r.done) {
					CHECK(ofi_amd_net_test(r.req, &done, r.sizes) == kOk);
					if (done) {
						r.done = true;
						void *data[8], *mh[8];
						int isz[8];
						for (size_t i = 0; i < r.tags.size(); i++) {
							data[i] = r.bufs[i].data();
							mh[i] = nullptr;
							isz[i] = r.sizes[i];
						}
						CHECK(ofi_amd_net_iflush(rComm, (int)r.tags.size(), data, isz, mh, &r.flush) == kOk);
					}
				} else if (r.flush) {
					CHECK(ofi_amd_net_test(r.flush, &done, nullptr) == kOk);
					if (done) {
						r.flush = nullptr;
					}
				}
			}
		}
		/* the k-th message of a tag is in the k-th (sub-)receive of that tag */
		std::map<int, std::vector<std::pair<size_t, size_t>>> slots;
		for (size_t r = 0; r < recvs.size(); r++) {
			for (size_t i = 0; i < recvs[r].tags.size(); i++) {
				slots[recvs[r].tags[i]].push_back({ r, i });
			}
		}
		std::map<int, std::vector<size_t>> order; /* messages were generated receive by receive: index order per tag */
		for (size_t i = 0; i < msgs.size(); i++) {
			order[msgs[i].tag].push_back(i);
		}
		for (auto &kv : order) {
			for (size_t k = 0; k < kv.second.size(); k++) {
				const message_t &m = msgs[kv.second[k]];
				const auto [r, i] = slots[kv.first][k];
				const size_t moved = m.size < recvs[r].caps[i] ? m.size : recvs[r].caps[i];
				CHECK(std::memcmp(recvs[r].bufs[i].data(), m.bytes.data(), moved) == 0);
				for (size_t b = moved; b < recvs[r].bufs[i].size(); b++) {
					CHECK(recvs[r].bufs[i][b] == 0xCD);
				}
				CHECK((size_t)recvs[r].sizes[i] == moved);
				CHECK((size_t)m.reported == moved);
			}
		}
	}
	ofi_amd_net_link_stats_t st;
	CHECK(ofi_amd_net_link_stats(link, &st) == 0 && st.eager_sends + st.write_sends > 0);
	CHECK(ofi_amd_net_link_destroy(link) == 0);
}

/* ------------------------------------------------------------------ RMA entry points */

void run_rma(uint64_t seed, int n_ops)
{
	rng_t rng{ seed };
	const uint32_t nranks = 2 + rng.below(3), rails = 1 + rng.below(4);
	const size_t window = 1u << 20;
	std::vector<uint8_t> src(window);
	for (uint8_t &b : src) {
		b = (uint8_t)rng.next();
	}
	std::vector<std::vector<uint8_t>> dst(nranks, std::vector<uint8_t>(window, 0xCD)), want = dst;
	std::vector<std::vector<uint64_t>> counters(nranks, std::vector<uint64_t>(64, 0)), want_cnt = counters;
	const uint64_t signal_base = 0x7f5500000000ull;
	std::vector<ofi_amd_gin_signal_region_t> regions;
	std::vector<uint32_t> ids;
	for (uint32_t r = 0; r < nranks; r++) {
		regions.push_back({ signal_base + ((uint64_t)r << 20), 512, counters[r].data() });
		ids.push_back(r);
	}
	ofi_amd_devfab_t *fab = nullptr;
	ofi_amd_gin_fabric_ops_t ops;
	CHECK(ofi_amd_devfab_create(rails, 4 + rng.below(60), nranks, ids.data(), regions.data(), nranks, nullptr, &fab) == 0);
	CHECK(ofi_amd_devfab_ops(fab, &ops) == 0);
	ofi_amd_rma_ctx_t *ctx = nullptr;
	CHECK(ofi_amd_rma_ctx_create(nranks, rails, 4096, 64, &ops, 1024, 2000, &ctx) == 0);
	CHECK(ofi_amd_devfab_on_ack(fab, [](void *c, uint32_t peer, uint64_t msg) {
		      return ofi_amd_rma_ack_received(static_cast<ofi_amd_rma_ctx_t *>(c), peer, msg);
	      }, ctx) == 0);
	std::vector<uint64_t> a_src(nranks, (uint64_t)(uintptr_t)src.data()), a_dst, a_sig, keys(nranks * 4, 7);
	for (uint32_t r = 0; r < nranks; r++) {
		a_dst.push_back((uint64_t)(uintptr_t)dst[r].data());
		a_sig.push_back(signal_base + ((uint64_t)r << 20));
	}
	ofi_amd_rma_mr_t *mr_src = nullptr, *mr_dst = nullptr, *mr_sig = nullptr;
	CHECK(ofi_amd_rma_mr_create(ctx, a_src[0], a_src.data(), a_src.data(), keys.data(), &mr_src) == 0);
	CHECK(ofi_amd_rma_mr_create(ctx, a_dst[0], a_dst.data(), a_dst.data(), keys.data(), &mr_dst) == 0);
	CHECK(ofi_amd_rma_mr_create(ctx, signal_base, a_sig.data(), a_sig.data(), keys.data(), &mr_sig) == 0);
	std::deque<void *> open;
	std::vector<size_t> cursor(nranks, 0);
	auto poll = [&](size_t keep) {
		for (int spins = 0; open.size() > keep; spins++) {
			CHECK(spins < 2000000);
			int done = 0;
			CHECK(ofi_amd_rma_test(ctx, open.front(), &done) == kOk);
			if (done) {
				open.pop_front();
			} else {
				CHECK(ofi_amd_rma_rmaProgress(ctx) == kOk);
				device_tick(rng.below(5));
			}
		}
	};
	for (int i = 0; i < n_ops; i++) {
		const uint32_t rank = rng.below(nranks);
		const size_t size = rng.chance(10) ? 0 : (rng.chance(60) ? rng.below(3000) : rng.below(40000));
		if (cursor[rank] + size + 8 > window) {
			continue;
		}
		const size_t src_off = rng.below((uint32_t)(window - size)), dst_off = cursor[rank] + rng.below(4);
		cursor[rank] = dst_off + size;
		void *req = nullptr;
		const uint32_t flags = rng.below(2);
		if (size && rng.chance(35)) {
			CHECK(ofi_amd_rma_iput(ctx, 0, src_off, mr_src, size, dst_off, mr_dst, rank, flags, &req) == kOk);
		} else {
			const uint32_t slot = rng.below(8), op = 1 + rng.below(2);
			const uint64_t value = op == 1 ? 1 : rng.next() >> 20;
			CHECK(ofi_amd_rma_iputSignal(ctx, 0, src_off, mr_src, size, dst_off, mr_dst, rank, 8 * slot, mr_sig, value, op, true,
						     flags, &req) == kOk);
			want_cnt[rank][slot] += value;
		}
		CHECK(req);
		open.push_back(req);
		std::memcpy(want[rank].data() + dst_off, src.data() + src_off, size);
		if (open.size() >= 48) {
			CHECK(ofi_amd_devfab_ring_all(fab) == 0);
			poll(rng.below(40));
		}
		device_tick(rng.below(3));
	}
	CHECK(ofi_amd_devfab_ring_all(fab) == 0);
	poll(0);
	/* the stand-in device moves only when ticked: let it run between bounded waits */
	for (int tries = 0;; tries++) {
		CHECK(tries < 10000);
		device_tick(~0u);
		const int rc = ofi_amd_devfab_quiesce(fab, 1);
		if (rc == 0) {
			break;
		}
		CHECK(rc == -ETIMEDOUT);
	}
	for (uint32_t r = 0; r < nranks; r++) {
		CHECK(dst[r] == want[r]);
		CHECK(counters[r] == want_cnt[r]);
	}
	ofi_amd_devfab_stats_t st;
	CHECK(ofi_amd_devfab_stats(fab, &st) == 0 && st.groups > 0);
	CHECK(ofi_amd_rma_mr_destroy(mr_src) == 0 && ofi_amd_rma_mr_destroy(mr_dst) == 0 && ofi_amd_rma_mr_destroy(mr_sig) == 0);
	CHECK(ofi_amd_rma_ctx_destroy(ctx) == 0 && ofi_amd_devfab_destroy(fab) == 0);
}

/* ------------------------------------------------------------------ GIN loop-back run */

/* ofi_amd_gin_loopback_run (gin_loopback.cpp) from end to end: a producer thread pushes random
 * puts, put-signals, signal-only operations and gets into rings in ordinary host memory, the run
 * drains them on this thread, and the stand-in device executes its launches on a thread of its own,
 * so the run's tables are read while it is already filling the next ones.  Bytes, landing
 * buffers, counters and the bookkeeping are compared with a plain replay. */
void run_gin_loopback(uint64_t seed, bool launches_wait_for_the_producer = false)
{
	rng_t rng{ seed };
	/* held: few enough operations for the table sets the run may add (256) */
	const uint32_t nctx = 1 + rng.below(launches_wait_for_the_producer ? 2 : 4), cap = 64;
	const uint64_t ops = launches_wait_for_the_producer ? 300 + rng.below(300) : 600 + rng.below(1500);
	const uint32_t max_size = rng.chance(50) ? 300000 : 40000;
	const size_t src_bytes = 4u << 20;
	std::vector<uint8_t> src(src_bytes), remote(src_bytes);
	for (size_t i = 0; i < src_bytes; i++) {
		src[i] = (uint8_t)rng.next();
		remote[i] = (uint8_t)rng.next();
	}
	std::vector<std::vector<ofi_amd_gin_desc_t>> table(nctx);
	uint64_t dst_pos = 0, land_pos = 0, n_signals = 0, n_bytes = 0, n_gets = 0;
	std::vector<uint64_t> want_cnt(64, 0), n_puts(nctx, 0);
	for (uint32_t c = 0; c < nctx; c++) {
		for (uint64_t i = 0; i < ops; i++) {
			ofi_amd_gin_desc_t d;
			std::memset(&d, 0, sizeof(d));
			d.rank = 1;
			d.context = c;
			d.opt_flags = rng.below(2);
			if (i % 4 == 3) { /* a get: remote handle 3, local handle 4 */
				d.size = rng.chance(90) ? rng.below(max_size) : 0;
				d.src_off = rng.below((uint32_t)(src_bytes - d.size));
				d.dst_off = land_pos + rng.below(24);
				land_pos = d.dst_off + d.size + rng.below(8);
				d.src_mr = 3;
				d.dst_mr = 4;
				d.sig_mr = 0xffff;
				d.kind = 3;
				d.opt_flags = 0;
				n_gets++;
			} else {
				const uint32_t k = rng.below(100);
				d.size = k < 8 ? 0 : (k < 60 ? 1 + rng.below(4095) : 8 + rng.below(max_size));
				d.src_off = rng.below((uint32_t)(src_bytes - d.size));
				d.dst_off = dst_pos + rng.below(24);
				dst_pos = d.dst_off + d.size + rng.below(8);
				const bool signal = d.size == 0 || i % 5 == 4;
				d.signal_op = signal ? 1 + rng.below(2) : 0;
				d.signal_value = d.signal_op == 2 ? rng.next() >> 24 : 0;
				const uint32_t slot = rng.below(64);
				d.signal_off = signal ? 8 * slot : 0;
				d.src_mr = 0;
				d.dst_mr = 1;
				d.sig_mr = signal ? 2 : 0xffff;
				d.kind = signal ? 2 : 1;
				if (signal) {
					want_cnt[slot] += d.signal_op == 1 ? 1 : d.signal_value;
					n_signals++;
				}
				n_puts[c]++;
			}
			n_bytes += d.size;
			table[c].push_back(d);
		}
	}
	std::vector<uint8_t> dst(dst_pos + 64, 0xEE), land(land_pos + 64, 0xDD), want_dst = dst, want_land = land;
	for (uint32_t c = 0; c < nctx; c++) {
		for (const ofi_amd_gin_desc_t &d : table[c]) {
			if (d.kind == 3) {
				std::memcpy(want_land.data() + d.dst_off, remote.data() + d.src_off, d.size);
			} else {
				std::memcpy(want_dst.data() + d.dst_off, src.data() + d.src_off, d.size);
			}
		}
	}
	std::vector<uint64_t> counters(64, 0);
	const uint64_t sig_base = 0x7F5500000000ull;
	ofi_amd_gin_mr_t mrs[5];
	std::memset(mrs, 0, sizeof(mrs));
	mrs[0].local_base = (uint64_t)(uintptr_t)src.data();
	mrs[1].remote_address_offset = (uint64_t)(uintptr_t)dst.data();
	mrs[2].remote_address = sig_base;
	mrs[3].remote_address_offset = (uint64_t)(uintptr_t)remote.data();
	mrs[4].local_base = (uint64_t)(uintptr_t)land.data();
	for (int i = 0; i < 5; i++) {
		for (int r = 0; r < 4; r++) {
			mrs[i].key[r] = 0x100 * (i + 1) + r;
		}
	}
	const uint32_t rails = 1u << rng.below(3); /* 1, 2 or 4 */
	std::vector<ofi_amd_gin_comm_t> comms(nctx);
	for (uint32_t c = 0; c < nctx; c++) {
		CHECK(ofi_amd_gin_comm_init(&comms[c], 100 + c, rails, 131072, 64, 0) == 0);
	}
	const ofi_amd_gin_signal_region_t region = { sig_base, 512, counters.data() };

	ofi_amd_gin_rings rings;
	std::memset(&rings, 0, sizeof(rings));
	rings.n_contexts = nctx;
	rings.capacity = cap;
	std::vector<ofi_amd_gin_desc_t> records((size_t)nctx * cap);
	std::vector<uint32_t> sequences((size_t)nctx * cap), enq((size_t)nctx * 16, 0), deq(nctx, 0), status(16, 0);
	for (uint32_t c = 0; c < nctx; c++) {
		for (uint32_t i = 0; i < cap; i++) {
			sequences[(size_t)c * cap + i] = i;
		}
	}
	rings.records = records.data();
	rings.sequences = sequences.data();
	rings.enqueue_pos = enq.data();
	rings.dequeue_pos = deq.data();
	rings.status = status.data();

	const bool own_device = !g_device_thread.load();
	if (own_device) {
		start_device_thread();
	}
	/* The case of the run's stream sharing a hardware queue with the producers' stream: no launch
	 * starts before the producers are through, and they are through only when the run has drained
	 * their rings.  The run must then go on draining into further table sets instead of waiting
	 * for a sentinel that cannot come. */
	g_device_hold.store(launches_wait_for_the_producer);
	std::thread producer([&]() {
		for (uint64_t i = 0; i < ops; i++) {
			for (uint32_t c = 0; c < nctx; c++) {
				for (;;) {
					const int rc = ofi_amd_gin_ring_push(&rings, c, &table[c][i]);
					if (rc == 1) {
						break;
					}
					CHECK(rc == 0); /* full: the run has to drain first */
					std::this_thread::yield();
				}
			}
		}
		g_device_hold.store(false);
	});
	ofi_amd_gin_loopback_stats_t st;
	const uint32_t sq_depth = rng.chance(50) ? 0 : 1 + rng.below(8);
	const uint32_t batch = launches_wait_for_the_producer ? 16 : 16 + rng.below(500); /* held: many sets needed */
	const int rc = ofi_amd_gin_loopback_run(&rings, ops, comms.data(), mrs, 5, &region, 1, rng.below(60), batch,
						sq_depth, sq_depth ? 16 : 1, 20000, nullptr, &st);
	producer.join();
	if (own_device) {
		stop_device_thread();
	} else {
		CHECK(ofi_amd_gpu_stream_synchronize(nullptr) == 0);
	}
	CHECK(rc == 0);
	CHECK(stream_empty());
	CHECK(dst == want_dst);
	CHECK(land == want_land);
	CHECK(counters == want_cnt);
	CHECK(st.descriptors == (uint64_t)nctx * ops && st.signals == n_signals && st.bytes == n_bytes);
	CHECK(st.flush_reads == (n_gets ? rails : 0));
	CHECK(!launches_wait_for_the_producer || st.table_sets_added > 0);
	CHECK(st.tx_completions == st.writes + st.signals + st.acks + st.reads + st.flush_reads);
	for (uint32_t c = 0; c < nctx; c++) {
		CHECK(comms[c].tx_head == n_puts[c] % 16384);
	}
}

/* ------------------------------------------------------------------ send/receive loop-back run */

/* ofi_amd_sendrecv_loopback_run (sendrecv_loopback.cpp): rounds of messages through the send and
 * receive state machines with the library as the wire, launches on the device thread. */
void run_sendrecv_loopback(uint64_t seed)
{
	rng_t rng{ seed };
	const size_t choices[] = { 0, 1, 7, 8, 1000, 8184, 8185, 65536, 131072, 131073, 300000 };
	const uint32_t group = 1 + rng.below(8), inflight = group * (1 + rng.below(64 / group)), rails = 1 + rng.below(4);
	const uint64_t n_msgs = (uint64_t)inflight * (1 + rng.below(6));
	std::vector<uint8_t> src(400000);
	for (uint8_t &b : src) {
		b = (uint8_t)rng.next();
	}
	std::vector<uint64_t> src_addrs, dst_addrs, sizes, caps;
	std::vector<std::vector<uint8_t>> bufs;
	for (uint64_t i = 0; i < n_msgs; i++) {
		const size_t size = choices[rng.below(sizeof(choices) / sizeof(choices[0]))];
		const size_t cap = rng.chance(75) ? size : choices[rng.below(sizeof(choices) / sizeof(choices[0]))];
		sizes.push_back(size);
		caps.push_back(cap);
		src_addrs.push_back((uint64_t)(uintptr_t)src.data() + rng.below((uint32_t)(src.size() - size)));
		bufs.emplace_back(cap + 16 + rng.below(8), (uint8_t)0xCD);
	}
	for (uint64_t i = 0; i < n_msgs; i++) {
		dst_addrs.push_back((uint64_t)(uintptr_t)bufs[i].data());
	}
	std::vector<uint8_t> rx_pool((size_t)inflight * 8320);
	const bool own_device = !g_device_thread.load();
	if (own_device) {
		start_device_thread();
	}
	ofi_amd_sendrecv_loopback_stats_t st;
	const int rc = ofi_amd_sendrecv_loopback_run(src_addrs.data(), dst_addrs.data(), sizes.data(), caps.data(), nullptr, n_msgs,
						     inflight, rails, group, rx_pool.data(), rx_pool.size(), rng.below(2), nullptr, &st);
	if (own_device) {
		stop_device_thread();
	}
	CHECK(rc == 0);
	uint64_t moved_all = 0;
	for (uint64_t i = 0; i < n_msgs; i++) {
		const size_t moved = sizes[i] < caps[i] ? sizes[i] : caps[i];
		CHECK(std::memcmp(bufs[i].data(), reinterpret_cast<const void *>(static_cast<uintptr_t>(src_addrs[i])), moved) == 0);
		for (size_t b = moved; b < bufs[i].size(); b++) {
			CHECK(bufs[i][b] == 0xCD);
		}
		moved_all += moved;
	}
	CHECK(st.messages == n_msgs && st.payload_bytes == moved_all && st.eager_messages + st.write_messages == n_msgs);
}

} // namespace

int main(int argc, char **argv)
{
	const uint64_t seeds = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 6;
	/* "threaded": every launch of the whole program runs on the device thread, for the build under
	 * ThreadSanitizer -- host code that writes a table, a slot or a buffer which a queued launch
	 * still reads (or reads what one still writes) is a data race there.  Otherwise launches run
	 * when this thread ticks the device, some calls after they were queued. */
	const bool threaded = argc > 2 && std::strcmp(argv[2], "threaded") == 0;
	if (threaded) {
		start_device_thread();
	}
	for (uint64_t s = 1; s <= seeds; s++) {
		run_net(s, 30);
		run_net(s + 100, 30);
		run_rma(s, 4000);
		run_rma(s + 100, 4000);
		run_gin_loopback(s);
		if (s % 8 == 1) {
			run_gin_loopback(s + 1000, true);
		}
		run_sendrecv_loopback(s);
		run_sendrecv_loopback(s + 100);
	}
	/* torn down with work in flight: nothing of it may be touched afterwards */
	{
		ofi_amd_net_link_t *link = nullptr;
		CHECK(ofi_amd_net_link_create(4, 8192, 0, 0, 0, nullptr, &link) == 0);
		std::vector<uint8_t> a(100000, 1), b(100000, 0);
		void *sreq = nullptr, *rreq = nullptr, *data = b.data(), *mh = nullptr;
		size_t cap = b.size();
		int tag = 1, done = 0;
		CHECK(ofi_amd_net_irecv(ofi_amd_net_link_recv_comm(link), 1, &data, &cap, &tag, &mh, nullptr, &rreq) == kOk);
		CHECK(ofi_amd_net_isend(ofi_amd_net_link_send_comm(link), a.data(), a.size(), 1, nullptr, nullptr, &sreq) == kOk && sreq);
		CHECK(ofi_amd_net_test(sreq, &done, nullptr) == kOk);
		CHECK(ofi_amd_net_link_destroy(link) == 0);
		CHECK(stream_empty());
	}
	/* what would be a fault on a device is an error code: address 0 with a length, an rx buffer
	 * handed back twice or one the pool does not have */
	{
		ofi_amd_net_link_t *link = nullptr;
		CHECK(ofi_amd_net_link_create(2, 8192, 0, 0, 4, nullptr, &link) == 0);
		void *req = nullptr, *data = nullptr, *mh = nullptr;
		size_t cap = 64;
		int tag = 1;
		CHECK(ofi_amd_net_isend(ofi_amd_net_link_send_comm(link), nullptr, 64, 1, nullptr, nullptr, &req) == ncclInternalError && !req);
		CHECK(ofi_amd_net_irecv(ofi_amd_net_link_recv_comm(link), 1, &data, &cap, &tag, &mh, nullptr, &req) == ncclInternalError && !req);
		cap = 0; /* nothing to receive into: address 0 is as good as any */
		CHECK(ofi_amd_net_irecv(ofi_amd_net_link_recv_comm(link), 1, &data, &cap, &tag, &mh, nullptr, &req) == kOk && req);
		CHECK(ofi_amd_net_link_destroy(link) == 0);

		ofi_amd_netfab_t *fab = nullptr;
		ofi_amd_net_fabric_ops_t s_ops, r_ops;
		CHECK(ofi_amd_netfab_create(2, 4, nullptr, &fab) == 0 && ofi_amd_netfab_ops(fab, &s_ops, &r_ops) == 0);
		CHECK(r_ops.repost_rx(r_ops.end, 0) == -EINVAL);         /* buffer 0 is free already */
		CHECK(r_ops.repost_rx(r_ops.end, 4 * 8320) == -EINVAL);  /* the pool has four */
		CHECK(r_ops.repost_rx(r_ops.end, 17) == -EINVAL);
		CHECK(s_ops.repost_rx(s_ops.end, 0) == -EINVAL);         /* not the receiving end */
		std::vector<uint8_t> payload(100, 7);
		ofi_amd_net_post_t p;
		std::memset(&p, 0, sizeof(p));
		p.kind = OFI_AMD_NET_POST_WRITE;
		p.len = 100;
		p.src = (uint64_t)(uintptr_t)payload.data();
		CHECK(s_ops.post(s_ops.end, &p) == -EINVAL);             /* to address 0 */
		p.dest = p.src;
		p.src = 0;
		CHECK(s_ops.post(s_ops.end, &p) == -EINVAL);             /* from address 0 */
		p.kind = OFI_AMD_NET_POST_EAGER;
		CHECK(s_ops.post(s_ops.end, &p) == -EINVAL);
		p.kind = OFI_AMD_NET_POST_CTRL;
		p.src = p.dest;
		p.dest = ~0ull - 10;                                     /* dest + len wraps */
		CHECK(r_ops.post(r_ops.end, &p) == -EINVAL);
		/* an eager send takes a buffer, the receiving end gives it back once */
		p.kind = OFI_AMD_NET_POST_EAGER;
		p.src = (uint64_t)(uintptr_t)payload.data();
		p.dest = 0;
		CHECK(s_ops.post(s_ops.end, &p) == 0);
		ofi_amd_net_cqe_t cqe[4];
		int n = 0;
		for (int tries = 0; n == 0 && tries < 100; tries++) {
			n = r_ops.cq_read(r_ops.end, cqe, 4);
			device_tick(4);
		}
		CHECK(n == 1 && cqe[0].kind == OFI_AMD_NET_CQ_EAGER && cqe[0].len == 100);
		CHECK(r_ops.repost_rx(r_ops.end, cqe[0].rx_cookie) == 0);
		CHECK(r_ops.repost_rx(r_ops.end, cqe[0].rx_cookie) == -EINVAL);
		CHECK(ofi_amd_netfab_destroy(fab) == 0);

		/* the device fabric: a write to address 0 is found when it would join a launch */
		ofi_amd_devfab_t *dfab = nullptr;
		ofi_amd_gin_fabric_ops_t d_ops;
		const uint32_t peer_id = 0;
		CHECK(ofi_amd_devfab_create(1, 8, 1, &peer_id, nullptr, 0, nullptr, &dfab) == 0 && ofi_amd_devfab_ops(dfab, &d_ops) == 0);
		ofi_amd_gin_post_t w;
		std::memset(&w, 0, sizeof(w));
		w.kind = OFI_AMD_GIN_POST_WRITE;
		w.len = 100;
		w.src = (uint64_t)(uintptr_t)payload.data();
		CHECK(d_ops.post(d_ops.fabric, &w) == 0);
		uint32_t ctxs[4];
		CHECK(d_ops.cq_read(d_ops.fabric, 0, ctxs, 4) == -EFAULT);
		CHECK(ofi_amd_devfab_destroy(dfab) == 0);
	}
	if (threaded) {
		stop_device_thread();
	}
	std::printf("links: entry points, fabrics and loop-back runs clean over %llu seeds, %llu launches on the stand-in device\n",
		    (unsigned long long)seeds, (unsigned long long)g_launches);
	return 0;
}

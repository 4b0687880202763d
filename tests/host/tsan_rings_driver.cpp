/*
 * Host producers and proxy threads on the GIN descriptor rings, and threads sharing one message
 * buffer, under ThreadSanitizer.
 *
 * The rings are built here from ordinary host memory (the product puts them in pinned host memory,
 * which needs a device); push, pop and the proxy loop are the product's own
 * (aws_ofi_nccl_amd/csrc/gin_proxy.cpp).  Several threads push into each ring -- the
 * multi-producer case of include/nccl_ofi_mpsc_ring.h:79-118 -- while
 *   phase 1: ofi_amd_gin_proxy_drain_mt copies the descriptors out with two proxy threads,
 *   phase 2: one thread per ring pops with ofi_amd_gin_ring_pop.
 * Checked: every descriptor arrives exactly once, each producer's descriptors in its own order, a
 * full ring refuses a push, and ThreadSanitizer sees no unordered access to a slot's 64 bytes.
 */
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "gin_rings.hpp"
#include "ofi_amd_sendrecv.h"

namespace {

constexpr uint32_t kContexts = 4;
constexpr uint32_t kCapacity = 64; /* small: producers run into a full ring all the time */
constexpr uint32_t kProducers = 3; /* per ring */

void fail(const char *what, uint64_t a, uint64_t b)
{
	std::fprintf(stderr, "FAILED: %s (%llu, %llu)\n", what, (unsigned long long)a, (unsigned long long)b);
	std::exit(1);
}

ofi_amd_gin_rings make_rings()
{
	ofi_amd_gin_rings r;
	std::memset(&r, 0, sizeof(r));
	r.n_contexts = kContexts;
	r.capacity = kCapacity;
	r.records = static_cast<ofi_amd_gin_desc_t *>(std::calloc((size_t)kContexts * kCapacity, sizeof(ofi_amd_gin_desc_t)));
	r.sequences = static_cast<uint32_t *>(std::calloc((size_t)kContexts * kCapacity, sizeof(uint32_t)));
	r.enqueue_pos = static_cast<uint32_t *>(std::calloc((size_t)kContexts * 16, sizeof(uint32_t)));
	r.dequeue_pos = static_cast<uint32_t *>(std::calloc(kContexts, sizeof(uint32_t)));
	r.status = static_cast<uint32_t *>(std::calloc(16, sizeof(uint32_t)));
	if (!r.records || !r.sequences || !r.enqueue_pos || !r.dequeue_pos || !r.status) {
		fail("allocation", 0, 0);
	}
	for (uint32_t c = 0; c < kContexts; c++) {
		for (uint32_t i = 0; i < kCapacity; i++) {
			r.sequences[(size_t)c * kCapacity + i] = i;
		}
	}
	return r;
}

void free_rings(ofi_amd_gin_rings &r)
{
	std::free(r.records);
	std::free(r.sequences);
	std::free(r.enqueue_pos);
	std::free(r.dequeue_pos);
	std::free(r.status);
}

ofi_amd_gin_desc_t make_desc(uint32_t context, uint32_t producer, uint64_t i)
{
	ofi_amd_gin_desc_t d;
	std::memset(&d, 0, sizeof(d));
	d.src_off = i * 64;
	d.dst_off = i * 64 + 8;
	d.size = 1 + (i % 4096);
	d.signal_off = producer;
	d.signal_value = i;
	d.rank = producer;
	d.signal_op = (uint32_t)(i % 3);
	d.context = context;
	d.kind = d.signal_op ? 2 : 1;
	d.sig_mr = d.signal_op ? 2 : 0xffff;
	return d;
}

/* One producer: `count` descriptors into ring `context`, spinning while the ring is full. */
void produce(ofi_amd_gin_rings *r, uint32_t context, uint32_t producer, uint64_t count, std::atomic<uint64_t> *refused)
{
	uint64_t full = 0;
	for (uint64_t i = 0; i < count; i++) {
		const ofi_amd_gin_desc_t d = make_desc(context, producer, i);
		for (;;) {
			const int rc = ofi_amd_gin_ring_push(r, context, &d);
			if (rc == 1) {
				break;
			}
			if (rc != 0) {
				fail("push", context, (uint64_t)(int64_t)rc);
			}
			full++;
			std::this_thread::yield();
		}
	}
	refused->fetch_add(full);
}

/* Every producer's descriptors, in its own order, each exactly once. */
void check_stream(const ofi_amd_gin_desc_t *got, uint32_t context, uint64_t per_producer)
{
	uint64_t next[kProducers] = {};
	for (uint64_t k = 0; k < per_producer * kProducers; k++) {
		const ofi_amd_gin_desc_t &d = got[k];
		if (d.rank >= kProducers || d.context != context) {
			fail("foreign descriptor", context, k);
		}
		const ofi_amd_gin_desc_t want = make_desc(context, d.rank, next[d.rank]);
		if (std::memcmp(&d, &want, sizeof(d)) != 0) {
			fail("descriptor out of order or torn", context, k);
		}
		next[d.rank]++;
	}
	for (uint32_t p = 0; p < kProducers; p++) {
		if (next[p] != per_producer) {
			fail("producer count", p, next[p]);
		}
	}
}

void phase_proxy_threads(uint64_t per_producer)
{
	ofi_amd_gin_rings r = make_rings();
	const uint64_t per_context = per_producer * kProducers;
	std::vector<ofi_amd_gin_desc_t> out((size_t)kContexts * per_context);
	std::atomic<uint64_t> refused{ 0 };
	std::vector<std::thread> producers;
	for (uint32_t c = 0; c < kContexts; c++) {
		for (uint32_t p = 0; p < kProducers; p++) {
			producers.emplace_back(produce, &r, c, p, per_producer, &refused);
		}
	}
	ofi_amd_gin_proxy_stats_t st;
	const int rc = ofi_amd_gin_proxy_drain_mt(&r, per_context, 1, out.data(), nullptr, nullptr, 0, nullptr, 60000, 2, &st);
	for (auto &t : producers) {
		t.join();
	}
	if (rc != 0) {
		fail("drain", (uint64_t)(int64_t)rc, 0);
	}
	if (st.descriptors != (uint64_t)kContexts * per_context) {
		fail("drained count", st.descriptors, 0);
	}
	for (uint32_t c = 0; c < kContexts; c++) {
		check_stream(out.data() + (size_t)c * per_context, c, per_producer);
		if (r.dequeue_pos[c] != (uint32_t)per_context) {
			fail("dequeue position", c, r.dequeue_pos[c]);
		}
	}
	std::printf("proxy threads: %llu descriptors, %llu pushes refused by a full ring\n",
		    (unsigned long long)st.descriptors, (unsigned long long)refused.load());
	free_rings(r);
}

/* The proxy threads with the whole derivation (mode 3, two threads, every wire record stored): one
 * producer per ring, so each context's descriptor stream is known, and the records must equal a
 * derivation of the same streams done here on one thread; the checksum summed over the contexts
 * must equal a single proxy thread's. */
void phase_proxy_threads_deriving(uint64_t per_context)
{
	ofi_amd_gin_mr_t mrs[3];
	std::memset(mrs, 0, sizeof(mrs));
	for (int i = 0; i < 3; i++) {
		mrs[i].local_base = 0x7e0000000000ull + ((uint64_t)i << 32);
		mrs[i].remote_address = 0x7f0000000000ull + ((uint64_t)i << 32);
		mrs[i].remote_address_offset = (uint64_t)i << 28;
		for (int r = 0; r < 4; r++) {
			mrs[i].key[r] = 0x100 * (i + 1) + r;
		}
	}
	uint64_t checksum[2] = { 0, 0 };
	std::vector<ofi_amd_gin_wire_t> wires[2];
	for (int run = 0; run < 2; run++) {
		ofi_amd_gin_rings r = make_rings();
		std::vector<ofi_amd_gin_comm_t> comms(kContexts);
		for (uint32_t c = 0; c < kContexts; c++) {
			/* ack_model 1: the window never closes, whatever the number of operations */
			if (ofi_amd_gin_comm_init(&comms[c], 10 + c, 4, 131072, 64, 1) != 0) {
				fail("comm_init", c, 0);
			}
		}
		wires[run].resize((size_t)kContexts * per_context);
		std::atomic<uint64_t> refused{ 0 };
		std::vector<std::thread> producers;
		for (uint32_t c = 0; c < kContexts; c++) {
			producers.emplace_back(produce, &r, c, 0u, per_context, &refused);
		}
		ofi_amd_gin_proxy_stats_t st;
		const int rc = ofi_amd_gin_proxy_drain_mt(&r, per_context, 3, nullptr, comms.data(), mrs, 3, wires[run].data(), 60000,
							  run == 0 ? 2 : 1, &st);
		for (auto &t : producers) {
			t.join();
		}
		if (rc != 0 || st.descriptors != (uint64_t)kContexts * per_context) {
			fail("deriving drain", (uint64_t)(int64_t)rc, st.descriptors);
		}
		checksum[run] = st.checksum;
		free_rings(r);
	}
	if (checksum[0] != checksum[1]) {
		fail("checksum depends on the number of proxy threads", checksum[0], checksum[1]);
	}
	for (uint32_t c = 0; c < kContexts; c++) {
		ofi_amd_gin_comm_t comm;
		if (ofi_amd_gin_comm_init(&comm, 10 + c, 4, 131072, 64, 1) != 0) {
			fail("comm_init", c, 1);
		}
		for (uint64_t i = 0; i < per_context; i++) {
			const ofi_amd_gin_desc_t d = make_desc(c, 0, i);
			ofi_amd_gin_wire_t want;
			if (ofi_amd_gin_iput_signal(&comm, mrs, 3, &d, &want) != 0) {
				fail("derivation", c, i);
			}
			for (int run = 0; run < 2; run++) {
				if (std::memcmp(&wires[run][(size_t)c * per_context + i], &want, sizeof(want)) != 0) {
					fail("wire record differs from the one-thread derivation", c, i);
				}
			}
		}
	}
	std::printf("proxy threads deriving: %llu wire records on two threads equal one thread's\n",
		    (unsigned long long)((uint64_t)kContexts * per_context));
}

void phase_pop(uint64_t per_producer)
{
	ofi_amd_gin_rings r = make_rings();
	const uint64_t per_context = per_producer * kProducers;
	std::vector<ofi_amd_gin_desc_t> out((size_t)kContexts * per_context);

	/* a ring that nobody drains takes exactly `capacity` descriptors */
	for (uint32_t i = 0; i < kCapacity + 3; i++) {
		const ofi_amd_gin_desc_t d = make_desc(0, 0, i);
		const int rc = ofi_amd_gin_ring_push(&r, 0, &d);
		if (rc != (i < kCapacity ? 1 : 0)) {
			fail("full ring", i, (uint64_t)(int64_t)rc);
		}
	}
	for (uint32_t i = 0; i < kCapacity; i++) {
		ofi_amd_gin_desc_t d;
		const ofi_amd_gin_desc_t want = make_desc(0, 0, i);
		if (ofi_amd_gin_ring_pop(&r, 0, &d) != 1 || std::memcmp(&d, &want, sizeof(d)) != 0) {
			fail("pop after full", i, 0);
		}
	}
	ofi_amd_gin_desc_t none;
	if (ofi_amd_gin_ring_pop(&r, 0, &none) != 0) {
		fail("pop from an empty ring", 0, 0);
	}

	std::atomic<uint64_t> refused{ 0 };
	std::vector<std::thread> threads;
	for (uint32_t c = 0; c < kContexts; c++) {
		for (uint32_t p = 0; p < kProducers; p++) {
			threads.emplace_back(produce, &r, c, p, per_producer, &refused);
		}
		threads.emplace_back([&r, &out, c, per_context]() {
			uint64_t got = 0;
			while (got < per_context) {
				const int rc = ofi_amd_gin_ring_pop(&r, c, &out[(size_t)c * per_context + got]);
				if (rc == 1) {
					got++;
				} else if (rc == 0) {
					std::this_thread::yield();
				} else {
					fail("pop", c, (uint64_t)(int64_t)rc);
				}
			}
		});
	}
	for (auto &t : threads) {
		t.join();
	}
	for (uint32_t c = 0; c < kContexts; c++) {
		check_stream(out.data() + (size_t)c * per_context, c, per_producer);
	}
	std::printf("pop: %llu descriptors, %llu pushes refused by a full ring\n",
		    (unsigned long long)(kContexts * per_context), (unsigned long long)refused.load());
	free_rings(r);
}

/*
 * The message buffer locks itself, as the reference's does (src/nccl_ofi_msgbuff.cpp): several
 * threads draw sequence numbers from one counter and each inserts, reads back and completes its
 * own.  A number beyond the window is refused (INVALID_IDX / UNAVAILABLE) until the older ones
 * have completed, so the threads advance the window together.
 */
void phase_msgbuff(uint64_t total)
{
	ofi_amd_msgbuff_t *mb = nullptr;
	if (ofi_amd_msgbuff_create(256, 10, 1, &mb) != 0) {
		fail("msgbuff create", 0, 0);
	}
	std::atomic<uint64_t> next{ 0 }, refused{ 0 };
	std::vector<uint64_t> cookies(total);
	auto work = [&]() {
		uint64_t not_yet = 0;
		for (;;) {
			const uint64_t k = next.fetch_add(1);
			if (k >= total) {
				break;
			}
			const uint16_t seq = (uint16_t)((1 + k) & 1023u);
			int status = -1;
			for (;;) {
				const int rc = ofi_amd_msgbuff_insert(mb, seq, &cookies[k], OFI_AMD_MSGBUFF_REQ, &status);
				if (rc == OFI_AMD_MSGBUFF_SUCCESS) {
					break;
				}
				if (rc != OFI_AMD_MSGBUFF_INVALID_IDX || status != OFI_AMD_MSGBUFF_UNAVAILABLE) {
					fail("msgbuff insert", k, (uint64_t)status);
				}
				not_yet++;
				std::this_thread::yield();
			}
			void *elem = nullptr;
			int type = -1;
			if (ofi_amd_msgbuff_retrieve(mb, seq, &elem, &type, &status) != OFI_AMD_MSGBUFF_SUCCESS ||
			    elem != &cookies[k] || type != OFI_AMD_MSGBUFF_REQ || status != OFI_AMD_MSGBUFF_INPROGRESS) {
				fail("msgbuff retrieve", k, (uint64_t)status);
			}
			if (ofi_amd_msgbuff_complete(mb, seq, &status) != OFI_AMD_MSGBUFF_SUCCESS) {
				fail("msgbuff complete", k, (uint64_t)status);
			}
		}
		refused.fetch_add(not_yet);
	};
	std::vector<std::thread> threads;
	for (int t = 0; t < 4; t++) {
		threads.emplace_back(work);
	}
	for (auto &t : threads) {
		t.join();
	}
	std::printf("message buffer: %llu sequence numbers on 4 threads, %llu inserts refused beyond the window\n",
		    (unsigned long long)total, (unsigned long long)refused.load());
	ofi_amd_msgbuff_destroy(mb);
}

} // namespace

int main(int argc, char **argv)
{
	const uint64_t per_producer = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 20000;
	phase_proxy_threads(per_producer);
	phase_proxy_threads_deriving(per_producer);
	phase_pop(per_producer);
	phase_msgbuff(per_producer * 4);
	std::printf("rings clean with %u producers per ring\n", kProducers);
	return 0;
}

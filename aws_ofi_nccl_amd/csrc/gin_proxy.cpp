/*
 * Host side of the GIN descriptor path: ring push/pop with the slot protocol of
 * include/nccl_ofi_mpsc_ring.h:56-163 and the proxy loop that drains all rings and
 * hands each descriptor to the wire derivation of gin_wire.cpp.
 */
#include <cerrno>
#include <chrono>
#include <thread>
#include <vector>
#include <cstring>

#include "gin_derive.hpp"
#include "gin_rings.hpp"

namespace {

inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

/* Order-sensitive fold of n 64-bit words into a running per-context hash. */
inline uint64_t fold_words(uint64_t h, const uint64_t *w, int n)
{
	static const uint64_t K[8] = {
		0x9E3779B97F4A7C15ull, 0xBF58476D1CE4E5B9ull, 0x94D049BB133111EBull, 0xD6E8FEB86659FD93ull,
		0xCA5A826395121157ull, 0x2545F4914F6CDD1Dull, 0xA0761D6478BD642Full, 0xE7037ED1A0B428DBull,
	};
	uint64_t x = 0;
	for (int k = 0; k < n; k++) {
		x += (w[k] + (uint64_t)(k + 1)) * K[k & 7];
	}
	return (rotl64(h, 5) ^ x) * 0x100000001B3ull;
}

} // namespace

extern "C" {

/* nccl_ofi_mpsc_ring::push, include/nccl_ofi_mpsc_ring.h:79-118 */
int ofi_amd_gin_ring_push(ofi_amd_gin_rings_t *r, uint32_t context, const ofi_amd_gin_desc_t *desc)
{
	if (!r || context >= r->n_contexts || !desc) {
		return -EINVAL;
	}
	const uint32_t mask = r->capacity - 1;
	uint32_t *enq = &r->enqueue_pos[context * 16];
	uint32_t *seq = r->sequences + (size_t)context * r->capacity;
	ofi_amd_gin_desc_t *rec = r->records + (size_t)context * r->capacity;

	uint32_t pos = __atomic_load_n(enq, __ATOMIC_RELAXED);
	for (;;) {
		const uint32_t s = __atomic_load_n(&seq[pos & mask], __ATOMIC_ACQUIRE);
		const int32_t diff = (int32_t)s - (int32_t)pos;
		if (diff == 0) {
			if (__atomic_compare_exchange_n(enq, &pos, pos + 1, true, __ATOMIC_RELAXED,
							__ATOMIC_RELAXED)) {
				break;
			}
		} else if (diff < 0) {
			return 0; /* full */
		} else {
			pos = __atomic_load_n(enq, __ATOMIC_RELAXED);
		}
	}
	rec[pos & mask] = *desc;
	__atomic_store_n(&seq[pos & mask], pos + 1, __ATOMIC_RELEASE);
	return 1;
}

/* nccl_ofi_mpsc_ring::pop, :124-144 */
int ofi_amd_gin_ring_pop(ofi_amd_gin_rings_t *r, uint32_t context, ofi_amd_gin_desc_t *desc)
{
	if (!r || context >= r->n_contexts || !desc) {
		return -EINVAL;
	}
	const uint32_t mask = r->capacity - 1;
	uint32_t *seq = r->sequences + (size_t)context * r->capacity;
	const uint32_t pos = r->dequeue_pos[context];
	if (__atomic_load_n(&seq[pos & mask], __ATOMIC_ACQUIRE) != pos + 1) {
		return 0;
	}
	*desc = r->records[(size_t)context * r->capacity + (pos & mask)];
	r->dequeue_pos[context] = pos + 1;
	__atomic_store_n(&seq[pos & mask], pos + r->capacity, __ATOMIC_RELEASE);
	return 1;
}

/* One proxy thread's share: contexts [c_begin, c_end). */
static int drain_contexts(ofi_amd_gin_rings_t *r, uint32_t c_begin, uint32_t c_end,
			  uint64_t ops_per_context, int mode, ofi_amd_gin_desc_t *out_desc,
			  ofi_amd_gin_comm_t *comms, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
			  ofi_amd_gin_wire_t *out_wire, uint32_t timeout_ms,
			  ofi_amd_gin_proxy_stats_t *stats)
{
	using clock = std::chrono::steady_clock;
	const uint32_t nctx = c_end - c_begin, cap = r->capacity, mask = cap - 1;
	const uint32_t burst = cap / 2 < 1024 ? cap / 2 : 1024;

	constexpr uint32_t kScratchWires = 64;
	uint64_t *done = new (std::nothrow) uint64_t[nctx]();
	uint64_t *hash = new (std::nothrow) uint64_t[nctx];
	ofi_amd_gin_wire_t *scratch_wire = new (std::nothrow) ofi_amd_gin_wire_t[kScratchWires]();
	if (!done || !hash || !scratch_wire) {
		delete[] done;
		delete[] hash;
		delete[] scratch_wire;
		return -ENOMEM;
	}
	for (uint32_t k = 0; k < nctx; k++) {
		hash[k] = 0x9E3779B97F4A7C15ull ^ (c_begin + k);
	}

	ofi_amd_gin_proxy_stats_t st;
	std::memset(&st, 0, sizeof(st));
	uint64_t remaining = (uint64_t)nctx * ops_per_context;
	int rc = 0;
	const auto t0 = clock::now();
	auto last_progress = t0;
	uint32_t idle_rounds = 0;

	while (remaining > 0) {
		bool progressed = false;
		for (uint32_t k = 0; k < nctx; k++) {
			if (done[k] >= ops_per_context) {
				continue;
			}
			const uint32_t c = c_begin + k;
			uint32_t *seq = r->sequences + (size_t)c * cap;
			const ofi_amd_gin_desc_t *rec = r->records + (size_t)c * cap;
			const uint32_t start = r->dequeue_pos[c];
			uint32_t pos = start;
			uint64_t want = ops_per_context - done[k];
			uint32_t limit = want < burst ? (uint32_t)want : burst;
			uint64_t h = hash[k];
			/* constant over the burst: the derivation keeps the counters below the rail count */
			const bool fast = mode >= 2 && ofi_amd_gin::derive_fast_path(&comms[c]);

			while (pos - start < limit &&
			       __atomic_load_n(&seq[pos & mask], __ATOMIC_ACQUIRE) == pos + 1) {
				const ofi_amd_gin_desc_t *d = &rec[pos & mask];
				const uint64_t i = done[k] + (pos - start);
				h = fold_words(h, reinterpret_cast<const uint64_t *>(d), 8);
				st.signals += d->signal_op != 0;
				if (mode == 1) {
					out_desc[(size_t)c * ops_per_context + i] = *d;
				} else if (mode >= 2) {
					/* the slot is handed back only after this burst, so the record is
					 * read in place; the wire record goes straight to its output slot */
					/* without an output array the records go round a small array of this thread's
					 * (64 records, 14 KiB: it stays in the core's cache), where a post step would
					 * pick them up */
					ofi_amd_gin_wire_t *wire = out_wire ? &out_wire[(size_t)c * ops_per_context + i]
									    : &scratch_wire[i & (kScratchWires - 1)];
					/* the derivation is inlined here (gin_derive.hpp): the communicator's state
					 * stays in registers from one descriptor of the burst to the next */
					int e;
					if (d->kind == OFI_AMD_GIN_KIND_GET) {
						e = ofi_amd_gin_iget(&comms[c], mrs, n_mrs, d, wire);
					} else if (fast) {
						e = ofi_amd_gin::derive<true>(&comms[c], mrs, n_mrs, d, wire);
					} else {
						e = ofi_amd_gin_iput_signal(&comms[c], mrs, n_mrs, d, wire);
					}
					if (e != 0) {
						rc = e;
						break;
					}
					/* the record is complete in memory here, whoever reads it next: the compiler may
					 * not keep it in registers or drop stores to fields this loop does not read */
					__asm__ volatile("" : : "r"(wire) : "memory");
					st.writes += wire->num_writes;
					if (mode == 3) {
						h = fold_words(h, reinterpret_cast<const uint64_t *>(wire),
							       (int)(sizeof(*wire) / 8));
					}
				}
				pos++;
			}
			if (pos != start) {
				/* hand the slots back in position order (pop, :139-143) */
				for (uint32_t p = start; p != pos; p++) {
					__atomic_store_n(&seq[p & mask], p + cap, __ATOMIC_RELEASE);
				}
				r->dequeue_pos[c] = pos;
				done[k] += pos - start;
				remaining -= pos - start;
				st.descriptors += pos - start;
				hash[k] = h;
				progressed = true;
			} else {
				st.empty_polls++;
			}
			if (rc != 0) {
				break;
			}
		}
		if (rc != 0) {
			break;
		}
		if (progressed) {
			idle_rounds = 0;
			last_progress = clock::now();
		} else if (++idle_rounds >= 64) {
			idle_rounds = 0;
			const auto now = clock::now();
			if (std::chrono::duration_cast<std::chrono::milliseconds>(now - last_progress).count() >
			    (long long)timeout_ms) {
				rc = -ETIMEDOUT;
				break;
			}
		}
	}
	st.seconds = std::chrono::duration<double>(clock::now() - t0).count();
	for (uint32_t k = 0; k < nctx; k++) {
		st.checksum += hash[k];
	}
	*stats = st;
	delete[] done;
	delete[] hash;
	delete[] scratch_wire;
	return rc;
}

int ofi_amd_gin_proxy_drain_mt(ofi_amd_gin_rings_t *r, uint64_t ops_per_context, int mode,
			       ofi_amd_gin_desc_t *out_desc, ofi_amd_gin_comm_t *comms,
			       const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs, ofi_amd_gin_wire_t *out_wire,
			       uint32_t timeout_ms, uint32_t n_threads, ofi_amd_gin_proxy_stats_t *stats)
{
	if (!r || mode < 0 || mode > 3 || (mode == 1 && !out_desc) ||
	    (mode >= 2 && (!comms || !mrs || n_mrs == 0)) ||
	    n_threads < 1 || n_threads > 64) {
		return -EINVAL;
	}
	const uint32_t nctx = r->n_contexts;
	const uint32_t workers = n_threads < nctx ? n_threads : nctx;
	std::vector<ofi_amd_gin_proxy_stats_t> part(workers);
	std::vector<int> rcs(workers, 0);
	const auto t0 = std::chrono::steady_clock::now();
	auto share = [&](uint32_t w) {
		/* contiguous ranges of contexts, sizes differing by at most one */
		const uint32_t lo = (uint32_t)((uint64_t)nctx * w / workers);
		const uint32_t hi = (uint32_t)((uint64_t)nctx * (w + 1) / workers);
		rcs[w] = drain_contexts(r, lo, hi, ops_per_context, mode, out_desc, comms, mrs, n_mrs, out_wire,
					timeout_ms, &part[w]);
	};
	try {
		std::vector<std::thread> threads;
		for (uint32_t w = 1; w < workers; w++) {
			threads.emplace_back(share, w);
		}
		share(0); /* the calling thread is a proxy thread too */
		for (auto &t : threads) {
			t.join();
		}
	} catch (...) {
		return -ENOMEM;
	}
	ofi_amd_gin_proxy_stats_t st;
	std::memset(&st, 0, sizeof(st));
	int rc = 0;
	for (uint32_t w = 0; w < workers; w++) {
		st.descriptors += part[w].descriptors;
		st.signals += part[w].signals;
		st.writes += part[w].writes;
		st.checksum += part[w].checksum;
		st.empty_polls += part[w].empty_polls;
		if (rcs[w] != 0 && rc == 0) {
			rc = rcs[w];
		}
	}
	st.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
	if (stats) {
		*stats = st;
	}
	return rc;
}

int ofi_amd_gin_proxy_drain(ofi_amd_gin_rings_t *r, uint64_t ops_per_context, int mode,
			    ofi_amd_gin_desc_t *out_desc, ofi_amd_gin_comm_t *comms,
			    const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs, ofi_amd_gin_wire_t *out_wire,
			    uint32_t timeout_ms, ofi_amd_gin_proxy_stats_t *stats)
{
	return ofi_amd_gin_proxy_drain_mt(r, ops_per_context, mode, out_desc, comms, mrs, n_mrs, out_wire,
					  timeout_ms, 1, stats);
}

} /* extern "C" */

/*
 * In-process loop-back of the GIN path on one GPU (ofi_amd_gin_loopback_run): descriptors
 * produced on the device are drained, turned into wire records, "transmitted" -- the RDMA
 * writes become device-side copies, the completions and metadata messages go to a receiver,
 * its ACKs come back to the sender -- and the released signals are applied to the counters
 * in HBM.  It composes the library's own entry points and stands where the reference has
 * two processes, a libfabric provider and GDRCopy (tests/functional/rma.cpp,
 * src/rdma/gin/nccl_ofi_gin.cpp:568-864 on the initiator, :1622-1924 on the target).
 */
#include <cerrno>
#include <chrono>
#include <cstring>
#include <new>
#include <vector>

#include "gin_derive.hpp"
#include "gin_rings.hpp"

namespace {

constexpr uint64_t kPiece = 1ull << 31; /* a table entry's length is 32 bits: longer writes take several */
constexpr uint64_t kSentinel = 0xdeadbeefdeadbeefull; /* NCCL_OFI_GIN_FLUSH_SENTINEL_VAL */

/* One launch pair's worth of copies and signal work, in pinned host memory the GPU reads in place. */
struct batch_t {
	uint64_t *src = nullptr, *dst = nullptr;
	uint32_t *len = nullptr;
	ofi_amd_gin_signal_work_t *work = nullptr;
	void *d_src = nullptr, *d_dst = nullptr, *d_len = nullptr, *d_work = nullptr;
	/* one 64-byte flush slot: the sentinel arrives here when the batch's launches are done */
	uint64_t *done_slot = nullptr;
	void *d_done_slot = nullptr;
	uint32_t n_copy = 0, n_work = 0;
	uint32_t max_len = 0; /* longest entry of the copy table */
	bool launched = false;
};

int alloc_pinned(void **host, void **dev, size_t bytes)
{
	int rc = ofi_amd_gpu_host_alloc(host, bytes);
	if (rc != 0) {
		return rc;
	}
	return ofi_amd_gpu_host_get_device_pointer(dev, *host);
}

void free_batch(batch_t &b)
{
	if (b.src) (void)ofi_amd_gpu_host_free(b.src);
	if (b.dst) (void)ofi_amd_gpu_host_free(b.dst);
	if (b.len) (void)ofi_amd_gpu_host_free(b.len);
	if (b.work) (void)ofi_amd_gpu_host_free(b.work);
	if (b.done_slot) (void)ofi_amd_gpu_host_free(b.done_slot);
	b = batch_t();
}

int alloc_batch(batch_t &b, uint32_t cap_copy, uint32_t cap_work)
{
	int rc = alloc_pinned(reinterpret_cast<void **>(&b.src), &b.d_src, sizeof(uint64_t) * cap_copy);
	if (rc == 0) rc = alloc_pinned(reinterpret_cast<void **>(&b.dst), &b.d_dst, sizeof(uint64_t) * cap_copy);
	if (rc == 0) rc = alloc_pinned(reinterpret_cast<void **>(&b.len), &b.d_len, sizeof(uint32_t) * cap_copy);
	if (rc == 0) rc = alloc_pinned(reinterpret_cast<void **>(&b.work), &b.d_work, sizeof(*b.work) * cap_work);
	if (rc == 0) rc = alloc_pinned(reinterpret_cast<void **>(&b.done_slot), &b.d_done_slot, 64);
	if (rc == 0) std::memset(b.done_slot, 0, 64);
	return rc;
}

/* A completion on its way from the "NIC" to the receiver: a write's immediate data, or the slot
 * of a metadata message in the side table (one event in seventy is one, so the 32 bytes do not
 * travel with every event). */
struct event_t {
	uint32_t peer;
	uint32_t imm;
	int32_t meta_slot; /* -1: a write completion */
};
struct meta_msg_t {
	uint64_t word[4];
};

/* Where the proxy thread's time goes: the time-stamp counter is read around the stages of every
 * 17th operation (reading it around all of them would be a tenth of the time measured) and
 * around every launch, and the sums are scaled to the whole run when it ends. */
struct stage_clock_t {
	uint64_t pop_derive = 0, tx_post = 0, wire = 0, progress = 0, rx = 0, launch_wait = 0;
	static uint64_t now() { return __builtin_ia32_rdtsc(); }
};
constexpr uint32_t kSampleEvery = 17; /* a prime: no beat with the caller's progress interval */

struct lcg_t {
	uint64_t s;
	uint32_t next(uint32_t n) /* n < 2^31; multiply-shift instead of a division per event */
	{
		s = s * 6364136223846793005ull + 1442695040888963407ull;
		return (uint32_t)(((s >> 33) * n) >> 31);
	}
};

} // namespace

extern "C" int ofi_amd_gin_loopback_run(ofi_amd_gin_rings_t *r, uint64_t ops_per_context,
					ofi_amd_gin_comm_t *comms, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
					const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
					uint32_t reorder_window, uint32_t batch_writes, uint32_t sq_depth,
					uint32_t progress_interval, uint32_t timeout_ms, void *stream,
					ofi_amd_gin_loopback_stats_t *stats)
{
	if (!r || !comms || !mrs || n_mrs == 0 || !regions || n_regions == 0 || batch_writes == 0 ||
	    batch_writes > (1u << 24) || reorder_window > 2048 || sq_depth > (1u << 20)) {
		return -EINVAL;
	}
	using clock = std::chrono::steady_clock;
	const uint32_t nctx = r->n_contexts;
	/* an op adds at most 4 writes of at most ... pieces; a flush is forced when either table
	 * cannot take one more op's worth */
	const uint32_t cap_copy = batch_writes + 4096, cap_work = batch_writes + 64;

	ofi_amd_gin_loopback_stats_t st;
	std::memset(&st, 0, sizeof(st));
	/* Table sets: two in the ordinary case, one being filled while the other's launches run.  More
	 * are added only when a launched set's sentinel stays away (see flush_inner). */
	constexpr uint32_t kMaxBatches = 256;
	constexpr uint64_t kMaxBatchBytes = 256ull << 20;
	constexpr long long kSentinelGraceMs = 20;
	std::vector<batch_t> batches;
	ofi_amd_gin_rx_t *rx = nullptr;
	ofi_amd_loopfab_t *fab = nullptr;
	ofi_amd_gin_tx_t *tx = nullptr;
	constexpr uint32_t kPool = 1u << 16;
	/* operations whose posts have not all completed, oldest first: positions into a power-of-two
	 * array of kPool entries (an open operation holds a pool entry, so there are never more) */
	std::vector<int32_t> open_ops;
	uint32_t open_head = 0, open_tail = 0;
	std::vector<uint32_t> comm_ids;
	std::vector<event_t> in_flight;
	std::vector<meta_msg_t> meta_msgs; /* metadata messages in flight, and the free slots among them */
	std::vector<int32_t> meta_free;
	std::vector<uint64_t> done;
	int rc = 0;
	try {
		batches.reserve(kMaxBatches); /* references into it stay good while it grows */
		batches.resize(2);
		comm_ids.resize(nctx);
		open_ops.assign(kPool, -1);
		done.assign(nctx, 0);
		in_flight.reserve(reorder_window + 8);
		meta_msgs.resize(reorder_window + 8);
		for (int32_t k = (int32_t)meta_msgs.size(); k > 0; k--) {
			meta_free.push_back(k - 1);
		}
	} catch (...) {
		return -ENOMEM;
	}
	uint32_t num_rails = 1;
	for (uint32_t c = 0; c < nctx; c++) {
		comm_ids[c] = comms[c].comm_id;
		if (comms[c].num_rails < 1 || comms[c].num_rails > OFI_AMD_MAX_NUM_RAILS) {
			return -EINVAL;
		}
		num_rails = comms[c].num_rails > num_rails ? comms[c].num_rails : num_rails;
	}
	/* completion of a batch is observed the reference's way: a sentinel flush read back into a
	 * host slot behind the batch's launches (iflush, src/rdma/gin/nccl_ofi_gin.cpp:941-1003) */
	void *d_flush_buf = nullptr;
	void *fence_slots = nullptr, *d_fence_slots = nullptr; /* iflush: one 64-byte host slot per rail */
	rc = ofi_amd_gin_rx_create(nctx, comm_ids.data(), &rx);
	if (rc == 0) rc = alloc_pinned(&fence_slots, &d_fence_slots, 64 * OFI_AMD_MAX_NUM_RAILS);
	for (int b = 0; b < 2 && rc == 0; b++) {
		rc = alloc_batch(batches[b], cap_copy, cap_work);
	}
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(d_flush_buf, kSentinel, stream);
	/* the initiator's posts go through the progress engine into a fabric with bounded send
	 * queues; the reference's defaults for the CQ drain (include/nccl_ofi_param.h:104-109) */
	if (rc == 0) rc = ofi_amd_loopfab_create(num_rails, sq_depth ? sq_depth : 4096, &fab);
	if (rc == 0) {
		ofi_amd_gin_fabric_ops_t ops;
		rc = ofi_amd_loopfab_ops(fab, &ops);
		if (rc == 0) rc = ofi_amd_gin_tx_create(num_rails, 4, 4, kPool, &ops, &tx);
	}
	auto release = [&]() {
		for (batch_t &b : batches) {
			free_batch(b);
		}
		if (d_flush_buf) (void)ofi_amd_gpu_mem_free(d_flush_buf);
		if (fence_slots) (void)ofi_amd_gpu_host_free(fence_slots);
		if (rx) (void)ofi_amd_gin_rx_destroy(rx);
		if (tx) (void)ofi_amd_gin_tx_destroy(tx);
		if (fab) (void)ofi_amd_loopfab_destroy(fab);
	};
	if (rc != 0) {
		release();
		return rc;
	}

	uint32_t cur = 0;
	uint64_t remaining = (uint64_t)nctx * ops_per_context; /* descriptors the producers still owe */
	const uint64_t batch_bytes = (uint64_t)cap_copy * 20u + (uint64_t)cap_work * sizeof(ofi_amd_gin_signal_work_t) + 64u;
	lcg_t rng{ 0x9E3779B97F4A7C15ull };
	ofi_amd_gin_ack_t acks[64];

	/* copies first, then the signals that were released while they were queued */
	stage_clock_t sc;
	bool sampling = false; /* this operation's stages are being timed */
	auto flush_inner = [&]() -> int {
		batch_t &b = batches[cur];
		if (b.n_copy == 0 && b.n_work == 0) {
			return 0;
		}
		int e = 0;
		if (b.n_copy) {
			/* one table entry per write, every 8 KiB of it a wavefront of its own; a launch holds
			 * at most 2^31 - 1 wavefronts, so a table with very long entries goes in parts */
			const uint64_t per_entry = ((uint64_t)b.max_len + 8191u) / 8192u;
			const uint64_t most = per_entry ? (0x7fff0000ull / per_entry) : b.n_copy;
			const uint32_t part = most < 1 ? 1u : (most < b.n_copy ? (uint32_t)most : b.n_copy);
			for (uint32_t at = 0; at < b.n_copy && e == 0; at += part) {
				const uint32_t cnt = b.n_copy - at < part ? b.n_copy - at : part;
				e = ofi_amd_copy_table_pieces(static_cast<const uint64_t *>(b.d_src) + at,
							      static_cast<const uint64_t *>(b.d_dst) + at,
							      static_cast<const uint32_t *>(b.d_len) + at, cnt, b.max_len, stream);
			}
		}
		/* the signal adds and the sentinel read-back behind them: one launch, up to the number of
		 * items one workgroup takes */
		uint32_t tail_work = b.n_work;
		if (e == 0 && b.n_work > 65536u) {
			e = ofi_amd_gin_signal_apply(static_cast<const ofi_amd_gin_signal_work_t *>(b.d_work), b.n_work,
						     regions, n_regions, nullptr, stream);
			tail_work = 0;
		}
		if (e == 0) {
			__atomic_store_n(&b.done_slot[0], 0ull, __ATOMIC_RELEASE);
			e = ofi_amd_gin_signal_apply_post(static_cast<const ofi_amd_gin_signal_work_t *>(b.d_work), tail_work,
							  regions, n_regions, nullptr, d_flush_buf, b.d_done_slot, 1, stream);
		}
		if (e != 0) {
			return e;
		}
		st.launches++;
		st.copy_entries += b.n_copy;
		st.work_items += b.n_work;
		b.launched = true;
		/* The next set to fill: one that was never launched or whose sentinel has arrived -- its
		 * tables may still be read by its launches until then (not the stream is waited for: the
		 * set just launched keeps running meanwhile).  If none frees up within a grace period the
		 * launches are not running at all: `stream` can share a hardware queue with the stream
		 * the device-side producers run on, and then they start only when the producers have
		 * finished, while the producers wait for this thread to drain their rings.  Waiting would
		 * close that circle, so another set is allocated instead and the draining goes on; the
		 * launches queue up and run once the producers are through. */
		const auto w0 = clock::now();
		for (;;) {
			for (uint32_t k = 1; k <= batches.size(); k++) {
				batch_t &cand = batches[(cur + k) % batches.size()];
				if (!cand.launched || ofi_amd_flush_test(cand.done_slot, 1, kSentinel) == 1) {
					cur = (cur + k) % (uint32_t)batches.size();
					cand.launched = false;
					cand.n_copy = cand.n_work = 0;
					cand.max_len = 0;
					return 0;
				}
			}
			const long long waited = std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - w0).count();
			if (waited > kSentinelGraceMs && remaining > 0 && batches.size() < kMaxBatches &&
			    (batches.size() + 1) * batch_bytes <= kMaxBatchBytes) {
				batches.emplace_back();
				const int a = alloc_batch(batches.back(), cap_copy, cap_work);
				if (a != 0) {
					free_batch(batches.back());
					batches.pop_back();
					return a;
				}
				st.table_sets_added++;
				cur = (uint32_t)batches.size() - 1;
				return 0;
			}
			if (waited > (long long)timeout_ms) {
				return -ETIMEDOUT;
			}
		}
	};
	/* launches and the wait for the other table pair are timed every time, and taken out of the
	 * sampled stage they interrupt */
	uint64_t flush_ticks_in_sample = 0;
	auto flush = [&]() -> int {
		const uint64_t f0 = stage_clock_t::now();
		const int e = flush_inner();
		const uint64_t dt = stage_clock_t::now() - f0;
		sc.launch_wait += dt;
		if (sampling) {
			flush_ticks_in_sample += dt;
		}
		return e;
	};

	/* hands one completion to the receiver */
	auto deliver = [&](const event_t &ev) -> int {
		if (ev.meta_slot >= 0) {
			const int e = ofi_amd_gin_rx_metadata(rx, ev.peer, meta_msgs[(size_t)ev.meta_slot].word);
			meta_free.push_back(ev.meta_slot);
			return e;
		}
		return ofi_amd_gin_rx_write_completion(rx, ev.peer, ev.imm);
	};
	/* collects what the completions delivered so far have released: the target sends its ACKs
	 * back through the same endpoint (send_ack, :267-315), the signal work joins the batch (its
	 * payloads' copies entered the table when their writes left the fabric, so it is behind them) */
	auto collect = [&]() -> int {
		int e = 0;
		for (;;) {
			const uint32_t n = ofi_amd_gin_rx_take_acks(rx, acks, 64);
			for (uint32_t i = 0; i < n && e == 0; i++) {
				e = ofi_amd_gin_tx_send_ack(tx, acks[i].peer, acks[i].msg);
			}
			if (e != 0) {
				return e;
			}
			if (n < 64) {
				break;
			}
		}
		for (;;) {
			batch_t &b = batches[cur];
			const uint32_t n = ofi_amd_gin_rx_take_work(rx, b.work + b.n_work, cap_work - b.n_work);
			b.n_work += n;
			if (b.n_work < cap_work) {
				break;
			}
			e = flush();
			if (e != 0) {
				return e;
			}
		}
		return 0;
	};

	uint32_t uncollected = 0; /* completions delivered since the receiver's ACKs and signal work were fetched */
	auto deliver_some_inner = [&](uint32_t keep) -> int {
		if (in_flight.size() <= keep) {
			return 0;
		}
		while (in_flight.size() > keep) {
			const uint32_t k = rng.next((uint32_t)in_flight.size());
			const event_t ev = in_flight[k];
			in_flight[k] = in_flight.back();
			in_flight.pop_back();
			int e = deliver(ev);
			if (e != 0) {
				return e;
			}
			uncollected++;
		}
		/* what the receiver has released is fetched every 16 completions, and whenever the
		 * caller waits for everything in flight to arrive */
		if (uncollected >= 16 || keep == 0) {
			uncollected = 0;
			return collect();
		}
		return 0;
	};

	auto deliver_some = [&](uint32_t keep) -> int {
		if (!sampling) {
			return deliver_some_inner(keep);
		}
		const uint64_t r0 = stage_clock_t::now();
		const uint64_t fl0 = flush_ticks_in_sample;
		const int e = deliver_some_inner(keep);
		sc.rx += stage_clock_t::now() - r0 - (flush_ticks_in_sample - fl0);
		return e;
	};

	/* The wire and the initiator's progress: what the fabric has transmitted is executed (a write
	 * becomes table entries of the next copy launch and a completion event for the target, a
	 * metadata message an event, an ACK moves the sender's window), then one progress call of
	 * the engine (bounded CQ drain, retry of the refused posts), then test() of the oldest
	 * operations. */
	auto pump = [&]() -> int {
		const uint64_t p0 = sampling ? stage_clock_t::now() : 0;
		const uint64_t fl0 = flush_ticks_in_sample;
		{
			/* read in place: the send-queue entries stay where they are until the progress call
			 * below reads their completions */
			while (const ofi_amd_gin_post_t *next = ofi_amd_loopfab_next_transmitted(fab)) {
				const ofi_amd_gin_post_t &p = *next;
				event_t ev{p.peer, 0, -1};
				if (p.kind == OFI_AMD_GIN_POST_WRITE || p.kind == OFI_AMD_GIN_POST_READ) {
					/* a read is the same copy the other way, and the target hears nothing of it */
					const bool read = p.kind == OFI_AMD_GIN_POST_READ;
					const uint64_t pieces = (p.len + kPiece - 1) / kPiece;
					if (pieces > cap_copy) {
						return -EMSGSIZE; /* a write larger than the table: raise batch_writes */
					}
					if (batches[cur].n_copy + pieces > cap_copy) {
						int e = flush();
						if (e != 0) {
							return e;
						}
					}
					batch_t &b = batches[cur];
					/* a flush read lands in host memory: the copy kernel reaches the pinned slots
					 * through their device address */
					const uint64_t landing = (read && p.peer == OFI_AMD_GIN_PEER_SELF)
									 ? p.src - reinterpret_cast<uintptr_t>(fence_slots) +
										   reinterpret_cast<uintptr_t>(d_fence_slots)
									 : p.src;
					for (uint64_t off = 0; off < p.len; off += kPiece) {
						const uint64_t len = p.len - off < kPiece ? p.len - off : kPiece;
						b.src[b.n_copy] = (read ? p.dest : p.src) + off;
						b.dst[b.n_copy] = (read ? landing : p.dest) + off;
						b.len[b.n_copy] = (uint32_t)len;
						b.max_len = (uint32_t)len > b.max_len ? (uint32_t)len : b.max_len;
						b.n_copy++;
					}
					if (read && p.peer == OFI_AMD_GIN_PEER_SELF) {
						st.flush_reads++;
					} else if (read) {
						st.bytes += p.len;
						st.reads++;
					} else {
						st.bytes += p.len;
						st.writes++;
						ev.imm = p.imm;
						in_flight.push_back(ev);
					}
				} else if (p.kind == OFI_AMD_GIN_POST_META) {
					if (meta_free.empty()) { /* more in flight than the window: grow the table */
						meta_free.push_back((int32_t)meta_msgs.size());
						meta_msgs.emplace_back();
					}
					ev.meta_slot = meta_free.back();
					meta_free.pop_back();
					std::memcpy(meta_msgs[(size_t)ev.meta_slot].word, p.msg, sizeof(p.msg));
					in_flight.push_back(ev);
				} else {
					/* gin_ack_msg_t: rx_consumed in bits 12..25 (handle_ack_completion, :1843-1869) */
					ofi_amd_gin_apply_ack(&comms[p.peer], (uint32_t)(p.msg[0] >> 12) & 0x3fffu);
					st.acks++;
				}
			}
		}
		const uint64_t p1 = sampling ? stage_clock_t::now() : 0;
		int e = ofi_amd_gin_tx_progress(tx);
		while (e == 0 && open_head != open_tail) {
			int done = 0;
			e = ofi_amd_gin_tx_test(tx, open_ops[open_head & (kPool - 1)], &done);
			if (e != 0 || !done) {
				break;
			}
			open_head++;
		}
		if (sampling) {
			sc.wire += p1 - p0 - (flush_ticks_in_sample - fl0);
			sc.progress += stage_clock_t::now() - p1;
		}
		return e;
	};

	const auto t0 = clock::now();
	const uint64_t tsc0 = stage_clock_t::now();
	auto last_progress = t0;
	uint32_t idle = 0;
	ofi_amd_gin_tx_stats_t ts;
	uint32_t since_progress = 0;
	while (remaining > 0 && rc == 0) {
		bool progressed = false;
		for (uint32_t c = 0; c < nctx && rc == 0; c++) {
			/* constant over the burst: the derivation keeps the counters below the rail count */
			const bool fast = ofi_amd_gin::derive_fast_path(&comms[c]);
			auto derive_one = [&](const ofi_amd_gin_desc_t &d, ofi_amd_gin_wire_t *wire) -> int {
				if (d.kind == OFI_AMD_GIN_KIND_GET) {
					return ofi_amd_gin_iget(&comms[c], mrs, n_mrs, &d, wire);
				}
				return fast ? ofi_amd_gin::derive<true>(&comms[c], mrs, n_mrs, &d, wire)
					    : ofi_amd_gin_iput_signal(&comms[c], mrs, n_mrs, &d, wire);
			};
			/* a burst is read in place and its slots are handed back together afterwards, in
			 * position order (nccl_ofi_mpsc_ring::pop, include/nccl_ofi_mpsc_ring.h:124-144, for a
			 * run of positions): no copy of the record, no store per operation into a line
			 * the producers poll */
			const uint32_t cap = r->capacity, mask = cap - 1;
			uint32_t *ring_seq = r->sequences + (size_t)c * cap;
			const ofi_amd_gin_desc_t *ring_rec = r->records + (size_t)c * cap;
			const uint32_t start = r->dequeue_pos[c];
			const uint64_t want = ops_per_context - done[c];
			const uint32_t most = cap / 2 < 256 ? cap / 2 : 256;
			const uint32_t limit = want < most ? (uint32_t)want : most;
			uint32_t pos = start;
			for (; pos - start < limit; pos++) {
				sampling = (st.descriptors % kSampleEvery) == 0;
				const uint64_t s0 = sampling ? stage_clock_t::now() : 0;
				if (__atomic_load_n(&ring_seq[pos & mask], __ATOMIC_ACQUIRE) != pos + 1) {
					break;
				}
				const ofi_amd_gin_desc_t &d = ring_rec[pos & mask];
				ofi_amd_gin_wire_t wire;
				rc = derive_one(d, &wire);
				if (sampling) {
					sc.pop_derive += stage_clock_t::now() - s0;
				}
				const auto w0 = rc == -EAGAIN ? clock::now() : clock::time_point();
				while (rc == -EAGAIN) {
					/* window closed (await_tx_window, :518-537, progresses until it opens): let
					 * everything in flight arrive, which brings the ACKs */
					rc = pump();
					if (rc == 0) rc = deliver_some(0);
					if (rc == 0) rc = pump();
					if (rc == 0) rc = derive_one(d, &wire);
					if (rc == -EAGAIN &&
					    std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - w0).count() >
						    (long long)timeout_ms) {
						rc = -ETIMEDOUT;
					}
				}
				/* room in the request pool for this operation and the ACKs it may trigger: an
				 * operation takes at most 6 entries and an ACK one, so looking every 1,024
				 * operations with 16,384 entries to spare is enough */
				if ((st.descriptors & 1023u) == 0) {
					while (rc == 0) {
						(void)ofi_amd_gin_tx_stats(tx, &ts);
						if (ts.requests + 16384 <= kPool) {
							break;
						}
						rc = pump();
						if (rc == 0) rc = deliver_some(0);
					}
				}
				if (rc != 0) {
					break;
				}
				int32_t req = -1;
				const uint64_t s1 = sampling ? stage_clock_t::now() : 0;
				rc = d.kind == OFI_AMD_GIN_KIND_GET ? ofi_amd_gin_tx_iget(tx, c, &wire, &req)
								   : ofi_amd_gin_tx_iput_signal(tx, c, &wire, &req);
				if (rc != 0) {
					break;
				}
				open_ops[open_tail++ & (kPool - 1)] = req;
				if (sampling) {
					sc.tx_post += stage_clock_t::now() - s1;
				}
				st.signals += wire.has_meta;
				/* NCCL's proxy submits what it has and then calls ginProgress: a progress call
				 * every progress_interval operations */
				if (++since_progress >= progress_interval) {
					since_progress = 0;
					rc = pump();
				}
				if (rc == 0) rc = deliver_some(reorder_window);
				if (rc == 0 && batches[cur].n_copy >= batch_writes) {
					rc = flush();
				}
				done[c]++;
				remaining--;
				st.descriptors++;
				progressed = true;
				sampling = false;
			}
			sampling = false;
			for (uint32_t p = start; p != pos; p++) {
				__atomic_store_n(&ring_seq[p & mask], p + cap, __ATOMIC_RELEASE);
			}
			r->dequeue_pos[c] = pos;
		}
		if (progressed) {
			idle = 0;
			last_progress = clock::now();
		} else if (++idle >= 64) {
			idle = 0;
			if (std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - last_progress).count() >
			    (long long)timeout_ms) {
				rc = -ETIMEDOUT;
			}
		}
	}
	/* The stream may end on operations whose doorbell was deferred for a successor that never
	 * came (NCCL sets the aggregate hint only when more operations follow): ring them.  Then
	 * run the wire, the target and the engine until nothing is left anywhere. */
	const auto d0 = clock::now();
	while (rc == 0) {
		ofi_amd_loopfab_ring_all(fab);
		rc = pump();
		if (rc == 0) rc = deliver_some(0);
		if (rc == 0) rc = pump();
		if (rc != 0) {
			break;
		}
		(void)ofi_amd_gin_tx_stats(tx, &ts);
		if (open_head == open_tail && in_flight.empty() && ts.requests == 0) {
			break;
		}
		if (std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - d0).count() >
		    (long long)timeout_ms) {
			rc = -ETIMEDOUT;
		}
	}
	if (rc == 0 && st.reads > 0) {
		/* the gets are fenced the reference's way (iflush, src/rdma/gin/nccl_ofi_gin.cpp:941-1003):
		 * a 64-byte read per rail from the device flush buffer into host slots, queued behind
		 * everything the reads of the gets became, and polled for the sentinel */
		int32_t fence = -1;
		rc = ofi_amd_gin_tx_iflush(tx, fence_slots, reinterpret_cast<uintptr_t>(d_flush_buf), kSentinel, &fence);
		const auto f0 = clock::now();
		while (rc == 0) {
			rc = pump();
			if (rc == 0 && batches[cur].n_copy > 0) {
				rc = flush(); /* what the fabric has transmitted so far, the fence's reads among it */
			}
			int fenced = 0;
			if (rc == 0) rc = ofi_amd_gin_tx_test(tx, fence, &fenced);
			if (rc != 0 || fenced) {
				break;
			}
			if (std::chrono::duration_cast<std::chrono::milliseconds>(clock::now() - f0).count() >
			    (long long)timeout_ms) {
				rc = -ETIMEDOUT;
			}
		}
		/* the reads' own completions return their requests to the pool */
		while (rc == 0) {
			(void)ofi_amd_gin_tx_stats(tx, &ts);
			if (ts.requests == 0) {
				break;
			}
			rc = pump();
		}
	}
	if (rc == 0) {
		rc = flush();
	}
	(void)ofi_amd_gin_tx_stats(tx, &ts);
	st.posts_refused = ts.refused;
	st.post_retries = ts.retries;
	st.tx_completions = ts.completions;
	st.pending_max = ts.pending_max;
	st.requests_max = ts.requests_max;
	int sync_rc = ofi_amd_gpu_stream_synchronize(stream);
	if (rc == 0) {
		rc = sync_rc;
	}
	st.seconds = std::chrono::duration<double>(clock::now() - t0).count();
	{
		/* ticks -> nanoseconds from this run's own two clocks; sampled stages scaled up */
		const double ns_per_tick = st.seconds * 1e9 / (double)(stage_clock_t::now() - tsc0);
		const double k = ns_per_tick * kSampleEvery;
		st.ns_pop_derive = (uint64_t)(sc.pop_derive * k);
		st.ns_tx_post = (uint64_t)(sc.tx_post * k);
		st.ns_wire = (uint64_t)(sc.wire * k);
		st.ns_progress = (uint64_t)(sc.progress * k);
		st.ns_rx = (uint64_t)(sc.rx * k);
		st.ns_launch_wait = (uint64_t)(sc.launch_wait * ns_per_tick);
	}
	if (stats) {
		*stats = st;
	}
	release();
	return rc;
}

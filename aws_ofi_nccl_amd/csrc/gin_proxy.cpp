/*
 * Host side of the GIN descriptor path: ring push/pop with the slot protocol of
 * include/nccl_ofi_mpsc_ring.h:56-163, the proxy loop that drains all rings,
 * and what the proxy derives from each descriptor -- the initiator part of
 * nccl_ofi_rdma_gin_put_comm::iputSignal, src/rdma/gin/nccl_ofi_gin.cpp:568-864
 * (sequence number, TX window, ACK-request hysteresis, stripes, rail pinning and
 * doorbell deferral, immediate data, 32-byte metadata message).  The libfabric
 * posts themselves (fi_writemsg / fi_sendmsg) are out of scope: the derivation
 * stops at their arguments.
 */
#include <cerrno>
#include <chrono>
#include <thread>
#include <vector>
#include <cstring>

#include "gin_rings.hpp"

namespace {

/* include/rdma/gin/nccl_ofi_gin_types.h:55-113,209 */
constexpr uint32_t kImmCommShift = 1;
constexpr uint32_t kImmSeqShift = 11;
constexpr uint32_t kImmSeqMask = (1u << 13) - 1;
constexpr uint32_t kImmSegCntShift = 24;
constexpr uint32_t kImmAckReqShift = 28;
constexpr uint32_t kCursorMask = (1u << 14) - 1;   /* GIN_RX_CONSUMED_MASK */
constexpr uint32_t kCursorHalf = 1u << 13;         /* GIN_RX_CONSUMED_HALF */
constexpr uint32_t kAckInterval = 64;              /* GIN_ACK_INTERVAL */
constexpr uint32_t kReqsPerDoorbell = 16;          /* GIN_REQS_PER_DOORBELL */
constexpr uint32_t kAckReqThreshold = (kImmSeqMask + 1) / 2;
constexpr uint32_t kSignalInc = 1, kSignalAdd = 2; /* nccl/net.h:28-29 */
constexpr uint32_t kOptAggregate = 1;              /* nccl/rma_v15.h:19-21 */
constexpr uint64_t kStripeAlign = 128;             /* src/nccl_ofi_scheduler.cpp:168 */

inline uint32_t cursor_inc(uint32_t c) { return (c + 1) & kCursorMask; }
inline uint32_t cursor_delta(uint32_t a, uint32_t b) { return (a - b) & kCursorMask; }

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

/* GIN_IMM_SEG_DATA, include/rdma/gin/nccl_ofi_gin_types.h:76-79 */
uint32_t ofi_amd_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return (ack_req << kImmAckReqShift) | (nseg << kImmSegCntShift) | (seq << kImmSeqShift) |
	       (comm_id << kImmCommShift);
}

/* nccl_net_ofi_gin_msg_header_t, :128-145 */
uint64_t ofi_amd_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req)
{
	return ((uint64_t)(comm_id & 0x3ffu) << 2) | ((uint64_t)(seq & kImmSeqMask) << 12) |
	       ((uint64_t)(nseg & 0xfu) << 25) | ((uint64_t)(ack_req & 1u) << 29);
}

/* gin_ack_msg_t, :170-181 */
uint64_t ofi_amd_gin_ack_msg(uint32_t comm_id, uint32_t rx_consumed)
{
	return 1ull | ((uint64_t)(comm_id & 0x3ffu) << 2) | ((uint64_t)(rx_consumed & kCursorMask) << 12);
}

int ofi_amd_gin_comm_init(ofi_amd_gin_comm_t *c, uint32_t comm_id, uint32_t num_rails,
			  uint64_t min_stripe, uint64_t max_small, uint32_t ack_model)
{
	if (!c || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS || min_stripe == 0 ||
	    comm_id >= 1024 || ack_model > 1) {
		return -EINVAL;
	}
	std::memset(c, 0, sizeof(*c));
	c->sched.max_small_msg_size = max_small;
	c->sched.min_stripe_size = min_stripe;
	c->sched.num_rails = (int32_t)num_rails;
	c->comm_id = comm_id;
	c->num_rails = num_rails;
	c->pinned_rail_id = -1;
	c->ack_model = ack_model;
	return 0;
}

/* handle_ack_completion, src/rdma/gin/nccl_ofi_gin.cpp:1843-1869, with apply_rx_consumed,
 * include/rdma/gin/nccl_ofi_gin.h:535-543 */
void ofi_amd_gin_apply_ack(ofi_amd_gin_comm_t *c, uint32_t wire_rx_consumed)
{
	const uint32_t rx = wire_rx_consumed & kCursorMask;
	const uint32_t delta = cursor_delta(rx, c->tx_tail);
	if (delta > 0 && delta <= kCursorHalf) {
		c->tx_tail = rx;
	}
	if (c->has_pending_ack_request &&
	    cursor_delta(rx, c->last_ack_requested_seq) <= kCursorHalf) {
		c->has_pending_ack_request = 0;
	}
}

int ofi_amd_gin_iput_signal(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs,
			    const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out)
{
	const bool aggregate = (d->opt_flags & kOptAggregate) != 0;
	std::memset(out, 0, sizeof(*out));

	if (d->signal_op != 0 && d->signal_op != kSignalInc && d->signal_op != kSignalAdd) {
		return -EINVAL; /* :580-584 */
	}
	const uint32_t seq = c->tx_head & kImmSeqMask; /* :588 */

	/* await_tx_window (:518-537) spins on progress; a pure derivation cannot, so
	 * a full window is handed back to the caller. */
	const uint32_t outstanding = cursor_delta(c->tx_head, c->tx_tail);
	if (outstanding >= kImmSeqMask + 1) {
		return -EAGAIN;
	}

	const bool has_signal = d->signal_op != 0;
	uint32_t ack_req = 0;
	if (outstanding >= kAckReqThreshold) { /* :611-620 */
		if (c->consecutive_puts_without_ack++ >= kAckInterval) {
			ack_req = 1;
			c->consecutive_puts_without_ack = 0;
		}
	}
	if (ack_req) { /* :624-627 */
		c->last_ack_requested_seq = c->tx_head;
		c->has_pending_ack_request = 1;
	}

	bool defer = false;
	uint32_t nseg = has_signal ? 1u : 0u;
	uint32_t rail_id;

	if (d->size > 0) {
		const uint64_t src = mrs[d->src_mr].local_base + d->src_off;
		const ofi_amd_gin_mr_t &dst_mr = mrs[d->dst_mr];
		const uint64_t dest = dst_mr.remote_address_offset + d->dst_off;

		ofi_amd_xfer_info_t xfers[OFI_AMD_MAX_NUM_RAILS];
		const int n = ofi_amd_sched_get_schedule(&c->sched, d->size, kStripeAlign, xfers);
		if (n < 1) {
			return -ENOMEM;
		}
		const uint32_t num_xfers = (uint32_t)n;

		if (num_xfers == 1 && c->pinned_rail_id >= 0) {
			/* ride the open pin so the deferred doorbell is rung on that rail (:698-707) */
			xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
		} else if (num_xfers > 1 && c->pinned_rail_id >= 0) {
			/* a striped op rings every rail it touches; make it touch the pin (:708-726) */
			bool touches = false;
			for (uint32_t i = 0; i < num_xfers; i++) {
				touches |= xfers[i].rail_id == c->pinned_rail_id;
			}
			if (!touches) {
				xfers[0].rail_id = (uint16_t)c->pinned_rail_id;
			}
		}
		defer = num_xfers == 1 && aggregate && (c->pinned_rail_run + 1 < kReqsPerDoorbell);

		nseg += num_xfers;
		out->imm = ofi_amd_gin_imm(c->comm_id, seq, nseg, ack_req); /* :732 */
		rail_id = xfers[0].rail_id;

		for (uint32_t k = 0; k < num_xfers; k++) { /* :737-784 */
			ofi_amd_gin_write_t &w = out->writes[k];
			w.rail = xfers[k].rail_id;
			w.src = src + xfers[k].offset;
			w.len = xfers[k].msg_size;
			w.dest = dest + xfers[k].offset;
			w.key = dst_mr.key[w.rail];
			w.more = ((has_signal && k == 0) || defer) ? 1u : 0u;
		}
		out->num_writes = num_xfers;
	} else {
		/* signal only (:787-793); get_next_rail, nccl_ofi_gin_resources.h:363-368 */
		if (c->pinned_rail_id >= 0) {
			rail_id = (uint32_t)c->pinned_rail_id;
		} else {
			rail_id = c->next_rail_id;
			c->next_rail_id = (c->next_rail_id + 1) % c->num_rails;
		}
		defer = aggregate && (c->pinned_rail_run + 1 < kReqsPerDoorbell);
	}

	if (has_signal) { /* :795-856 */
		out->has_meta = 1;
		out->meta[0] = ofi_amd_gin_meta_header(c->comm_id, seq, nseg, ack_req);
		out->meta[1] = d->sig_mr != 0xffff ? mrs[d->sig_mr].remote_address : 0;
		out->meta[2] = d->signal_off;
		out->meta[3] = d->signal_op == kSignalInc ? 1 : (d->signal_op == kSignalAdd ? d->signal_value : 0);
		out->meta_rail = rail_id;
		out->meta_more = defer ? 1u : 0u;
	}

	if (defer) { /* update_pin, :550-566 */
		c->pinned_rail_id = (int32_t)rail_id;
		c->pinned_rail_run++;
	} else {
		c->pinned_rail_id = -1;
		c->pinned_rail_run = 0;
	}
	c->tx_head = cursor_inc(c->tx_head); /* :860 */

	out->seq = seq;
	out->nseg = nseg;
	out->ack_req = ack_req;

	if (ack_req && c->ack_model == 1) {
		/* the standalone ACK for this op carries rx_consumed == tx_head */
		ofi_amd_gin_apply_ack(c, c->tx_head);
		c->has_pending_ack_request = 0;
	}
	return 0;
}

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
			  ofi_amd_gin_comm_t *comms, const ofi_amd_gin_mr_t *mrs,
			  ofi_amd_gin_wire_t *out_wire, uint32_t timeout_ms,
			  ofi_amd_gin_proxy_stats_t *stats)
{
	using clock = std::chrono::steady_clock;
	const uint32_t nctx = c_end - c_begin, cap = r->capacity, mask = cap - 1;
	const uint32_t burst = cap / 2 < 1024 ? cap / 2 : 1024;

	uint64_t *done = new (std::nothrow) uint64_t[nctx]();
	uint64_t *hash = new (std::nothrow) uint64_t[nctx];
	if (!done || !hash) {
		delete[] done;
		delete[] hash;
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

			while (pos - start < limit &&
			       __atomic_load_n(&seq[pos & mask], __ATOMIC_ACQUIRE) == pos + 1) {
				const ofi_amd_gin_desc_t *d = &rec[pos & mask];
				const uint64_t i = done[k] + (pos - start);
				h = fold_words(h, reinterpret_cast<const uint64_t *>(d), 8);
				st.signals += d->signal_op != 0;
				if (mode == 1) {
					out_desc[(size_t)c * ops_per_context + i] = *d;
				} else if (mode == 2) {
					ofi_amd_gin_wire_t wire;
					ofi_amd_gin_desc_t copy = *d; /* the slot is recycled below */
					int e = ofi_amd_gin_iput_signal(&comms[c], mrs, &copy, &wire);
					if (e != 0) {
						rc = e;
						break;
					}
					st.writes += wire.num_writes;
					h = fold_words(h, reinterpret_cast<const uint64_t *>(&wire),
						       (int)(sizeof(wire) / 8));
					if (out_wire) {
						out_wire[(size_t)c * ops_per_context + i] = wire;
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
	return rc;
}

int ofi_amd_gin_proxy_drain_mt(ofi_amd_gin_rings_t *r, uint64_t ops_per_context, int mode,
			       ofi_amd_gin_desc_t *out_desc, ofi_amd_gin_comm_t *comms,
			       const ofi_amd_gin_mr_t *mrs, ofi_amd_gin_wire_t *out_wire,
			       uint32_t timeout_ms, uint32_t n_threads, ofi_amd_gin_proxy_stats_t *stats)
{
	if (!r || mode < 0 || mode > 2 || (mode == 1 && !out_desc) || (mode == 2 && (!comms || !mrs)) ||
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
		rcs[w] = drain_contexts(r, lo, hi, ops_per_context, mode, out_desc, comms, mrs, out_wire,
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
			    const ofi_amd_gin_mr_t *mrs, ofi_amd_gin_wire_t *out_wire,
			    uint32_t timeout_ms, ofi_amd_gin_proxy_stats_t *stats)
{
	return ofi_amd_gin_proxy_drain_mt(r, ops_per_context, mode, out_desc, comms, mrs, out_wire,
					  timeout_ms, 1, stats);
}

} /* extern "C" */

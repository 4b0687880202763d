/*
 * Host-side differential driver, meant to be built with -fsanitize=address,undefined:
 * the product's plain-C++ state machines (message buffer, send/receive comms, eager receive
 * queue, GIN sender and receiver) run side by side with the CPU oracle on random programs.  Any
 * disagreement, and anything the sanitizers see, ends the run with a non-zero status.
 * Test infrastructure: built and run by tests/test_host_sanitizers.py, CPU only.
 */
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <vector>

#include "ofi_amd_rma_abi.h"
#include "ofi_amd_sendrecv.h"
#include "oracle.h"

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
	std::fprintf(stderr, "MISMATCH: %s (%llu vs %llu)\n", what, (unsigned long long)a, (unsigned long long)b);
	std::exit(1);
}

#define SAME(what, a, b)                                        \
	do {                                                    \
		if ((uint64_t)(a) != (uint64_t)(b)) {           \
			fail(what, (uint64_t)(a), (uint64_t)(b)); \
		}                                               \
	} while (0)

/* ------------------------------------------------------------ message buffer */
void run_msgbuff(uint64_t seed, uint16_t window, uint16_t bits, int steps)
{
	rng_t rng{ seed };
	const uint16_t field = (uint16_t)(1u << bits);
	const uint16_t start = (uint16_t)rng.below(field);
	oracle_msgbuff_t *a = oracle_msgbuff_create(window, bits, start);
	ofi_amd_msgbuff_t *b = nullptr;
	const int rc = ofi_amd_msgbuff_create(window, bits, start, &b);
	SAME("msgbuff create", a != nullptr, rc == 0);
	if (!a) {
		return;
	}
	static char cells[4096];
	uint16_t head = start;
	for (int i = 0; i < steps; i++) {
		const uint16_t idx = (uint16_t)((head + field + rng.below(2u * window + 5u) - window - 2u) % field);
		void *elem = &cells[rng.below(sizeof(cells))];
		int sa = -1, sb = -1, ta = -1, tb = -1;
		void *ea = nullptr, *eb = nullptr;
		switch (rng.below(4)) {
		case 0: {
			const int type = (int)rng.below(2);
			const int ra = oracle_msgbuff_insert(a, idx, elem, type, &sa);
			SAME("insert result", ra, ofi_amd_msgbuff_insert(b, idx, elem, type, &sb));
			if (ra == ORACLE_MSGBUFF_SUCCESS) {
				head = (uint16_t)((idx + 1) % field);
			}
			break;
		}
		case 1:
			SAME("replace result", oracle_msgbuff_replace(a, idx, elem, 1, &sa),
			     ofi_amd_msgbuff_replace(b, idx, elem, 1, &sb));
			break;
		case 2: {
			const int ra = oracle_msgbuff_retrieve(a, idx, &ea, &ta, &sa);
			SAME("retrieve result", ra, ofi_amd_msgbuff_retrieve(b, idx, &eb, &tb, &sb));
			if (ra == ORACLE_MSGBUFF_SUCCESS) {
				SAME("retrieve elem", (uintptr_t)ea, (uintptr_t)eb);
				SAME("retrieve type", ta, tb);
			}
			break;
		}
		default:
			SAME("complete result", oracle_msgbuff_complete(a, idx, &sa), ofi_amd_msgbuff_complete(b, idx, &sb));
			break;
		}
		SAME("status", sa, sb);
	}
	oracle_msgbuff_destroy(a);
	ofi_amd_msgbuff_destroy(b);
}

/* -------------------------------------------------------- send / receive comms */
struct msg_t {
	uint64_t size;
	int32_t tag;
};
struct recv_plan_t {
	int n;
	uint64_t sizes[8];
	int tags[8];
};
struct flight_t {
	int kind; /* 1 eager, 2 write stripe */
	int32_t req_a, req_b;
	oracle_send_action_t act;
	uint32_t stripe;
};

void same_action(const oracle_send_action_t &x, const ofi_amd_send_action_t &y)
{
	SAME("action kind", x.kind, y.kind);
	SAME("action seq", x.msg_seq_num, y.msg_seq_num);
	SAME("action recv_idx", x.recv_idx, y.recv_idx);
	SAME("action imm", x.imm, y.imm);
	SAME("action size", x.size, y.size);
	SAME("action remote", x.remote_buff_offset, y.remote_buff_offset);
	SAME("action xfers", x.num_xfers, y.num_xfers);
	SAME("action no_target_completion", x.no_target_completion, y.no_target_completion);
	SAME("action hdr", std::memcmp(&x.hdr, &y.hdr, sizeof(x.hdr)), 0);
	for (uint32_t k = 0; k < x.num_xfers; k++) {
		SAME("xfer rail", x.xfers[k].rail_id, y.xfers[k].rail_id);
		SAME("xfer offset", x.xfers[k].offset, y.xfers[k].offset);
		SAME("xfer size", x.xfers[k].msg_size, y.xfers[k].msg_size);
	}
	for (int r = 0; r < 4; r++) {
		SAME("action key", x.mr_key[r], y.mr_key[r]);
	}
}

void run_sendrecv(uint64_t seed, uint32_t n_msgs, bool unique_tags)
{
	rng_t rng{ seed };
	static const uint64_t kSizes[] = { 0, 8, 100, 1024, 8184, 8185, 16384, 200000, 600000 };
	std::vector<msg_t> msgs(n_msgs);
	for (uint32_t i = 0; i < n_msgs; i++) {
		msgs[i] = msg_t{ kSizes[rng.below(9)], unique_tags ? (int32_t)(100 + i) : (int32_t)(1 + rng.below(5)) };
	}
	std::vector<recv_plan_t> plans;
	for (uint32_t i = 0; i < n_msgs;) {
		recv_plan_t p{};
		p.n = (int)(1 + rng.below(4));
		if ((uint32_t)p.n > n_msgs - i) {
			p.n = (int)(n_msgs - i);
		}
		for (int k = 0; k < p.n; k++) { /* a rotation of the group's sends */
			const msg_t &m = msgs[i + (uint32_t)((k + 1) % p.n)];
			p.tags[k] = m.tag;
			p.sizes[k] = rng.chance(80) ? m.size : (m.size / 2 ? m.size / 2 : 1);
		}
		plans.push_back(p);
		i += (uint32_t)p.n;
	}

	oracle_send_comm_t *sa = oracle_send_comm_create(77, 4, 8192, 131072, 64);
	oracle_recv_comm_t *ra = oracle_recv_comm_create(4);
	ofi_amd_send_comm_t *sb = nullptr;
	ofi_amd_recv_comm_t *rb = nullptr;
	if (!sa || !ra || ofi_amd_send_comm_create(77, 4, 8192, 131072, 64, &sb) != 0 ||
	    ofi_amd_recv_comm_create(4, &rb) != 0) {
		fail("create comms");
	}
	oracle_ctrl_msg_t *mba = oracle_send_comm_mailbox(sa);
	ofi_amd_ctrl_msg_t *mbb = ofi_amd_send_comm_mailbox(sb);

	std::deque<uint32_t> queue;
	for (uint32_t i = 0; i < n_msgs; i++) {
		queue.push_back(i);
	}
	std::vector<flight_t> wire;
	std::vector<std::pair<int32_t, int32_t>> send_reqs, recv_reqs;
	std::vector<int> recv_n;
	size_t next_plan = 0;
	uint64_t next_dst = 0x10000000, cookie = 1;

	for (int round = 0; round < 300; round++) {
		/* sends: a tag that was told to call again blocks later sends of that tag */
		std::vector<int32_t> blocked;
		std::deque<uint32_t> again;
		for (uint32_t i : queue) {
			bool skip = rng.chance(20);
			for (int32_t t : blocked) {
				skip = skip || t == msgs[i].tag;
			}
			if (skip) {
				blocked.push_back(msgs[i].tag);
				again.push_back(i);
				continue;
			}
			oracle_send_action_t xa;
			ofi_amd_send_action_t xb;
			SAME("send rc", oracle_send_comm_send(sa, msgs[i].size, msgs[i].tag, &xa),
			     ofi_amd_send_comm_send(sb, msgs[i].size, msgs[i].tag, &xb));
			same_action(xa, xb);
			if (xa.kind == ORACLE_SEND_AGAIN) {
				blocked.push_back(msgs[i].tag);
				again.push_back(i);
				continue;
			}
			send_reqs.emplace_back(xa.req, xb.req);
			if (xa.kind == ORACLE_SEND_EAGER) {
				wire.push_back(flight_t{ 1, xa.req, xb.req, xa, 0 });
			} else {
				for (uint32_t k = 0; k < xa.num_xfers; k++) {
					wire.push_back(flight_t{ 2, xa.req, xb.req, xa, k });
				}
			}
		}
		queue.swap(again);
		/* receives */
		for (uint32_t r = rng.below(3); r > 0 && next_plan < plans.size(); r--) {
			const recv_plan_t &p = plans[next_plan];
			uint64_t dsts[8], keys[32];
			for (int k = 0; k < p.n; k++) {
				dsts[k] = next_dst + 0x100000ull * (uint64_t)k;
				for (int q = 0; q < 4; q++) {
					keys[k * 4 + q] = 0xA000 + next_plan * 32 + (uint64_t)(k * 4 + q);
				}
			}
			int32_t qa = -1, qb = -1;
			uint16_t seq_a = 0, seq_b = 0;
			const int rca = oracle_recv_comm_recv(ra, p.n, dsts, p.sizes, p.tags, keys, 0, mba, &qa, &seq_a);
			SAME("recv rc", rca, ofi_amd_recv_comm_recv(rb, p.n, dsts, p.sizes, p.tags, keys, 0, mbb, &qb, &seq_b));
			if (rca != 0) {
				break; /* the receiver is full: try again in a later round */
			}
			SAME("recv seq", seq_a, seq_b);
			SAME("ctrl_sent", oracle_recv_comm_ctrl_sent(ra, qa), ofi_amd_recv_comm_ctrl_sent(rb, qb));
			recv_reqs.emplace_back(qa, qb);
			recv_n.push_back(p.n);
			next_dst += 0x800000;
			next_plan++;
		}
		/* the wire, in random order */
		if (rng.chance(80)) {
			while (!wire.empty()) {
				const size_t k = rng.below((uint32_t)wire.size());
				const flight_t f = wire[k];
				wire[k] = wire.back();
				wire.pop_back();
				if (f.kind == 1) {
					ofi_amd_eager_hdr_t hb;
					std::memcpy(&hb, &f.act.hdr, sizeof(hb));
					SAME("eager arrival",
					     oracle_recv_comm_eager_arrival(ra, f.act.msg_seq_num, &f.act.hdr, (uint32_t)f.act.size, cookie),
					     ofi_amd_recv_comm_eager_arrival(rb, f.act.msg_seq_num, &hb, (uint32_t)f.act.size, cookie));
					cookie++;
				} else {
					const uint64_t len = f.act.xfers[f.stripe].msg_size;
					SAME("write arrival", oracle_recv_comm_write_arrival(ra, f.act.imm, len),
					     ofi_amd_recv_comm_write_arrival(rb, f.act.imm, len));
				}
				SAME("send completion", oracle_send_comm_completion(sa, f.req_a),
				     ofi_amd_send_comm_completion(sb, f.req_b));
			}
		}
		/* eager copies */
		for (;;) {
			oracle_eager_copy_item_t ia[16];
			ofi_amd_eager_copy_item_t ib[16];
			const uint32_t na = oracle_recv_comm_take_copies(ra, ia, 16);
			SAME("copies", na, ofi_amd_recv_comm_take_copies(rb, ib, 16));
			for (uint32_t k = 0; k < na; k++) {
				SAME("copy cookie", ia[k].rx_cookie, ib[k].rx_cookie);
				SAME("copy dst", ia[k].dst, ib[k].dst);
				SAME("copy dst_len", ia[k].dst_len, ib[k].dst_len);
				SAME("copy recv_len", ia[k].recv_len, ib[k].recv_len);
				SAME("copy sub", ia[k].sub_idx, ib[k].sub_idx);
				SAME("copy needs", ia[k].needs_copy, ib[k].needs_copy);
				if (ia[k].needs_copy) {
					SAME("copy done", oracle_recv_comm_copy_done(ra, ia[k].req, ia[k].sub_idx),
					     ofi_amd_recv_comm_copy_done(rb, ib[k].req, ib[k].sub_idx));
				}
			}
			if (na < 16) {
				break;
			}
		}
		/* test() on a random subset of the open requests */
		for (size_t k = 0; k < send_reqs.size(); k++) {
			if (send_reqs[k].first < 0 || !rng.chance(70)) {
				continue;
			}
			int da = 0, db = 0;
			uint64_t za = 0, zb = 0;
			SAME("send test", oracle_send_comm_test(sa, send_reqs[k].first, &da, &za),
			     ofi_amd_send_comm_test(sb, send_reqs[k].second, &db, &zb));
			SAME("send done", da, db);
			if (da) {
				SAME("send size", za, zb);
				send_reqs[k].first = -1;
			}
		}
		for (size_t k = 0; k < recv_reqs.size(); k++) {
			if (recv_reqs[k].first < 0 || !rng.chance(70)) {
				continue;
			}
			int da = 0, db = 0, za[8] = {}, zb[8] = {};
			SAME("recv test", oracle_recv_comm_test(ra, recv_reqs[k].first, &da, za),
			     ofi_amd_recv_comm_test(rb, recv_reqs[k].second, &db, zb));
			SAME("recv done", da, db);
			if (da) {
				for (int q = 0; q < recv_n[k]; q++) {
					SAME("recv size", za[q], zb[q]);
				}
				recv_reqs[k].first = -1;
			}
		}
		oracle_send_state_t ssa;
		ofi_amd_send_state_t ssb;
		oracle_send_comm_state(sa, &ssa);
		ofi_amd_send_comm_state(sb, &ssb);
		static_assert(sizeof(ssa) == sizeof(ssb), "state layouts");
		SAME("send state", std::memcmp(&ssa, &ssb, sizeof(ssa)), 0);
		oracle_recv_state_t rsa;
		ofi_amd_recv_state_t rsb;
		oracle_recv_comm_state(ra, &rsa);
		ofi_amd_recv_comm_state(rb, &rsb);
		static_assert(sizeof(rsa) == sizeof(rsb), "state layouts");
		SAME("recv state", std::memcmp(&rsa, &rsb, sizeof(rsa)), 0);
	}
	if (unique_tags) { /* with one tag per message everything must have been delivered */
		SAME("sends left", queue.size(), 0);
		for (const auto &q : send_reqs) {
			SAME("send still open", q.first, -1);
		}
		for (const auto &q : recv_reqs) {
			SAME("recv still open", q.first, -1);
		}
	}
	oracle_send_comm_destroy(sa);
	oracle_recv_comm_destroy(ra);
	ofi_amd_send_comm_destroy(sb);
	ofi_amd_recv_comm_destroy(rb);
}

/* -------------------------------------------------------- eager receive queue */
void run_rxq(uint64_t seed)
{
	rng_t rng{ seed };
	oracle_eager_rxq_t *a = oracle_eager_rxq_create();
	ofi_amd_eager_rxq_t *b = nullptr;
	if (!a || ofi_amd_eager_rxq_create(&b) != 0) {
		fail("rxq create");
	}
	oracle_eager_tx_t tx;
	oracle_eager_tx_init(&tx);
	std::vector<oracle_eager_entry_t> pending;
	uint64_t cookie = 0;
	for (int i = 0; i < 4000; i++) {
		if (pending.size() < 24 && rng.chance(60)) {
			oracle_eager_hdr_t h;
			oracle_eager_tx_assign(&tx, (int32_t)rng.below(9), &h);
			oracle_eager_entry_t e{};
			e.eager_offset = h.eager_offset;
			e.prev_batch_count = h.prev_batch_count;
			e.eager_seq = h.eager_seq;
			e.tag = h.tag;
			e.cookie = cookie++;
			pending.push_back(e);
			if (rng.chance(40)) {
				oracle_eager_tx_advance(&tx);
			}
		}
		if (!pending.empty() && rng.chance(70)) {
			const size_t k = rng.below((uint32_t)pending.size());
			ofi_amd_eager_entry_t eb;
			static_assert(sizeof(eb) == sizeof(pending[k]), "entry layouts");
			std::memcpy(&eb, &pending[k], sizeof(eb));
			SAME("rxq insert", oracle_eager_rxq_insert(a, &pending[k]), ofi_amd_eager_rxq_insert(b, &eb));
			pending[k] = pending.back();
			pending.pop_back();
			oracle_eager_entry_t oa[8];
			ofi_amd_eager_entry_t ob[8];
			const uint32_t na = oracle_eager_rxq_drain(a, oa, 8);
			SAME("rxq drain", na, ofi_amd_eager_rxq_drain(b, ob, 8));
			SAME("rxq entries", std::memcmp(oa, ob, na * sizeof(oa[0])), 0);
			SAME("rxq pending", oracle_eager_rxq_pending(a), ofi_amd_eager_rxq_pending(b));
		}
	}
	oracle_eager_rxq_destroy(a);
	ofi_amd_eager_rxq_destroy(b);
}

/* --------------------------------------------------------------- GIN receiver */
void run_gin_rx(uint64_t seed, uint32_t n_ops)
{
	rng_t rng{ seed };
	const uint32_t comm_ids[2] = { 5, 9 };
	oracle_gin_rx_t *a = oracle_gin_rx_create(2, comm_ids);
	ofi_amd_gin_rx_t *b = nullptr;
	if (!a || ofi_amd_gin_rx_create(2, comm_ids, &b) != 0) {
		fail("gin rx create");
	}
	oracle_gin_mr_t mrs[3];
	std::memset(mrs, 0, sizeof(mrs));
	mrs[0].local_base = 0x1000000;
	mrs[1].remote_address_offset = 0x2000000;
	mrs[2].remote_address = 0x7F5500000000ull;
	struct event_t {
		uint32_t peer, is_meta, imm;
		uint64_t meta[4];
	};
	std::vector<event_t> flight;
	oracle_gin_comm_t comms[2];
	for (int p = 0; p < 2; p++) {
		oracle_gin_comm_init(&comms[p], comm_ids[p], 4, 131072, 64, 0);
	}
	auto deliver = [&](const event_t &e) {
		if (e.is_meta) {
			SAME("gin meta", oracle_gin_rx_metadata(a, e.peer, e.meta), ofi_amd_gin_rx_metadata(b, e.peer, e.meta));
		} else {
			SAME("gin write", oracle_gin_rx_write(a, e.peer, e.imm), ofi_amd_gin_rx_write_completion(b, e.peer, e.imm));
		}
		oracle_gin_signal_work_t wa[32];
		ofi_amd_gin_signal_work_t wb[32];
		static_assert(sizeof(wa[0]) == sizeof(wb[0]), "work layouts");
		const uint32_t nw = oracle_gin_rx_take_work(a, wa, 32);
		SAME("gin work count", nw, ofi_amd_gin_rx_take_work(b, wb, 32));
		SAME("gin work", std::memcmp(wa, wb, nw * sizeof(wa[0])), 0);
		oracle_gin_ack_t ka[32];
		ofi_amd_gin_ack_t kb[32];
		static_assert(sizeof(ka[0]) == sizeof(kb[0]), "ack layouts");
		const uint32_t nk = oracle_gin_rx_take_acks(a, ka, 32);
		SAME("gin ack count", nk, ofi_amd_gin_rx_take_acks(b, kb, 32));
		SAME("gin acks", std::memcmp(ka, kb, nk * sizeof(ka[0])), 0);
		for (uint32_t k = 0; k < nk; k++) {
			oracle_gin_apply_ack(&comms[ka[k].peer], ka[k].rx_consumed);
		}
	};
	for (uint32_t i = 0; i < n_ops; i++) {
		const uint32_t peer = rng.below(2);
		oracle_gin_desc_t d;
		oracle_gin_gen_desc(seed, peer, i, 1, 3, 1 + rng.below(2), 1, &d);
		oracle_gin_wire_t w;
		if (oracle_gin_iput_signal(&comms[peer], mrs, &d, &w) != 0) {
			while (!flight.empty()) { /* window full: let everything land, then go on */
				const event_t e = flight.back();
				flight.pop_back();
				deliver(e);
			}
			continue;
		}
		for (uint32_t k = 0; k < w.num_writes; k++) {
			flight.push_back(event_t{ peer, 0, w.imm, { 0, 0, 0, 0 } });
		}
		if (w.has_meta) {
			flight.push_back(event_t{ peer, 1, 0, { w.meta[0], w.meta[1], w.meta[2], w.meta[3] } });
		}
		while (flight.size() > 40 || (!flight.empty() && rng.chance(50))) {
			const size_t k = rng.below((uint32_t)flight.size());
			const event_t e = flight[k];
			flight[k] = flight.back();
			flight.pop_back();
			deliver(e);
		}
	}
	while (!flight.empty()) {
		const event_t e = flight.back();
		flight.pop_back();
		deliver(e);
	}
	oracle_gin_rx_destroy(a);
	ofi_amd_gin_rx_destroy(b);
}

/* ----------------------------------------------------------------- GIN sender */
void run_gin_tx(uint64_t seed, uint32_t n_ops, uint32_t ack_model)
{
	rng_t rng{ seed };
	static_assert(sizeof(oracle_gin_comm_t) == sizeof(ofi_amd_gin_comm_t), "comm layouts");
	static_assert(sizeof(oracle_gin_wire_t) == sizeof(ofi_amd_gin_wire_t), "wire layouts");
	static_assert(sizeof(oracle_gin_desc_t) == sizeof(ofi_amd_gin_desc_t), "descriptor layouts");
	static_assert(sizeof(oracle_gin_mr_t) == sizeof(ofi_amd_gin_mr_t), "registration layouts");
	oracle_gin_comm_t ca;
	ofi_amd_gin_comm_t cb;
	const uint32_t rails = 1 + rng.below(4);
	oracle_gin_comm_init(&ca, 321, rails, 131072, 64, ack_model);
	SAME("gin comm init", ofi_amd_gin_comm_init(&cb, 321, rails, 131072, 64, ack_model), 0);
	oracle_gin_mr_t mrs[3];
	std::memset(mrs, 0, sizeof(mrs));
	mrs[0].local_base = 0x1000000;
	mrs[1].remote_address_offset = 0x2000000;
	mrs[2].remote_address = 0x7F5500000000ull;
	for (int r = 0; r < 4; r++) {
		mrs[1].key[r] = 0xB000 + (uint64_t)r;
		mrs[2].key[r] = 0xC000 + (uint64_t)r;
	}
	ofi_amd_gin_mr_t mrs_b[3];
	std::memcpy(mrs_b, mrs, sizeof(mrs));
	for (uint32_t i = 0; i < n_ops; i++) {
		oracle_gin_desc_t d;
		oracle_gin_gen_desc(seed, 0, i, 1, 1 + rng.below(5), rng.below(4), rng.below(2), &d); /* op 3 is invalid */
		ofi_amd_gin_desc_t db;
		std::memcpy(&db, &d, sizeof(db));
		oracle_gin_wire_t wa;
		ofi_amd_gin_wire_t wb;
		std::memset(&wa, 0, sizeof(wa));
		std::memset(&wb, 0, sizeof(wb));
		int ra;
		if (rng.chance(15)) { /* a get: remote handle 1, local handle 0 */
			d.kind = db.kind = 3;
			d.src_mr = db.src_mr = 1;
			d.dst_mr = db.dst_mr = 0;
			d.signal_op = db.signal_op = 0;
			ra = oracle_gin_iget(&ca, mrs, &d, &wa);
			SAME("iget rc", ra, ofi_amd_gin_derive(&cb, mrs_b, 3, &db, &wb));
		} else {
			ra = oracle_gin_iput_signal(&ca, mrs, &d, &wa);
			SAME("iput rc", ra, ofi_amd_gin_iput_signal(&cb, mrs_b, 3, &db, &wb));
		}
		if (ra == 0) {
			SAME("wire record", std::memcmp(&wa, &wb, sizeof(wa)), 0);
		} else if (ra == -11) { /* window full: the receiver has consumed up to some point */
			const uint32_t consumed = (ca.tx_tail + 1 + rng.below(4000)) & 0x3FFFu;
			oracle_gin_apply_ack(&ca, consumed);
			ofi_amd_gin_apply_ack(&cb, consumed);
		}
		SAME("comm state", std::memcmp(&ca, &cb, sizeof(ca)), 0);
	}
}

/* ------------------------------------------------- GIN transmit engine (posts, retry, CQ) */

/* A fabric with a bounded send queue per rail; everything done to it is logged. */
struct sim_fabric_t {
	uint32_t depth;
	std::deque<uint32_t> sq[4], cq[4];
	std::vector<uint64_t> log;
	uint64_t attempts = 0, fail_every = 0;
	template <typename P>
	int post(const P *p)
	{
		attempts++;
		log.push_back(((uint64_t)p->kind << 56) | ((uint64_t)p->rail << 48) | ((uint64_t)p->more << 40) |
			      ((uint64_t)p->context << 8));
		log.push_back(p->src ^ (p->len << 1) ^ (p->dest << 2) ^ (p->key << 3) ^ p->msg[0] ^ p->imm ^ p->peer);
		if (fail_every && attempts % fail_every == 0) {
			log.push_back(5);
			return -5;
		}
		if (sq[p->rail].size() >= depth) {
			log.push_back(11);
			return -11;
		}
		sq[p->rail].push_back(p->context);
		return 0;
	}
	int cq_read(uint32_t rail, uint32_t *contexts, uint32_t max)
	{
		uint32_t n = 0;
		while (n < max && !cq[rail].empty()) {
			contexts[n++] = cq[rail].front();
			cq[rail].pop_front();
		}
		log.push_back(0xC000000000000000ull | ((uint64_t)rail << 32) | n);
		return (int)n;
	}
	void complete_some(rng_t &rng)
	{
		for (int r = 0; r < 4; r++) {
			while (!sq[r].empty() && rng.chance(60)) {
				cq[r].push_back(sq[r].front());
				sq[r].pop_front();
			}
		}
	}
};

int oracle_post_cb(void *f, const oracle_gin_post_t *p) { return static_cast<sim_fabric_t *>(f)->post(p); }
int oracle_cq_cb(void *f, uint32_t rail, uint32_t *c, uint32_t max) { return static_cast<sim_fabric_t *>(f)->cq_read(rail, c, max); }
int product_post_cb(void *f, const ofi_amd_gin_post_t *p) { return static_cast<sim_fabric_t *>(f)->post(p); }
int product_cq_cb(void *f, uint32_t rail, uint32_t *c, uint32_t max) { return static_cast<sim_fabric_t *>(f)->cq_read(rail, c, max); }

void run_gin_engine(uint64_t seed, uint32_t n_ops)
{
	rng_t rng{ seed };
	static_assert(sizeof(oracle_gin_post_t) == sizeof(ofi_amd_gin_post_t), "post layouts");
	static_assert(sizeof(oracle_gin_tx_stats_t) == sizeof(ofi_amd_gin_tx_stats_t), "stats layouts");
	sim_fabric_t fa, fb;
	fa.depth = fb.depth = 1 + rng.below(6);
	fa.fail_every = fb.fail_every = rng.chance(50) ? 0 : 200 + rng.below(300);
	const uint32_t pool = 24 + rng.below(64);
	const uint32_t cq_count = 1 + rng.below(5), cq_iter = 1 + rng.below(4);
	oracle_gin_fabric_ops_t oa = { oracle_post_cb, oracle_cq_cb, &fa };
	ofi_amd_gin_fabric_ops_t ob = { product_post_cb, product_cq_cb, &fb };
	oracle_gin_tx_t *a = oracle_gin_tx_create(4, cq_count, cq_iter, pool, &oa);
	ofi_amd_gin_tx_t *b = nullptr;
	SAME("tx create", a != nullptr, ofi_amd_gin_tx_create(4, cq_count, cq_iter, pool, &ob, &b) == 0);
	std::vector<int32_t> open;
	for (uint32_t i = 0; i < n_ops; i++) {
		const uint32_t what = rng.below(100);
		if (what < 55) { /* an operation: a put (writes, perhaps a metadata send) or a get (reads) */
			const bool get = rng.chance(25);
			oracle_gin_wire_t wa;
			std::memset(&wa, 0, sizeof(wa));
			wa.num_writes = get ? 1 + rng.below(4) : rng.below(5);
			for (uint32_t k = 0; k < wa.num_writes; k++) {
				wa.writes[k].rail = rng.below(4);
				wa.writes[k].more = get ? 0 : rng.below(2);
				wa.writes[k].src = rng.next();
				wa.writes[k].len = rng.below(1u << 20);
				wa.writes[k].dest = rng.next();
				wa.writes[k].key = rng.next();
			}
			if (!get) {
				wa.imm = (uint32_t)rng.next();
				wa.nseg = wa.num_writes;
				if (wa.num_writes == 0 || rng.chance(30)) {
					wa.has_meta = 1;
					wa.nseg++;
					wa.meta_rail = rng.below(4);
					wa.meta_more = rng.below(2);
					for (int k = 0; k < 4; k++) {
						wa.meta[k] = rng.next();
					}
				}
			}
			ofi_amd_gin_wire_t wb;
			std::memcpy(&wb, &wa, sizeof(wb));
			int32_t qa = -2, qb = -2;
			const uint32_t peer = rng.below(8);
			const int ra = get ? oracle_gin_tx_iget(a, peer, &wa, &qa) : oracle_gin_tx_iput_signal(a, peer, &wa, &qa);
			const int rb = get ? ofi_amd_gin_tx_iget(b, peer, &wb, &qb) : ofi_amd_gin_tx_iput_signal(b, peer, &wb, &qb);
			SAME("engine op rc", ra, rb);
			SAME("engine request", qa, qb);
			if (ra == 0) {
				open.push_back(qa);
			}
		} else if (what < 58) { /* a flush: one read per rail into slots that a later step fills */
			static uint64_t slots_a[32]; /* one array for both engines: the posts carry its address */
			uint64_t *const slots_b = slots_a;
			int32_t qa = -2, qb = -2;
			const int ra = oracle_gin_tx_iflush(a, slots_a, 0x5000, 0xdeadbeefdeadbeefull, &qa);
			SAME("iflush rc", ra, ofi_amd_gin_tx_iflush(b, slots_b, 0x5000, 0xdeadbeefdeadbeefull, &qb));
			SAME("iflush request", qa, qb);
			if (ra == 0) {
				SAME("slots cleared", slots_a[0] | slots_a[8] | slots_a[16] | slots_a[24], 0);
				/* the reads land at once or not at all before the request is tested */
				const bool landed = rng.chance(70);
				for (int r = 0; r < 4; r++) {
					slots_a[8 * r] = slots_b[8 * r] = landed ? 0xdeadbeefdeadbeefull : 0;
				}
				int da = -1, db = -1;
				SAME("flush test rc", oracle_gin_tx_test(a, qa, &da), ofi_amd_gin_tx_test(b, qb, &db));
				SAME("flush done", da, db);
				if (!da) {
					for (int r = 0; r < 4; r++) {
						slots_a[8 * r] = slots_b[8 * r] = 0xdeadbeefdeadbeefull;
					}
					SAME("flush test rc", oracle_gin_tx_test(a, qa, &da), ofi_amd_gin_tx_test(b, qb, &db));
					SAME("flush done late", da, 1);
					SAME("flush done late", db, 1);
				}
			}
		} else if (what < 65) {
			const uint64_t msg = rng.next();
			const uint32_t peer = rng.below(8);
			SAME("send_ack rc", oracle_gin_tx_send_ack(a, peer, msg), ofi_amd_gin_tx_send_ack(b, peer, msg));
		} else if (what < 85) {
			rng_t ra{ rng.s }, rb{ rng.s };
			fa.complete_some(ra);
			fb.complete_some(rb);
			rng.s = ra.s;
			SAME("progress rc", oracle_gin_tx_progress(a), ofi_amd_gin_tx_progress(b));
		} else if (!open.empty()) {
			const size_t k = rng.below((uint32_t)open.size());
			int da = -1, db = -1;
			SAME("test rc", oracle_gin_tx_test(a, open[k], &da), ofi_amd_gin_tx_test(b, open[k], &db));
			SAME("test done", da, db);
			if (da == 1) {
				open[k] = open.back();
				open.pop_back();
			}
		}
		SAME("fabric log length", fa.log.size(), fb.log.size());
		if (fa.log != fb.log) {
			fail("fabric logs differ", i);
		}
		fa.log.clear();
		fb.log.clear();
		oracle_gin_tx_stats_t sa;
		ofi_amd_gin_tx_stats_t sb;
		oracle_gin_tx_stats(a, &sa);
		ofi_amd_gin_tx_stats(b, &sb);
		SAME("engine stats", std::memcmp(&sa, &sb, sizeof(sa)), 0);
	}
	oracle_gin_tx_destroy(a);
	ofi_amd_gin_tx_destroy(b);
}

/* ------------------------- the ncclRma_v15_t data-path entry points over derivation + engine */

/* what nccl_net_ofi_retval_translate (include/nccl_ofi_api.h:30-75) makes of the codes met here */
uint64_t g_rma_accepted, g_rma_refused, g_rma_done;

int nccl_code_of(int rc)
{
	return rc == 0 ? ncclSuccess : rc == -22 ? ncclInternalError : rc == -90 ? ncclInvalidUsage : ncclSystemError;
}

void run_rma_abi(uint64_t seed, uint32_t n_ops)
{
	rng_t rng{ seed };
	const uint32_t nranks = 1 + rng.below(6), rails = 1 + rng.below(4), pool = 32 + rng.below(64);
	const uint64_t min_stripe = rng.chance(50) ? 131072 : 4096, max_small = 64;
	sim_fabric_t fa, fb;
	fa.depth = fb.depth = 2 + rng.below(6);
	fa.fail_every = fb.fail_every = rng.chance(60) ? 0 : 150 + rng.below(300);
	oracle_gin_fabric_ops_t oa = { oracle_post_cb, oracle_cq_cb, &fa };
	ofi_amd_gin_fabric_ops_t ob = { product_post_cb, product_cq_cb, &fb };
	/* oracle side: one initiator state per rank, the scheduler / pin / rail cursor lent from one
	 * shared state round each derivation, one engine with the reference's 4 x 4 CQ defaults */
	std::vector<oracle_gin_comm_t> pa(nranks);
	for (uint32_t r = 0; r < nranks; r++) {
		oracle_gin_comm_init(&pa[r], r, rails, min_stripe, max_small, 0);
	}
	oracle_gin_comm_t sa;
	oracle_gin_comm_init(&sa, 0, rails, min_stripe, max_small, 0);
	oracle_gin_tx_t *a = oracle_gin_tx_create(rails, 4, 4, pool, &oa);
	ofi_amd_rma_ctx_t *ctx = nullptr;
	SAME("rma ctx create", ofi_amd_rma_ctx_create(nranks, rails, min_stripe, max_small, &ob, pool, 1, &ctx), 0);
	if (!a) {
		fail("oracle engine");
	}
	/* three registrations: source, destination, signal */
	oracle_gin_mr_t mra[3][6];
	ofi_amd_rma_mr_t *mrb[3];
	for (int h = 0; h < 3; h++) {
		uint64_t base = 0x10000000ull * (uint64_t)(h + 1), addr[6], off[6], keys[6 * 4];
		for (uint32_t r = 0; r < nranks; r++) {
			addr[r] = rng.next() >> 16;
			off[r] = rng.chance(50) ? 0 : addr[r];
			mra[h][r].local_base = base;
			mra[h][r].remote_address = addr[r];
			mra[h][r].remote_address_offset = off[r];
			for (int k = 0; k < 4; k++) {
				keys[r * 4 + k] = mra[h][r].key[k] = rng.next();
			}
		}
		SAME("rma mr create", ofi_amd_rma_mr_create(ctx, base, addr, off, keys, &mrb[h]), 0);
	}
	static uint64_t slots[32];
	SAME("flush buffers", ofi_amd_rma_set_flush_buffers(ctx, slots, 0x5000, 0xdeadbeefdeadbeefull), 0);

	struct open_t {
		int32_t q;
		void *req;
	};
	std::vector<open_t> open;
	for (uint32_t i = 0; i < n_ops; i++) {
		const uint32_t what = rng.below(100);
		if (what < 38) {
			const uint32_t rank = rng.below(nranks);
			/* keep the peer's sequence window open: an ACK for everything sent so far */
			if (((pa[rank].tx_head - pa[rank].tx_tail) & 0x3FFFu) >= 200 || rng.chance(5)) {
				const uint32_t consumed = pa[rank].tx_head & 0x3FFFu;
				oracle_gin_apply_ack(&pa[rank], consumed);
				SAME("ack rc", ofi_amd_rma_ack_received(ctx, rank, oracle_gin_ack_msg(rank, consumed)), 0);
			}
			const uint32_t kind = rng.below(10); /* 0-1 get, 2-4 put, 5-9 put with signal */
			const bool get = kind < 2, sig = kind >= 5;
			oracle_gin_desc_t d;
			std::memset(&d, 0, sizeof(d));
			d.src_off = rng.below(1u << 24);
			d.dst_off = rng.below(1u << 24);
			d.size = rng.chance(10) ? 0 : rng.chance(50) ? rng.below(4096) : rng.below(1u << 22);
			d.rank = rank;
			d.opt_flags = rng.below(2);
			d.src_mr = 0;
			d.dst_mr = 1;
			d.sig_mr = 0xffff;
			d.kind = get ? 3 : 1;
			if (sig) {
				d.signal_off = 8 * rng.below(1024);
				d.signal_value = rng.next();
				d.signal_op = 1 + rng.below(3); /* 3 is rejected by both */
				d.sig_mr = 2;
				d.kind = 2;
			}
			if (get && d.size == 0) {
				d.size = 1;
			}
			const oracle_gin_mr_t table[3] = { mra[0][rank], mra[1][rank], mra[2][rank] };
			oracle_gin_comm_t *peer = &pa[rank];
			const oracle_gin_comm_t peer_before = *peer, shared_before = sa;
			peer->sched = sa.sched;
			peer->pinned_rail_id = sa.pinned_rail_id;
			peer->pinned_rail_run = sa.pinned_rail_run;
			peer->next_rail_id = sa.next_rail_id;
			oracle_gin_wire_t wa;
			std::memset(&wa, 0, sizeof(wa));
			int ra = get ? oracle_gin_iget(peer, table, &d, &wa) : oracle_gin_iput_signal(peer, table, &d, &wa);
			sa.sched = peer->sched;
			sa.pinned_rail_id = peer->pinned_rail_id;
			sa.pinned_rail_run = peer->pinned_rail_run;
			sa.next_rail_id = peer->next_rail_id;
			int32_t qa = -1;
			if (ra == 0) {
				ra = get ? oracle_gin_tx_iget(a, rank, &wa, &qa) : oracle_gin_tx_iput_signal(a, rank, &wa, &qa);
				if (ra == -ENOMEM) {
					/* The engine's pool is full and nothing was posted.  The reference's pool throws
					 * there; the entry points instead undo the derivation, so that no sequence number
					 * is used up by an operation that never reaches the wire. */
					*peer = peer_before;
					sa = shared_before;
				}
			}
			void *req = &req; /* must be overwritten */
			int rb;
			if (get) {
				rb = ofi_amd_rma_iget(ctx, 0, d.src_off, mrb[0], d.size, d.dst_off, mrb[1], rank, d.opt_flags, &req);
			} else if (sig) {
				rb = ofi_amd_rma_iputSignal(ctx, 0, d.src_off, mrb[0], d.size, d.dst_off, mrb[1], rank, d.signal_off,
							    mrb[2], d.signal_value, d.signal_op, true, d.opt_flags, &req);
			} else {
				rb = ofi_amd_rma_iput(ctx, 0, d.src_off, mrb[0], d.size, d.dst_off, mrb[1], rank, d.opt_flags, &req);
			}
			SAME("rma op code", nccl_code_of(ra), rb);
			if (ra == 0) {
				SAME("rma request", qa, *static_cast<int32_t *>(req));
				open.push_back({ qa, req });
				g_rma_accepted++;
			} else {
				g_rma_refused++;
				SAME("rma request cleared", req == nullptr, 1);
			}
			SAME("rma peer state", std::memcmp(peer, ofi_amd_rma_peer_state(ctx, rank), sizeof(*peer)), 0);
			SAME("rma shared state", std::memcmp(&sa, ofi_amd_rma_peer_state(ctx, UINT32_MAX), sizeof(sa)), 0);
		} else if (what < 41) {
			int32_t qa = -1;
			void *req = nullptr;
			const int ra = oracle_gin_tx_iflush(a, slots, 0x5000, 0xdeadbeefdeadbeefull, &qa);
			SAME("rma iflush code", nccl_code_of(ra), ofi_amd_rma_iflush(ctx, 0, mrb[1], 0, &req));
			if (ra == 0) {
				SAME("rma flush request", qa, *static_cast<int32_t *>(req));
				for (int r = 0; r < 4; r++) {
					slots[8 * r] = 0xdeadbeefdeadbeefull; /* the reads land */
				}
				open.push_back({ qa, req });
			}
		} else if (what < 62) {
			rng_t r1{ rng.s }, r2{ rng.s };
			fa.complete_some(r1);
			fb.complete_some(r2);
			rng.s = r1.s;
			SAME("rma progress code", nccl_code_of(oracle_gin_tx_progress(a)), ofi_amd_rma_rmaProgress(ctx));
		} else if (!open.empty()) {
			const size_t k = rng.below((uint32_t)open.size());
			int da = -1, db = -1;
			SAME("rma test code", nccl_code_of(oracle_gin_tx_test(a, open[k].q, &da)),
			     ofi_amd_rma_test(ctx, open[k].req, &db));
			SAME("rma test done", da, db);
			if (da == 1) {
				g_rma_done++;
				/* the request is back in the pool: a second test is refused, nothing posted */
				SAME("rma test twice", ofi_amd_rma_test(ctx, open[k].req, &db), ncclInternalError);
				open[k] = open.back();
				open.pop_back();
			}
		}
		if (fa.log != fb.log) {
			fail("rma fabric logs differ", i);
		}
		fa.log.clear();
		fb.log.clear();
		oracle_gin_tx_stats_t sta;
		ofi_amd_gin_tx_stats_t stb;
		oracle_gin_tx_stats(a, &sta);
		SAME("rma stats rc", ofi_amd_rma_tx_stats(ctx, &stb), 0);
		SAME("rma engine stats", std::memcmp(&sta, &stb, sizeof(sta)), 0);
	}
	for (int h = 0; h < 3; h++) {
		SAME("rma mr destroy", ofi_amd_rma_mr_destroy(mrb[h]), 0);
	}
	SAME("rma ctx destroy", ofi_amd_rma_ctx_destroy(ctx), 0);
	oracle_gin_tx_destroy(a);
}

} // namespace

int main(int argc, char **argv)
{
	const uint64_t seeds = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 6;
	for (uint64_t s = 1; s <= seeds; s++) {
		run_msgbuff(s, 4, 4, 3000);
		run_msgbuff(s + 100, 7, 4, 3000);
		run_msgbuff(s + 200, 256, 10, 6000);
		run_msgbuff(s + 300, 9, 4, 10); /* rejected by both */
		run_sendrecv(s, 60 + 20 * (uint32_t)s, true);
		run_sendrecv(s + 1000, 60 + 20 * (uint32_t)s, false);
		run_rxq(s);
		run_gin_rx(s, 20000);
		run_gin_tx(s, 30000, 0);
		run_gin_tx(s + 50, 30000, 1);
		run_gin_engine(s, 20000);
		run_gin_engine(s + 90, 20000);
		run_rma_abi(s, 20000);
		run_rma_abi(s + 70, 20000);
	}
	std::printf("rma entry points: %llu operations accepted, %llu refused, %llu tested to completion\n",
		    (unsigned long long)g_rma_accepted, (unsigned long long)g_rma_refused, (unsigned long long)g_rma_done);
	if (g_rma_accepted < 1000 * seeds || g_rma_refused == 0 || g_rma_done < 500 * seeds) {
		fail("the rma program did not exercise the entry points", g_rma_accepted, g_rma_done);
	}
	std::printf("host state machines: oracle and product agree over %llu seeds\n", (unsigned long long)seeds);
	return 0;
}

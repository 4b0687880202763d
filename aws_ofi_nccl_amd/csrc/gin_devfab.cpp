/*
 * A fabric for the GIN / RMA transmit engine (ofi_amd_gin_fabric_ops_t) that really moves the
 * bytes, for an initiator and its targets inside one process on one GPU.  It stands where the
 * reference has libfabric endpoints, the target's progress thread and GDRCopy: what
 * tests/functional/rma.cpp sets up with two ranks.
 *
 * Posts enter bounded send queues per rail, with the doorbell rule of the in-process loop-back
 * fabric (a post without FI_MORE, or a full queue, transmits everything queued on the rail).
 * Transmitted posts are gathered into launch groups on the caller's stream: an RDMA write or
 * read is one entry of a device copy table (ofi_amd_copy_table_pieces), and a group ends in a
 * sentinel read-back into a pinned word.  When a group's sentinel is seen, its posts complete
 * (cq_read returns their contexts, in post order per rail) and the target hears of them, in
 * the order they were transmitted: write completions and metadata messages go to the receiver
 * (ofi_amd_gin_rx_*: reassembly, in-order retire, folding), the signal work it releases is
 * applied to the counters in HBM by the next group's launch (ofi_amd_gin_signal_apply, behind
 * the copies whose completion released it), and its ACKs go back to the initiator through
 * the callback.  All of that happens inside cq_read, i.e. inside the engine's progress call.
 */
#include <cerrno>
#include <cstring>
#include <ctime>
#include <new>
#include <vector>

#include "host_util.hpp"
#include "ofi_amd_hotpath.h"

namespace {

using ofi_amd::pinned_t;
using ofi_amd::ring_t;

constexpr uint32_t kGroups = 4;
constexpr uint32_t kGroupsKeptBusy = 2; /* in flight before posts start gathering instead of leaving at once */
constexpr uint32_t kGroupEntries = 4096;
constexpr uint32_t kGroupWork = 4096;
constexpr uint64_t kSentinel = 0xdeadbeefdeadbeefull; /* NCCL_OFI_GIN_FLUSH_SENTINEL_VAL */

/* What the target (or, for an ACK, the initiator) hears when a group has landed. */
struct event_t {
	uint8_t kind; /* OFI_AMD_GIN_POST_WRITE / _META / _ACK */
	uint32_t peer;
	uint32_t imm;
	uint64_t msg[4];
};

struct group_t {
	pinned_t src, dst, len, work, done;
	uint32_t n_copy = 0, n_work = 0, max_len = 0;
	uint32_t per_rail[OFI_AMD_MAX_NUM_RAILS] = {};
	std::vector<event_t> events;
	bool launched = false;
	int alloc()
	{
		int rc = src.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = dst.alloc(sizeof(uint64_t) * kGroupEntries);
		if (rc == 0) rc = len.alloc(sizeof(uint32_t) * kGroupEntries);
		if (rc == 0) rc = work.alloc(sizeof(ofi_amd_gin_signal_work_t) * kGroupWork);
		if (rc == 0) rc = done.alloc(64);
		return rc;
	}
	void release()
	{
		for (pinned_t *p : { &src, &dst, &len, &work, &done }) {
			p->release();
		}
	}
	bool empty() const { return n_copy == 0 && n_work == 0 && events.empty() && !any_post(); }
	bool any_post() const
	{
		uint32_t n = 0;
		for (uint32_t r = 0; r < OFI_AMD_MAX_NUM_RAILS; r++) {
			n += per_rail[r];
		}
		return n != 0;
	}
	void reset()
	{
		n_copy = n_work = max_len = 0;
		std::memset(per_rail, 0, sizeof(per_rail));
		events.clear();
		launched = false;
	}
};

} // namespace

struct ofi_amd_devfab {
	struct rail_t {
		ring_t<ofi_amd_gin_post_t> sq; /* posted, completion not read yet */
		uint32_t transmitted = 0;      /* of which the doorbell has rung for */
		uint32_t taken = 0;            /* of which in a launch group */
		uint32_t readable = 0;         /* of which landed: the completion can be read */
	};
	uint32_t num_rails = 0, sq_depth = 0;
	void *stream = nullptr;
	std::vector<rail_t> rails;
	ring_t<uint8_t> rung;
	ofi_amd_gin_rx_t *rx = nullptr;
	std::vector<ofi_amd_gin_signal_region_t> regions;
	void *d_flush_buf = nullptr;
	group_t groups[kGroups];
	uint32_t head = 0, cur = 0;
	int (*on_ack)(void *arg, uint32_t peer, uint64_t ack_msg) = nullptr;
	void *on_ack_arg = nullptr;
	ofi_amd_devfab_stats_t st = {};

	group_t &filling() { return groups[cur % kGroups]; }
	bool can_launch() const { return cur - head < kGroups - 1; }

	static int post(void *self, const ofi_amd_gin_post_t *p)
	{
		ofi_amd_devfab *f = static_cast<ofi_amd_devfab *>(self);
		if (!p || p->rail >= f->num_rails) {
			return -EINVAL;
		}
		if ((p->kind == OFI_AMD_GIN_POST_WRITE || p->kind == OFI_AMD_GIN_POST_READ) && p->len > 0xffffffffull) {
			return -EMSGSIZE; /* a table entry's length is 32 bits; a stripe of the scheduler never is that long */
		}
		rail_t &r = f->rails[p->rail];
		if (r.sq.size() >= f->sq_depth) {
			return -EAGAIN;
		}
		r.sq.push(*p);
		if (!p->more || r.sq.size() >= f->sq_depth) {
			while (r.transmitted < r.sq.size()) {
				f->rung.push((uint8_t)p->rail);
				r.transmitted++;
			}
		}
		return 0;
	}

	/* transmitted posts join the group being filled, in the order their doorbells rang */
	int gather()
	{
		group_t &g = filling();
		/* every post takes at most one table entry and one event; the events were reserved for */
		while (!rung.empty() && g.n_copy < kGroupEntries && g.events.size() < kGroupEntries) {
			const uint32_t rail = rung.at(0);
			rail_t &r = rails[rail];
			const ofi_amd_gin_post_t &p = r.sq.at(r.taken);
			event_t ev;
			std::memset(&ev, 0, sizeof(ev));
			ev.kind = (uint8_t)p.kind;
			ev.peer = p.peer;
			if (p.kind == OFI_AMD_GIN_POST_WRITE || p.kind == OFI_AMD_GIN_POST_READ) {
				const bool read = p.kind == OFI_AMD_GIN_POST_READ;
				uint64_t local = p.src;
				if (read && p.peer == OFI_AMD_GIN_PEER_SELF) {
					/* a flush read lands in pinned host memory: the copy kernel reaches it through
					 * its device address */
					void *dev = nullptr;
					const int rc = ofi_amd_gpu_host_get_device_pointer(&dev, reinterpret_cast<void *>(p.src));
					if (rc != 0) {
						return rc;
					}
					local = reinterpret_cast<uintptr_t>(dev);
					st.flush_reads++;
				} else if (read) {
					st.reads++;
					st.bytes += p.len;
				} else {
					st.writes++;
					st.bytes += p.len;
				}
				if (p.len && (local == 0 || p.dest == 0)) {
					return -EFAULT; /* on the device a copy from or to address 0 is a fault, not an error code */
				}
				if (p.len) {
					g.src.as<uint64_t>()[g.n_copy] = read ? p.dest : p.src;
					g.dst.as<uint64_t>()[g.n_copy] = read ? local : p.dest;
					g.len.as<uint32_t>()[g.n_copy++] = (uint32_t)p.len;
					g.max_len = g.max_len < (uint32_t)p.len ? (uint32_t)p.len : g.max_len;
				}
				if (!read) {
					ev.imm = p.imm;
					g.events.push_back(ev); /* the target's CQ shows the write with its immediate data */
				}
			} else if (p.kind == OFI_AMD_GIN_POST_META || p.kind == OFI_AMD_GIN_POST_ACK) {
				std::memcpy(ev.msg, p.msg, sizeof(ev.msg));
				g.events.push_back(ev);
				st.metas += p.kind == OFI_AMD_GIN_POST_META;
			} else {
				return -EINVAL;
			}
			g.per_rail[rail]++;
			r.taken++;
			rung.pop();
		}
		/* the signal work released by what has landed so far */
		if (g.n_work < kGroupWork) {
			g.n_work += ofi_amd_gin_rx_take_work(rx, g.work.as<ofi_amd_gin_signal_work_t>() + g.n_work,
							     kGroupWork - g.n_work);
		}
		return 0;
	}

	/* While two groups are in flight, what is transmitted keeps gathering in the group being
	 * filled instead of leaving as a group of its own: the pipeline stays busy, and the size of a
	 * group follows the time a launch takes.  A full table leaves regardless. */
	int launch()
	{
		group_t &g = filling();
		const bool full = g.n_copy >= kGroupEntries || g.n_work >= kGroupWork || g.events.size() >= kGroupEntries;
		if (g.empty() || !can_launch() || (!full && cur - head >= kGroupsKeptBusy)) {
			return 0;
		}
		int rc = 0;
		if (g.n_copy) {
			/* a launch holds at most 2^31 - 1 wavefronts, one per 8 KiB of the longest entry */
			const uint64_t per_entry = ((uint64_t)g.max_len + 8191u) / 8192u;
			const uint64_t most = per_entry ? 0x7fff0000ull / per_entry : g.n_copy;
			const uint32_t part = most < 1 ? 1u : (most < g.n_copy ? (uint32_t)most : g.n_copy);
			for (uint32_t at = 0; at < g.n_copy && rc == 0; at += part) {
				const uint32_t cnt = g.n_copy - at < part ? g.n_copy - at : part;
				rc = ofi_amd_copy_table_pieces(g.src.dev_as<uint64_t>() + at, g.dst.dev_as<uint64_t>() + at,
							       g.len.dev_as<uint32_t>() + at, cnt, g.max_len, stream);
				st.launches++;
			}
			st.copy_entries += g.n_copy;
		}
		if (rc == 0) {
			/* the signal adds and the sentinel read-back behind them are one launch */
			__atomic_store_n(g.done.as<uint64_t>(), 0ull, __ATOMIC_RELEASE);
			rc = ofi_amd_gin_signal_apply_post(g.work.dev_as<ofi_amd_gin_signal_work_t>(), g.n_work, regions.data(),
							   (uint32_t)regions.size(), nullptr, d_flush_buf, g.done.dev, 1, stream);
			st.launches++;
			st.work_items += g.n_work;
		}
		if (rc != 0) {
			return rc;
		}
		g.launched = true;
		st.groups++;
		cur++;
		return 0;
	}

	/* groups whose sentinel has arrived: their posts complete, the target hears of them */
	int reap()
	{
		while (head != cur) {
			group_t &g = groups[head % kGroups];
			if (ofi_amd_flush_test(g.done.host, 1, kSentinel) != 1) {
				break;
			}
			for (const event_t &ev : g.events) {
				int rc = 0;
				if (ev.kind == OFI_AMD_GIN_POST_WRITE) {
					rc = ofi_amd_gin_rx_write_completion(rx, ev.peer, ev.imm);
				} else if (ev.kind == OFI_AMD_GIN_POST_META) {
					rc = ofi_amd_gin_rx_metadata(rx, ev.peer, ev.msg);
				} else if (on_ack) {
					rc = on_ack(on_ack_arg, ev.peer, ev.msg[0]);
					st.acks++;
				}
				if (rc != 0) {
					return rc;
				}
			}
			for (uint32_t r = 0; r < num_rails; r++) {
				rails[r].readable += g.per_rail[r];
			}
			g.reset();
			head++;
			/* the target's ACKs travel back on its own endpoint: straight to the initiator */
			ofi_amd_gin_ack_t acks[64];
			for (;;) {
				const uint32_t n = ofi_amd_gin_rx_take_acks(rx, acks, 64);
				for (uint32_t i = 0; i < n; i++) {
					if (on_ack) {
						const int rc = on_ack(on_ack_arg, acks[i].peer, acks[i].msg);
						if (rc != 0) {
							return rc;
						}
					}
					st.acks++;
				}
				if (n < 64) {
					break;
				}
			}
		}
		return 0;
	}

	int advance()
	{
		int rc = reap();
		if (rc == 0) rc = gather();
		if (rc == 0) rc = launch();
		return rc;
	}

	static int cq_read(void *self, uint32_t rail, uint32_t *contexts, uint32_t max)
	{
		ofi_amd_devfab *f = static_cast<ofi_amd_devfab *>(self);
		if (rail >= f->num_rails || !contexts) {
			return -EINVAL;
		}
		const int rc = f->advance();
		if (rc != 0) {
			return rc;
		}
		rail_t &r = f->rails[rail];
		uint32_t n = 0;
		while (n < max && r.readable > 0) {
			contexts[n++] = r.sq.at(0).context;
			r.sq.pop();
			r.readable--;
			r.taken--;
			r.transmitted--;
		}
		return (int)n;
	}

	/* nothing in flight and nothing waiting: advance() has just run, so whatever the last landing
	 * released is either launched (head != cur) or still in the group being filled */
	bool idle() { return head == cur && rung.empty() && filling().empty(); }
};

extern "C" {

int ofi_amd_devfab_create(uint32_t num_rails, uint32_t sq_depth, uint32_t n_peers, const uint32_t *peer_comm_ids,
			  const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions, void *stream,
			  ofi_amd_devfab_t **out)
{
	if (!out || num_rails < 1 || num_rails > OFI_AMD_MAX_NUM_RAILS || sq_depth == 0 || sq_depth > (1u << 20) ||
	    n_peers == 0 || n_regions > 16 || (n_regions && !regions)) {
		return -EINVAL;
	}
	*out = nullptr;
	int rc = ofi_amd_gpu_init();
	if (rc != 0) {
		return rc;
	}
	ofi_amd_devfab *f = new (std::nothrow) ofi_amd_devfab;
	if (!f) {
		return -ENOMEM;
	}
	try {
		f->rails.resize(num_rails);
		for (auto &r : f->rails) {
			r.sq.reset(sq_depth);
		}
		f->rung.reset(num_rails * sq_depth);
		f->regions.assign(regions, regions + n_regions);
		for (group_t &g : f->groups) {
			g.events.reserve(kGroupEntries);
		}
	} catch (...) {
		delete f;
		return -ENOMEM;
	}
	f->num_rails = num_rails;
	f->sq_depth = sq_depth;
	f->stream = stream;
	rc = ofi_amd_gin_rx_create(n_peers, peer_comm_ids, &f->rx);
	if (rc == 0) rc = ofi_amd_gpu_mem_alloc(&f->d_flush_buf, 64);
	if (rc == 0) rc = ofi_amd_flush_buffer_fill(f->d_flush_buf, kSentinel, stream);
	for (uint32_t k = 0; k < kGroups && rc == 0; k++) {
		rc = f->groups[k].alloc();
	}
	if (rc != 0) {
		(void)ofi_amd_devfab_destroy(f);
		return rc;
	}
	*out = f;
	return 0;
}

int ofi_amd_devfab_destroy(ofi_amd_devfab_t *f)
{
	if (!f) {
		return -EINVAL;
	}
	const int rc = f->d_flush_buf ? ofi_amd_gpu_stream_synchronize(f->stream) : 0;
	for (group_t &g : f->groups) {
		g.release();
	}
	if (f->d_flush_buf) (void)ofi_amd_gpu_mem_free(f->d_flush_buf);
	if (f->rx) (void)ofi_amd_gin_rx_destroy(f->rx);
	delete f;
	return rc;
}

int ofi_amd_devfab_ops(ofi_amd_devfab_t *f, ofi_amd_gin_fabric_ops_t *ops)
{
	if (!f || !ops) {
		return -EINVAL;
	}
	ops->post = &ofi_amd_devfab::post;
	ops->cq_read = &ofi_amd_devfab::cq_read;
	ops->fabric = f;
	return 0;
}

int ofi_amd_devfab_on_ack(ofi_amd_devfab_t *f, int (*on_ack)(void *arg, uint32_t peer, uint64_t ack_msg), void *arg)
{
	if (!f) {
		return -EINVAL;
	}
	f->on_ack = on_ack;
	f->on_ack_arg = arg;
	return 0;
}

int ofi_amd_devfab_ring_all(ofi_amd_devfab_t *f)
{
	if (!f) {
		return -EINVAL;
	}
	for (uint32_t rail = 0; rail < f->num_rails; rail++) {
		ofi_amd_devfab::rail_t &r = f->rails[rail];
		while (r.transmitted < r.sq.size()) {
			f->rung.push((uint8_t)rail);
			r.transmitted++;
		}
	}
	return 0;
}

int ofi_amd_devfab_quiesce(ofi_amd_devfab_t *f, uint32_t timeout_ms)
{
	if (!f) {
		return -EINVAL;
	}
	/* bounded by the clock of the flush slots: every pass either lands a group or finds nothing left */
	const uint64_t limit = (uint64_t)(timeout_ms ? timeout_ms : 10000) * 1000000ull;
	struct timespec t0;
	clock_gettime(CLOCK_MONOTONIC, &t0);
	for (;;) {
		const int rc = f->advance();
		if (rc != 0) {
			return rc;
		}
		if (f->idle()) {
			return ofi_amd_gpu_stream_synchronize(f->stream);
		}
		struct timespec t1;
		clock_gettime(CLOCK_MONOTONIC, &t1);
		const uint64_t ns = (uint64_t)(t1.tv_sec - t0.tv_sec) * 1000000000ull + (uint64_t)t1.tv_nsec - (uint64_t)t0.tv_nsec;
		if (ns > limit) {
			return -ETIMEDOUT;
		}
	}
}

int ofi_amd_devfab_stats(const ofi_amd_devfab_t *f, ofi_amd_devfab_stats_t *out)
{
	if (!f || !out) {
		return -EINVAL;
	}
	*out = f->st;
	return 0;
}

} /* extern "C" */

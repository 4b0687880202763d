/*
 * CPU oracle: a scalar restatement of the aws-ofi-nccl algorithms on the hot
 * path, one function per reference function, each citing the reference
 * file:line it follows.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg load liboracle.so, and only
 * as the checker / timed baseline.  Nothing under aws_ofi_nccl_amd/ links or
 * calls it.
 *
 * Parity status of each function (what pins it beyond reading the code):
 *   scheduler        24 known answers of tests/unit/scheduler.cpp:126-309, plus
 *                    invariants and brute force vs an independent big-int model
 *   mpsc/spsc ring   reference headers compiled as-is (oracle/_ref) and driven
 *                    side by side; behaviour cases of tests/unit/mpsc_ring.cpp
 *   gin imm/meta/ack reference macros + bit-field structs compiled as-is
 *                    (oracle/_ref), encode/decode cross-checked field by field
 *   gin iputSignal   state machine (window, ACK hysteresis, pin / defer, FI_MORE): a
 *                    known answer worked out by hand for every branch (first ACK
 *                    request at op 4160, period 4161; window closed at 8192
 *                    outstanding; 15 + 1 doorbell batches; pin redirect cases).  The
 *                    reference has no wire-level test and its source does not build
 *                    here, so nothing beyond those cases and the encoders pins it
 *   gin iget         reads of four gets worked out by hand (stripe counts, rails, lengths,
 *                    local and remote addresses, keys), the scheduler shared with the
 *                    puts, window / sequence / pin untouched, a full window that holds
 *                    puts back but not gets.  The reference has no wire-level test of it
 *   gin receiver     end values of tests/functional/rma.cpp (64 put-signals -> 64)
 *                    and rma_multiseg_signal.cpp (two slots, each its count)
 *                    under arbitrary arrival orders; hand-derived fold runs;
 *                    exactly-once in-order delivery; ACK cursor + encoding; the ACK
 *                    cadence (one ACK per retire walk, carrying the cursor after the
 *                    walk) worked out by hand on literal wire words for in-order,
 *                    reversed and swapped arrivals, either submission path, folded
 *                    runs, the 14-bit cursor wrap and per-peer comm ids
 *   gin tx engine    post / retry / completion orders worked out by hand against scripted
 *                    fabrics (full send queues, FI_MORE dropped on retry, head-of-line stop of
 *                    the retry, 16 completions per rail per progress call); a get's reads
 *                    the same way (refused read queued, failed read gives the get up), and
 *                    the flush (one read per rail to the own rank, done by the sentinel)
 *   gin signal apply per-slot sums against a plain scatter-add (mod 2^64)
 *   region geometry  ~70 points + 4 extend_region cases of
 *                    tests/unit/region_based_tuner.cpp
 *   region tables    re-parsed from the reference source text and compared
 *   region decisions (algorithm, protocol) over the configured grid and random points of
 *                    all four platforms against a textbook even-odd point-in-polygon
 *                    rule on the same tables (another ray than the reference's), first
 *                    polygon in table order wins; points within 1e-6 of an edge, where
 *                    the reference's epsilon rules decide and not geometry, rest on the
 *                    geometry row above alone.
 *   nChannels /      every breakpoint of calculateChunkSizeTreeLL128, calculateBestNChannel
 *   chunk sizes      Tree / Pat and the two P5en chunk ladders worked out on paper from
 *                    the reference's thresholds, both sides of each asserted, for several
 *                    (channels, nodes) shapes; tie-break, window ends, dispatch
 *                    conditions; monotonicity / rung-set / grain invariants
 *   model cost       exact-rational closed forms to 1e-6 rel., linearity and
 *                    protocol-ratio identities; exact fp32 bit pattern of the
 *                    reference binary: PARITY UNPINNED (not buildable here)
 *   bounce copy      memcpy semantics; patterns of tests/unit/gdrcopy.cpp:15-133
 *   eager copy       memcpy semantics with truncation (a plain numpy slice copy)
 *   rdma wire items  known answers of tests/unit/ctrl_msg.cpp (tag search, ready bit,
 *                    full groups, sorted insert 1-7, chain decisions, wrap
 *                    regression) and the static_asserts of include/nccl_ofi_rdma.h
 *                    (8 / 64 / 512 / 560 bytes); sender numbering -> reordered
 *                    delivery -> chain drain returns send order; header bytes of a
 *                    three-batch example and the 16-bit wrap worked out by hand
 *   message buffer   the scenario of tests/unit/msgbuff.cpp:42-122 (4 in flight, 4-bit
 *                    numbers, four rounds) plus wrap, skip and out-of-order cases
 *   send/recv state  who-receives-what and reported sizes of the scenarios of
 *   machines         tests/functional/eager_multirecv.cpp (T5-T19, T21-T25) replayed with
 *                    the test as the wire; per-tag order under random interleavings
 *                    with unique tags; the sender's decision stream call by call
 *                    (again / eager + header / writes + immediate data, schedule,
 *                    size, state) worked out on paper for a single-receive program, a
 *                    truncating rendezvous and a grouped receive
 */
#ifndef ORACLE_H_
#define ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORACLE_MAX_RAILS 4

/* ---------------------------------------------------------------- scheduler */

/* Same field order and padding as nccl_net_ofi_xfer_info_t
 * (include/nccl_ofi_scheduler.h:20-27): 24 bytes. */
typedef struct {
	uint16_t rail_id;
	uint16_t pad0;
	uint32_t pad1;
	uint64_t offset;
	uint64_t msg_size;
} oracle_xfer_t;

/* State of nccl_net_ofi_threshold_scheduler (include/nccl_ofi_scheduler.h:115-121). */
typedef struct {
	uint32_t rr_small_counter;
	uint32_t rr_counter;
	uint64_t max_small_msg_size;
	uint64_t min_stripe_size;
	int32_t num_rails;
	int32_t pad;
} oracle_sched_t;

void oracle_sched_init(oracle_sched_t *s, int num_rails, uint64_t min_stripe_size,
		       uint64_t max_small_msg_size);
int oracle_sched_num_stripes(const oracle_sched_t *s, uint64_t size);
/* One get_schedule() call; writes up to num_rails entries, returns the count. */
int oracle_sched_get_schedule(oracle_sched_t *s, uint64_t size, uint64_t align,
			      oracle_xfer_t *xfers);
/* n calls in index order on one instance.  Output is fixed width: num_xfers[i]
 * and xfers[i*4 .. i*4+3], unused entries zero. */
void oracle_sched_batch(oracle_sched_t *s, const uint64_t *sizes, uint64_t n, uint64_t align,
			uint32_t *num_xfers, oracle_xfer_t *xfers);
/* The same loop with one heap allocation + free per message, mirroring the
 * reference's freelist alloc per schedule (src/nccl_ofi_scheduler.cpp:172). */
void oracle_sched_batch_alloc(oracle_sched_t *s, const uint64_t *sizes, uint64_t n,
			      uint64_t align, uint32_t *num_xfers, oracle_xfer_t *xfers);

/* ------------------------------------------------------------- bounce copy */

/* Batched eager copy (src/nccl_ofi_rdma.cpp:2729-2776 semantics, one call per
 * buffer there): arena[dst_off[i] .. +len[i]) = src[src_off[i] .. +len[i]).
 * flush[i] = first 4 bytes at arena+dst_off[i] read after the copy (little
 * endian, zero-extended when len[i] < 4 reads whatever the arena holds). */
void oracle_bounce_scatter(const uint8_t *src, uint8_t *arena, const uint64_t *src_off,
			   const uint64_t *dst_off, const uint32_t *len, uint32_t n,
			   uint32_t *flush);

/* ------------------------------------------------------------------- rings */

typedef struct oracle_mpsc oracle_mpsc_t;
oracle_mpsc_t *oracle_mpsc_create(uint32_t capacity, uint32_t payload_bytes);
void oracle_mpsc_destroy(oracle_mpsc_t *r);
int oracle_mpsc_push(oracle_mpsc_t *r, const void *entry); /* 1 pushed, 0 full */
int oracle_mpsc_pop(oracle_mpsc_t *r, void *entry);        /* 1 popped, 0 empty */
/* For tests: place both cursors at `pos` (sequence words re-seeded accordingly). */
void oracle_mpsc_set_positions(oracle_mpsc_t *r, uint32_t pos);

/* Threaded self-check (producers x per_producer pushes, caller consumes): 0 = all
 * of per-producer FIFO, no loss, no duplicate held. */
int oracle_mpsc_stress(uint32_t capacity, uint32_t producers, uint32_t per_producer);

typedef struct oracle_spsc oracle_spsc_t;
oracle_spsc_t *oracle_spsc_create(uint32_t capacity, uint32_t payload_bytes);
void oracle_spsc_destroy(oracle_spsc_t *r);
int oracle_spsc_push(oracle_spsc_t *r, const void *entry);
int oracle_spsc_pop(oracle_spsc_t *r, void *entry);

/* --------------------------------------------------------------------- GIN */

/* The 64-byte put / put-signal descriptor: the argument tuple of iputSignal
 * (include/nccl_ofi_gin_base.h:83-91, nccl/rma_v15.h:43-50). */
typedef struct {
	uint64_t src_off;
	uint64_t dst_off;
	uint64_t size;
	uint64_t signal_off;
	uint64_t signal_value;
	uint32_t rank;
	uint32_t signal_op;
	uint32_t opt_flags;
	uint32_t context;
	uint16_t src_mr;
	uint16_t dst_mr;
	uint16_t sig_mr;
	uint16_t kind;
} oracle_gin_desc_t;

uint32_t oracle_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req);
uint64_t oracle_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req);
uint64_t oracle_gin_ack_msg(uint32_t comm_id, uint32_t rx_consumed);

/* Counter-based synthetic op stream: descriptor i of context c under `seed`. */
void oracle_gin_gen_desc(uint64_t seed, uint32_t context, uint64_t i, uint32_t peer_rank,
			 uint32_t signal_every, uint32_t signal_op, uint32_t aggregate_mask,
			 oracle_gin_desc_t *out);

/* One fi_writemsg the reference would post (src/rdma/gin/nccl_ofi_gin.cpp:737-784). */
typedef struct {
	uint64_t src;
	uint64_t len;
	uint64_t dest;
	uint64_t key;
	uint32_t rail;
	uint32_t more; /* FI_MORE set */
} oracle_gin_write_t;

/* Everything iputSignal derives from one descriptor. 224 bytes. */
typedef struct {
	uint32_t seq;
	uint32_t nseg;
	uint32_t imm;
	uint32_t num_writes;
	uint32_t has_meta;
	uint32_t meta_rail;
	uint32_t meta_more;
	uint32_t ack_req;
	oracle_gin_write_t writes[ORACLE_MAX_RAILS];
	uint64_t meta[4];
} oracle_gin_wire_t;

/* Memory registration as the harness fixes it: local base address, the peer's
 * address / address_offset, per-rail keys (include/rdma/gin/nccl_ofi_gin.h:168-183). */
typedef struct {
	uint64_t local_base;
	uint64_t remote_address;
	uint64_t remote_address_offset;
	uint64_t key[ORACLE_MAX_RAILS];
} oracle_gin_mr_t;

typedef struct {
	oracle_sched_t sched;
	uint32_t comm_id;      /* remote comm id */
	uint32_t num_rails;
	uint32_t tx_head;
	uint32_t tx_tail;
	uint32_t consecutive_puts_without_ack;
	uint32_t last_ack_requested_seq;
	uint32_t has_pending_ack_request;
	int32_t pinned_rail_id;
	uint32_t pinned_rail_run;
	uint32_t next_rail_id;
	/* 0: ACKs never arrive (call fails with -11 once the window is full);
	 * 1: the ACK for an ack-requesting op arrives right after that op. */
	uint32_t ack_model;
	uint32_t pad;
} oracle_gin_comm_t;

void oracle_gin_comm_init(oracle_gin_comm_t *c, uint32_t comm_id, uint32_t num_rails,
			  uint64_t min_stripe, uint64_t max_small, uint32_t ack_model);
/* src/rdma/gin/nccl_ofi_gin.cpp:568-864.  Returns 0, -22 (bad signal op) or
 * -11 (window full and no ACK can arrive). */
int oracle_gin_iput_signal(oracle_gin_comm_t *c, const oracle_gin_mr_t *mrs,
			   const oracle_gin_desc_t *d, oracle_gin_wire_t *out);
int oracle_gin_iget(oracle_gin_comm_t *c, const oracle_gin_mr_t *mrs, const oracle_gin_desc_t *d,
		    oracle_gin_wire_t *out);
void oracle_gin_apply_ack(oracle_gin_comm_t *c, uint32_t wire_rx_consumed);

/* ---- initiator below the derivation (oracle_gin_tx.c): posts, pending retry, CQ drain ---- */
#define ORACLE_GIN_POST_WRITE 1
#define ORACLE_GIN_POST_META 2
#define ORACLE_GIN_POST_ACK 3
#define ORACLE_GIN_POST_READ 4
typedef struct {
	uint32_t kind, rail, more, context, peer, imm;
	uint64_t src, len, dest, key;
	uint64_t msg[4];
} oracle_gin_post_t;
typedef struct {
	int (*post)(void *fabric, const oracle_gin_post_t *post);
	int (*cq_read)(void *fabric, uint32_t rail, uint32_t *contexts, uint32_t max);
	void *fabric;
} oracle_gin_fabric_ops_t;
typedef struct {
	uint64_t posts, refused, retries, retried_ok, completions;
	uint32_t pending, pending_max, requests, requests_max, outstanding_acks, pad;
} oracle_gin_tx_stats_t;
typedef struct oracle_gin_tx oracle_gin_tx_t;
oracle_gin_tx_t *oracle_gin_tx_create(uint32_t num_rails, uint32_t cq_read_count,
				      uint32_t cq_process_max_iter, uint32_t max_requests,
				      const oracle_gin_fabric_ops_t *ops);
void oracle_gin_tx_destroy(oracle_gin_tx_t *tx);
int oracle_gin_tx_iput_signal(oracle_gin_tx_t *tx, uint32_t peer, const oracle_gin_wire_t *wire,
			      int32_t *request);
int oracle_gin_tx_iget(oracle_gin_tx_t *tx, uint32_t peer, const oracle_gin_wire_t *wire,
		       int32_t *request);
int oracle_gin_tx_iflush(oracle_gin_tx_t *tx, void *host_slots, uint64_t device_flush_buffer,
			 uint64_t sentinel, int32_t *request);
int oracle_gin_tx_send_ack(oracle_gin_tx_t *tx, uint32_t peer, uint64_t ack_msg);
int oracle_gin_tx_progress(oracle_gin_tx_t *tx);
int oracle_gin_tx_test(oracle_gin_tx_t *tx, int32_t request, int *done);
void oracle_gin_tx_stats(const oracle_gin_tx_t *tx, oracle_gin_tx_stats_t *out);

/* ---- receiver side (oracle_gin_rx.c) ---- */

/* One folded signal delivery: +value on the 8-byte counter at base + offset. 32 bytes. */
typedef struct {
	uint64_t base;
	uint64_t offset;
	uint64_t value;
	uint32_t peer;
	uint16_t gate_seq; /* sequence number of the run's last op */
	uint16_t run_len;  /* ops folded into this item */
} oracle_gin_signal_work_t;

typedef struct {
	uint32_t peer;
	uint32_t rx_consumed;
	uint64_t msg; /* gin_ack_msg_t */
} oracle_gin_ack_t;

typedef struct oracle_gin_rx oracle_gin_rx_t;
oracle_gin_rx_t *oracle_gin_rx_create(uint32_t n_peers, const uint32_t *peer_comm_ids);
void oracle_gin_rx_destroy(oracle_gin_rx_t *rx);
/* a write-with-immediate completion / a 32-byte metadata message from `peer` */
int oracle_gin_rx_write(oracle_gin_rx_t *rx, uint32_t peer, uint32_t imm);
int oracle_gin_rx_metadata(oracle_gin_rx_t *rx, uint32_t peer, const uint64_t meta[4]);
uint32_t oracle_gin_rx_take_work(oracle_gin_rx_t *rx, oracle_gin_signal_work_t *out, uint32_t cap);
uint32_t oracle_gin_rx_take_acks(oracle_gin_rx_t *rx, oracle_gin_ack_t *out, uint32_t cap);
void oracle_gin_rx_cursors(const oracle_gin_rx_t *rx, uint32_t peer, uint32_t *rx_consumed,
			   uint32_t *next_seq);
int oracle_gin_signal_apply(const oracle_gin_signal_work_t *batch, uint32_t n, const uint64_t *bases,
			    const uint64_t *sizes, uint64_t *const *counters, uint32_t n_regions);

uint64_t oracle_gin_fold(uint64_t h, const uint64_t *w, int n);
uint64_t oracle_gin_stream_checksum(uint64_t seed, uint32_t n_contexts, uint64_t ops,
				    uint32_t peer_rank, uint32_t signal_every, uint32_t signal_op,
				    uint32_t aggregate_mask, int with_wire, uint32_t num_rails,
				    uint64_t min_stripe, uint64_t max_small, uint32_t ack_model,
				    const oracle_gin_mr_t *mrs);
/* CPU producer threads -> one MPSC ring per context (push with CAS) -> the calling thread as
 * the only consumer; *checksum equals oracle_gin_stream_checksum(with_wire = 0) */
int oracle_gin_cpu_rings_run(uint64_t seed, uint32_t n_contexts, uint64_t ops, uint32_t capacity,
			     uint32_t producers, uint32_t peer_rank, uint32_t signal_every,
			     uint32_t signal_op, uint32_t aggregate_mask, uint64_t *checksum,
			     double *seconds);

/* ------------------------------------------------------------------- tuner */

enum { ORACLE_PLAT_P5_P5E = 0, ORACLE_PLAT_P5EN = 1, ORACLE_PLAT_P6 = 2, ORACLE_PLAT_P6_B300 = 3 };

/* nccl_ofi_tuner_compute_cost, src/tuner/nccl_ofi_model.cpp:46-122. */
float oracle_model_cost(int platform, int coll, int algo, int proto, int pipe_ops,
			uint64_t size, uint64_t num_ranks, uint64_t num_nodes,
			int num_channels, int net_comp_overhead);
/* model_get_coll_info_internal_v3, :154-234.  algo and proto are -1 when nothing is chosen. */
void oracle_model_decide(int platform, int coll, int pipe_ops, uint64_t size,
			 uint64_t num_ranks, uint64_t num_nodes, int num_channels,
			 int net_comp_overhead, int *algo, int *proto);

/* model_get_coll_info_internal_v2, :236-309 */
void oracle_model_decide_v2(int platform, int coll, int pipe_ops, uint64_t size,
			    uint64_t num_ranks, uint64_t num_nodes, int num_channels,
			    int net_comp_overhead, int nvls_support, int *algo, int *proto);

typedef struct { double x, y; } oracle_point_t;
/* extend_region, src/tuner/nccl_ofi_regions.cpp:254-289 (linear in, linear out). */
oracle_point_t oracle_region_extend(oracle_point_t a, oracle_point_t b, oracle_point_t z);
/* transform_log2, include/tuner/nccl_ofi_tuner_region.h:87-109. */
oracle_point_t oracle_region_log2(oracle_point_t p);
/* is_inside_region, :159-221; polygon and point in log2 space. */
int oracle_region_inside(oracle_point_t p, const oracle_point_t *verts, size_t n);
/* region_get_coll_info_internal_v3, :2070-2157, on a table with no ignored cell.
 * algo and proto are -1 on fall-back; nchannels is left alone unless overridden. */
void oracle_region_decide(int platform, int coll, uint64_t size, uint64_t num_ranks,
			  uint64_t num_nodes, int *algo, int *proto, int *nchannels);
/* The same, skipping every region whose (algorithm*3 + protocol) bit is clear in allowed_mask. */
void oracle_region_decide_masked(int platform, int coll, uint64_t size, uint64_t num_ranks,
				 uint64_t num_nodes, uint32_t allowed_mask, int *algo, int *proto,
				 int *nchannels);
/* Number of polygons and log2-space vertices for one (platform, shape, coll):
 * used by tests to inspect the built table. Returns polygon count. */
int oracle_region_polys(int platform, uint64_t num_ranks, uint64_t num_nodes, int coll,
			int *algos, int *protos, int *nverts, oracle_point_t *verts, int max_polys);
/* region_get_chunk_size_internal, :2276-2306.  Returns 1 when *chunk was set. */
int oracle_region_chunk_size(int platform, int coll, uint64_t size, int algo, int proto,
			     uint64_t num_ranks, uint64_t num_nodes, uint64_t *chunk);
uint64_t oracle_chunk_tree_ll128(uint64_t message_size, int nchannels, int log2_nnodes);
/* calculateBestNChannelTree / calculateBestNChannelPat, :1943-1971 */
int oracle_best_nchannel_tree(uint64_t message_size, int log2_nnodes);
int oracle_best_nchannel_pat(uint64_t message_size, uint64_t num_nodes);

/* Whole-grid loops over the functions above.  point = ((coll*n_sizes + size)*n_nodes +
 * node)*n_ppn + ppn; cost[point*n_algos*3 + a*3 + proto]; choice[point*2 + {algo, proto}];
 * region choice[point*3 + {algo, proto, nchannels}]. */
void oracle_model_grid(int platform, int pipe_ops, int num_channels, int net_comp_overhead,
		       const int32_t *colls, uint32_t n_colls, const uint64_t *sizes, uint32_t n_sizes,
		       const uint64_t *nodes, uint32_t n_nodes, const uint32_t *ppn, uint32_t n_ppn,
		       const int32_t *algos, uint32_t n_algos, double *cost, int8_t *choice);
void oracle_region_grid(int platform, const int32_t *colls, uint32_t n_colls, const uint64_t *sizes,
			uint32_t n_sizes, const uint64_t *nodes, uint32_t n_nodes, const uint32_t *ppn,
			uint32_t n_ppn, int32_t *choice);

/* ------------------------------------------------- RDMA wire formats (oracle_wire.c) */

/* nccl_ofi_eager_msg_header_t, include/nccl_ofi_rdma.h:217-228 */
typedef struct {
	uint8_t eager_offset;
	uint8_t prev_batch_count;
	uint16_t eager_seq;
	int32_t tag;
} oracle_eager_hdr_t;

/* nccl_net_ofi_ctrl_msg_entry_t / nccl_net_ofi_ctrl_msg_t, :235-290 */
typedef struct {
	uint64_t buff_offset;
	uint64_t mr_key[4];
	uint32_t buff_len;
	int16_t tag;
	uint16_t flags;
	uint16_t num_recvs;
	uint8_t recv_idx;
	uint8_t entry_used;
	uint8_t pad[10];
	uint16_t msg_seq_num;
} oracle_ctrl_entry_t;

typedef struct {
	oracle_ctrl_entry_t entries[8];
} oracle_ctrl_msg_t;

/* the ordering fields of nccl_ofi_recv_eager_entry_t, :650-663 */
typedef struct {
	uint8_t eager_offset;
	uint8_t prev_batch_count;
	uint16_t eager_seq;
	uint16_t msg_seq_num;
	uint16_t pad;
	int32_t tag;
	uint32_t recv_len;
	uint64_t cookie;
} oracle_eager_entry_t;

typedef struct {
	uint16_t eager_seq_next;
	uint16_t cur_eager_seq;
	uint8_t eager_offset_next;
	uint8_t prev_eager_batch_count;
	uint16_t pad;
} oracle_eager_tx_t;

uint32_t oracle_rdma_imm(uint32_t comm_id, uint32_t seq, uint32_t recv_idx, uint32_t nseg);
void oracle_rdma_imm_decode(uint32_t imm, uint32_t *comm_id, uint32_t *seq, uint32_t *recv_idx,
			    uint32_t *nseg);
uint32_t oracle_ctrl_mailbox_slot(uint16_t msg_seq_num);
int oracle_ctrl_msg_fill(oracle_ctrl_msg_t *mailbox, uint16_t msg_seq_num, uint16_t num_recvs,
			 const uint64_t *buff_offsets, const uint32_t *sizes, const int *tags,
			 const uint64_t *mr_keys, uint32_t num_rails, int recv_completion_optional);
int oracle_ctrl_msg_ready(const oracle_ctrl_msg_t *mailbox, uint16_t seq_num, int tag,
			  int ignore_tag_match);
int oracle_ctrl_msg_find_tag(const oracle_ctrl_msg_t *msg, int tag);
int oracle_seq_before(uint16_t a, uint16_t b);
int oracle_eager_seq_before(uint16_t a, uint16_t b);
int oracle_eager_entry_less(const oracle_eager_entry_t *a, const oracle_eager_entry_t *b);
int oracle_eager_entry_can_process(int has_processed, uint16_t last_eager_seq, uint8_t last_offset,
				   const oracle_eager_entry_t *entry);
typedef struct oracle_eager_rxq oracle_eager_rxq_t;
oracle_eager_rxq_t *oracle_eager_rxq_create(void);
void oracle_eager_rxq_destroy(oracle_eager_rxq_t *q);
int oracle_eager_rxq_insert(oracle_eager_rxq_t *q, const oracle_eager_entry_t *e);
uint32_t oracle_eager_rxq_drain(oracle_eager_rxq_t *q, oracle_eager_entry_t *out, uint32_t cap);
uint32_t oracle_eager_rxq_pending(const oracle_eager_rxq_t *q);
uint32_t oracle_eager_rxq_peek(const oracle_eager_rxq_t *q, oracle_eager_entry_t *out, uint32_t cap);
void oracle_eager_tx_init(oracle_eager_tx_t *tx);
void oracle_eager_tx_assign(oracle_eager_tx_t *tx, int32_t tag, oracle_eager_hdr_t *hdr);
void oracle_eager_tx_advance(oracle_eager_tx_t *tx);
int oracle_eager_fits(uint64_t size, int64_t eager_send_size);
void oracle_flush_post(const uint64_t flush_buf[8], uint64_t *slots, uint32_t num_rails);
int oracle_flush_completed(const uint64_t *slots, uint32_t num_rails, uint64_t sentinel);
void oracle_eager_copy_batch(const uint8_t *rx_base, const uint64_t *rx_off, const uint32_t *recv_len,
			     uint8_t *dst_base, const uint64_t *dst_off, const uint32_t *dst_len, uint32_t n,
			     uint32_t *copied);

/* ------------------------------------------- send/receive protocol state machines */

/* nccl_ofi_msgbuff_status_t / _result_t / _elemtype_t, include/nccl_ofi_msgbuff.h:42-69 */
enum { ORACLE_MSGBUFF_COMPLETED = 0, ORACLE_MSGBUFF_INPROGRESS, ORACLE_MSGBUFF_NOTSTARTED,
       ORACLE_MSGBUFF_UNAVAILABLE };
enum { ORACLE_MSGBUFF_SUCCESS = 0, ORACLE_MSGBUFF_INVALID_IDX, ORACLE_MSGBUFF_ERROR };
enum { ORACLE_MSGBUFF_REQ = 0, ORACLE_MSGBUFF_BUFF };

typedef struct oracle_msgbuff oracle_msgbuff_t;
oracle_msgbuff_t *oracle_msgbuff_create(uint16_t max_inprogress, uint16_t bit_width, uint16_t start_seq);
void oracle_msgbuff_destroy(oracle_msgbuff_t *m);
int oracle_msgbuff_insert(oracle_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status);
int oracle_msgbuff_replace(oracle_msgbuff_t *m, uint16_t msg_index, void *elem, int type, int *status);
int oracle_msgbuff_retrieve(oracle_msgbuff_t *m, uint16_t msg_index, void **elem, int *type, int *status);
int oracle_msgbuff_complete(oracle_msgbuff_t *m, uint16_t msg_index, int *status);

enum { ORACLE_SEND_AGAIN = 0, ORACLE_SEND_EAGER = 1, ORACLE_SEND_WRITE = 2 };

/* what send() would hand to the fabric */
typedef struct {
	int32_t kind;
	int32_t req;
	uint16_t msg_seq_num;
	uint8_t recv_idx;
	uint8_t no_target_completion;
	uint32_t imm;
	oracle_eager_hdr_t hdr;
	uint64_t size;
	uint64_t remote_buff_offset;
	uint64_t mr_key[4];
	uint32_t num_xfers;
	uint32_t pad;
	oracle_xfer_t xfers[4];
} oracle_send_action_t;

typedef struct {
	uint16_t next_msg_seq_num;
	uint16_t group_sends_remaining;
	uint16_t group_num_recvs;
	uint16_t cur_eager_seq;
	uint16_t eager_seq_next;
	uint8_t eager_queue_count;
	uint8_t eager_offset_next;
	uint8_t prev_eager_batch_count;
	uint8_t pad[3];
	uint32_t num_inflight_reqs;
	uint32_t num_inflight_writes;
	uint64_t n_ctrl_received;
} oracle_send_state_t;

typedef struct oracle_send_comm oracle_send_comm_t;
oracle_send_comm_t *oracle_send_comm_create(uint32_t remote_comm_id, uint32_t num_rails,
					    int64_t eager_send_size, uint64_t min_stripe,
					    uint64_t max_small);
void oracle_send_comm_destroy(oracle_send_comm_t *s);
oracle_ctrl_msg_t *oracle_send_comm_mailbox(oracle_send_comm_t *s);
void oracle_send_comm_state(const oracle_send_comm_t *s, oracle_send_state_t *out);
int oracle_send_comm_send(oracle_send_comm_t *s, uint64_t size, int32_t tag, oracle_send_action_t *act);
int oracle_send_comm_completion(oracle_send_comm_t *s, int32_t req);
int oracle_send_comm_test(oracle_send_comm_t *s, int32_t req, int *done, uint64_t *size);

/* one eager arrival matched to a posted receive: the copy the reference posts as a loop-back read */
typedef struct {
	uint64_t rx_cookie;
	uint64_t dst;
	uint64_t dst_len;
	uint32_t recv_len;
	int32_t req;
	int32_t sub_idx;
	int32_t needs_copy; /* 0: zero-length message, completed at the match */
} oracle_eager_copy_item_t;

typedef struct {
	uint16_t next_msg_seq_num;
	uint16_t eager_drain_recv_seq;
	uint16_t last_eager_seq;
	uint16_t last_completed_seq;
	uint8_t last_eager_offset;
	uint8_t has_processed_eager;
	uint8_t pad[2];
	uint32_t num_inflight_reqs;
	uint32_t eager_pending;
	uint32_t pad2;
	uint64_t n_ctrl_sent;
} oracle_recv_state_t;

typedef struct oracle_recv_comm oracle_recv_comm_t;
oracle_recv_comm_t *oracle_recv_comm_create(uint32_t num_rails);
void oracle_recv_comm_destroy(oracle_recv_comm_t *r);
int oracle_recv_comm_recv(oracle_recv_comm_t *r, int n, const uint64_t *dsts, const uint64_t *sizes,
			  const int *tags, const uint64_t *mr_keys, int completion_optional,
			  oracle_ctrl_msg_t *mailbox, int32_t *req_out, uint16_t *seq_out);
int oracle_recv_comm_eager_arrival(oracle_recv_comm_t *r, uint16_t msg_seq_num,
				   const oracle_eager_hdr_t *hdr, uint32_t recv_len, uint64_t rx_cookie);
int oracle_recv_comm_write_arrival(oracle_recv_comm_t *r, uint32_t imm, uint64_t len);
int oracle_recv_comm_ctrl_sent(oracle_recv_comm_t *r, int32_t req);
uint32_t oracle_recv_comm_take_copies(oracle_recv_comm_t *r, oracle_eager_copy_item_t *out, uint32_t cap);
int oracle_recv_comm_copy_done(oracle_recv_comm_t *r, int32_t req, int32_t sub_idx);
int oracle_recv_comm_test(oracle_recv_comm_t *r, int32_t req, int *done, int *sizes);
int oracle_recv_comm_flush(oracle_recv_comm_t *r, int n, const int *sizes, int32_t *req);
int oracle_recv_comm_flush_test(oracle_recv_comm_t *r, int32_t req, const uint64_t *slots,
				uint32_t num_rails, uint64_t sentinel, int *done);
void oracle_recv_comm_state(const oracle_recv_comm_t *r, oracle_recv_state_t *out);

#ifdef __cplusplus
}
#endif
#endif /* ORACLE_H_ */

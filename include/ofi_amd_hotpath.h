/*
 * C ABI of libofi_amd_hotpath.so: the gfx950 (MI355X) implementation of the
 * data-parallel hot path of the OFI NCCL/RCCL network plugin.
 *
 * Conventions (those of the reference's internal GPU layer,
 * include/nccl_ofi_rocm.h:11-63): every function returns 0 on success or a
 * negative errno; no exception and no HIP type crosses this boundary.  A
 * `stream` argument is a hipStream_t passed as void* (NULL = the default
 * stream).  Pointers named d_* must be device-accessible (HBM or pinned host
 * memory); all others are ordinary host pointers.  Every entry point that needs
 * the GPU returns -ENODEV when no device is present; nothing falls back to the
 * CPU.
 *
 * Threads: the batch launches (sections 2 and 3) keep no state between calls and
 * may be called from any thread on any stream; ofi_amd_sched_batch serialises
 * its own per-stream scratch, the caller orders batches that share one
 * scheduler state.  An object (tuner plan, GIN rings' consumer side, GIN
 * receiver, send or receive comm) belongs to one thread at a time, as a comm
 * belongs to its proxy thread in NCCL; a ring takes any number of producers;
 * the message buffer and the tuner plugin contexts lock themselves as the
 * reference's do.
 */
#ifndef OFI_AMD_HOTPATH_H_
#define OFI_AMD_HOTPATH_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OFI_AMD_MAX_NUM_RAILS 4 /* MAX_NUM_RAILS, include/nccl_ofi_rdma.h:37 */

/* ======================================================================
 * 1. GPU runtime glue: replaces src/nccl_ofi_rocm.cpp (8 functions of
 *    include/nccl_ofi_rocm.h:11-63) and covers the CUDA-only calls GIN needs
 *    (include/nccl_ofi_cuda.h:34-139).
 * ====================================================================== */

/* nccl_net_ofi_gpu_init, include/nccl_ofi_rocm.h:11 */
int ofi_amd_gpu_init(void);
/* nccl_net_ofi_get_gpu_device_for_addr, :24.  Unlike the ROCm stub of the
 * reference (src/nccl_ofi_rocm.cpp:58-76, always -1) this reports the ordinal. */
int ofi_amd_gpu_get_device_for_addr(void *data, int *dev_id);
/* nccl_net_ofi_gpu_flush_gpudirect_rdma_writes, :31.  -EPERM: not available,
 * callers use the read-back flush (ofi_amd_flush_read) instead. */
int ofi_amd_gpu_flush_gpudirect_rdma_writes(void);
/* nccl_net_ofi_gpu_mem_alloc / _free / _copy_host_to_device, :38-52 */
int ofi_amd_gpu_mem_alloc(void **ptr, size_t size);
int ofi_amd_gpu_mem_free(void *ptr);
int ofi_amd_gpu_mem_copy_host_to_device(void *dst, const void *src, size_t size);
/* nccl_net_ofi_gpu_get_dma_buf_fd, :60 */
int ofi_amd_gpu_get_dma_buf_fd(void *aligned_ptr, size_t aligned_size, int *fd, size_t *offset);
/* nccl_net_ofi_gpu_have_dma_buf_attr / _have_gdr_support_attr, :62-63 (1/0) */
int ofi_amd_gpu_have_dma_buf_attr(void);
int ofi_amd_gpu_have_gdr_support_attr(void);
/* nccl_net_ofi_gpu_set/get_current_context, include/nccl_ofi_cuda.h:34-39.
 * HIP has no driver contexts; the "context" is the device ordinal. */
int ofi_amd_gpu_set_current_device(int dev_id);
int ofi_amd_gpu_get_current_device(int *dev_id);
/* nccl_net_ofi_gpu_get_address_range, include/nccl_ofi_cuda.h:46 */
int ofi_amd_gpu_get_address_range(void *ptr, void **base_out, size_t *size_out);
/* nccl_net_ofi_gpu_seg_is_host, include/nccl_ofi_cuda.h:54 */
int ofi_amd_gpu_seg_is_host(void *seg_base, int *is_host_out);
/* Pinned host memory the GPU can address.  Stands in for
 * nccl_net_ofi_gpu_host_register_iomem / _host_unregister
 * (include/nccl_ofi_cuda.h:91-98): memory is allocated pinned rather than
 * registered after the fact.  nccl_net_ofi_gpu_vmm_alloc / _vmm_free (:131-139) have no
 * counterpart: they serve the GDAKI device queues, which are outside this path, and
 * ofi_amd_gpu_mem_alloc covers what the path itself allocates. */
int ofi_amd_gpu_host_alloc(void **ptr, size_t size);
int ofi_amd_gpu_host_free(void *ptr);
/* nccl_net_ofi_gpu_host_get_device_pointer, include/nccl_ofi_cuda.h:106 */
int ofi_amd_gpu_host_get_device_pointer(void **dev_ptr, void *host_ptr);
int ofi_amd_gpu_mem_copy_device_to_host(void *dst, const void *src, size_t size);
int ofi_amd_gpu_stream_synchronize(void *stream);
/* Kernels that skip work because a documented precondition does not hold (a
 * destination range outside the arena, a producer giving up on a full ring) set
 * a bit in a library-owned pinned word.  Fetch-and-clear it after synchronising:
 * bit 0 = bounce destination out of range / misaligned, bit 1 = GIN producer
 * timed out, bit 2 = scheduler state unusable (num_rails outside 1..4 or a zero
 * min_stripe_size; the batch is then left unwritten), bit 3 = an entry of
 * ofi_amd_copy_table_pieces longer than max_len (its bytes beyond are not copied). */
int ofi_amd_async_error_fetch(uint32_t *bits);

/* ======================================================================
 * 2. Rail striping (threshold scheduler), batched.
 *    Replaces per-message nccl_net_ofi_threshold_scheduler::get_schedule,
 *    src/nccl_ofi_scheduler.cpp:47-190.
 * ====================================================================== */

/* nccl_net_ofi_xfer_info_t, include/nccl_ofi_scheduler.h:20-27 (24 bytes) */
typedef struct {
	uint16_t rail_id;
	uint16_t pad0;
	uint32_t pad1;
	uint64_t offset;
	uint64_t msg_size;
} ofi_amd_xfer_info_t;

/* Scheduler state, include/nccl_ofi_scheduler.h:115-121.  Lives in device
 * memory so consecutive batches chain on a stream without a host round trip. */
typedef struct {
	uint32_t rr_small_counter;
	uint32_t rr_counter;
	uint64_t max_small_msg_size; /* OFI_NCCL_SCHED_MAX_SMALL_MSG_SIZE, default 64 */
	uint64_t min_stripe_size;    /* OFI_NCCL_MIN_STRIPE_SIZE, default 131072 */
	int32_t num_rails;           /* 1..4 */
	int32_t pad;
} ofi_amd_sched_state_t;

/*
 * Schedules d_sizes[0..n) in index order, exactly as n consecutive
 * get_schedule(size, num_rails) calls on one scheduler would, and advances the
 * two round-robin counters in *d_state.  Output is fixed width:
 * d_num_xfers[i] = number of stripes, d_xfers[4*i .. 4*i+3] = the stripes
 * (unused entries all-zero).  align is the stripe alignment (128 in the
 * reference, src/nccl_ofi_scheduler.cpp:168).  n <= 2^28 per call.
 */
int ofi_amd_sched_batch(ofi_amd_sched_state_t *d_state, const uint64_t *d_sizes, uint64_t n,
			uint64_t align, uint32_t *d_num_xfers, ofi_amd_xfer_info_t *d_xfers,
			void *stream);
/* ofi_amd_sched_batch keeps a few KiB of device scratch per stream it has been called with
 * (the reference's scheduler keeps a freelist per instance, src/nccl_ofi_scheduler.cpp:135-190).
 * A caller that destroys a stream hands the scratch back first: waits for the stream, frees. */
int ofi_amd_sched_stream_release(void *stream);

/*
 * ofi_amd_sched_batch for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same results and the same kernels; the tile totals and prefixes
 * that ofi_amd_sched_batch keeps in a per-stream allocation live here in a fixed array inside
 * the library's device code (about 512 KiB per GPU, held until the process ends), so the call
 * allocates and frees nothing.  n <= 2^26 messages per call, -E2BIG beyond.  Call
 * ofi_amd_gpu_init() once beforehand (it allocates the asynchronous error word and looks up
 * the array's address on every GPU); -ENXIO otherwise.  All calls on one GPU share that GPU's
 * array: calls that overlap there -- different streams, or two threads -- race; order them.
 * Nothing in the array has to start at zero: a call writes every word before it reads it.
 */
int ofi_amd_sched_batch_noalloc(ofi_amd_sched_state_t *d_state, const uint64_t *d_sizes, uint64_t n,
				uint64_t align, uint32_t *d_num_xfers, ofi_amd_xfer_info_t *d_xfers,
				void *stream);

/* Host-side single-message form with the reference's semantics, for per-op
 * callers (the GIN proxy).  `state` is a host struct. Returns the stripe count. */
int ofi_amd_sched_get_schedule(ofi_amd_sched_state_t *state, uint64_t size, uint64_t align,
			       ofi_amd_xfer_info_t *xfers);

/* ======================================================================
 * 3. Bounce / eager copy and flush, batched, plus the device-copy interface.
 *    Replaces one loop-back fi_read per eager buffer
 *    (rdma_eager_copy_req::post, src/nccl_ofi_rdma.cpp:2729-2776) and the
 *    read-back flush (rdma_flush_req::post, :2664-2713).
 * ====================================================================== */

/*
 * For i in [0,n): copies d_len[i] bytes from d_src + d_src_off[i] (inside [0, src_bytes))
 * to d_arena + d_dst_off[i] (d_dst_off[i] 64-byte aligned, destination ranges
 * disjoint, each inside [0, arena_bytes)), then, if d_flush is not NULL, reads
 * back the first 4 bytes at each destination into d_flush[i] (device or pinned
 * host memory; those 4 bytes must lie inside the arena also for shorter buffers).
 * No byte outside the destination ranges is written.  A buffer that breaks a
 * precondition is skipped and reported through ofi_amd_async_error_fetch (bit 0).
 * n <= 2^30.
 *
 * Visibility: the arena bytes and the flush words are complete, for the host and for
 * work on any stream, once the launch has completed on `stream` (an event, a stream
 * wait, ofi_amd_flush_post queued behind it) -- as for any kernel.  d_flush[i] is
 * written while the kernel runs, each after its own wavefront's stores, with no
 * device-wide ordering: a value that a poller sees before the launch has completed
 * says nothing about the arena bytes of buffer i, and must not be used as a
 * per-buffer completion flag.  The completion that the reference's flush gives its
 * caller (rdma_flush_req, src/nccl_ofi_rdma.cpp:2664-2713) is the sentinel flush
 * below, queued on the same stream.
 */
int ofi_amd_bounce_scatter(const void *d_src, uint64_t src_bytes, void *d_arena, uint64_t arena_bytes,
			   const uint64_t *d_src_off, const uint64_t *d_dst_off,
			   const uint32_t *d_len, uint32_t n, uint32_t *d_flush, void *stream);

/*
 * Eager arrivals as they sit in rx buffers: buffer i starts at rx_base + d_rx_off[i] with
 * the 8-byte nccl_ofi_eager_msg_header_t (include/nccl_ofi_rdma.h:217-228) followed by
 * d_recv_len[i] payload bytes.  Copies min(d_recv_len[i], d_dst_len[i]) payload bytes to
 * dst_base + d_dst_off[i] -- any alignment; dst_base may be NULL with absolute addresses in
 * d_dst_off -- as rdma_eager_copy_req::post does one fi_read at a time
 * (src/nccl_ofi_rdma.cpp:2729-2776; truncation :2738-2743; zero length copies nothing,
 * :753-762).  rx_base is any device-accessible memory (pinned host rx buffers or HBM).
 * d_copied[i] (optional) receives the byte count; d_flush[i] (optional) the first
 * min(4, count) destination bytes, little-endian, read back after the copy (valid, like
 * the copied bytes, once the launch has completed on `stream`; see above).
 */
int ofi_amd_eager_copy_batch(const void *rx_base, const uint64_t *d_rx_off, const uint32_t *d_recv_len,
			     void *dst_base, const uint64_t *d_dst_off, const uint32_t *d_dst_len,
			     uint32_t n, uint32_t *d_copied, uint32_t *d_flush, void *stream);

/*
 * The general form: entry i copies d_len[i] bytes from address d_src_addr[i] to address
 * d_dst_addr[i] (any device-accessible addresses, any alignment, ranges of one batch
 * disjoint), one wavefront per entry.  This is the data movement of a batch of RDMA writes
 * whose source and target live on the same device -- what a loop-back provider does for
 * fi_writemsg (src/rdma/gin/nccl_ofi_gin_reqs.cpp:244-310).  Tables are device-accessible.
 */
int ofi_amd_copy_table(const uint64_t *d_src_addr, const uint64_t *d_dst_addr, const uint32_t *d_len,
		       uint32_t n, void *stream);

/*
 * The same copies for tables that hold long entries: one wavefront per 8 KiB piece of an
 * entry rather than per entry, so that a few long RDMA writes (a rendezvous message's
 * stripes: one fi_writedata per rail, src/nccl_ofi_rdma.cpp:2447-2479) are swept by the whole chip
 * instead of by one wavefront each, and the caller need not cut them.  max_len >= every
 * d_len[i]; the launch has n * ceil(max_len / 8192) wavefronts (-E2BIG beyond 2^31 - 1: split
 * the table), those past the end of their entry leave at once.  An entry longer than max_len
 * is copied up to exactly max_len bytes (nothing of it when max_len is 0) and reported through
 * ofi_amd_async_error_fetch (bit 3).
 */
int ofi_amd_copy_table_pieces(const uint64_t *d_src_addr, const uint64_t *d_dst_addr, const uint32_t *d_len,
			      uint32_t n, uint32_t max_len, void *stream);

/* Flush only: d_flush[i] = 4 bytes at d_arena + d_dst_off[i], read with
 * device-scope acquire semantics (the C5 read-back without a copy). */
int ofi_amd_flush_read(const void *d_arena, const uint64_t *d_dst_off, uint32_t n,
		       uint32_t *d_flush, void *stream);

/*
 * The reference's sentinel flush, kept slot for slot.  A 64-byte flush buffer in GPU memory
 * holds eight copies of a sentinel (0x00000000ffffffff for the RDMA transport,
 * include/nccl_ofi_rdma.h:45 and src/nccl_ofi_rdma.cpp:7390-7394; 0xdeadbeefdeadbeef for GIN,
 * include/rdma/gin/nccl_ofi_gin_reqs.h:274); a flush reads it back into one 64-byte host
 * slot per rail (nccl_net_ofi_flush_data_t, include/nccl_ofi_rdma.h:326-332) and is complete
 * when the first 8 bytes of every slot equal the sentinel (has_flush_completed,
 * src/nccl_ofi_rdma.cpp:2110-2126; nccl_ofi_gin_iflush_req::test,
 * src/rdma/gin/nccl_ofi_gin_reqs.cpp:373-394).  Here the read-back is one small kernel on
 * `stream` instead of one loop-back fi_read per rail (rdma_flush_req::post, :2664-2713).
 *   fill: writes the sentinels into d_flush_buf (64 bytes, device memory);
 *   post: copies d_flush_buf into slots_dev[0..num_rails) -- the device address of pinned
 *         host memory -- with system-scope ordering; the caller zeroes the slots first;
 *   test: host side, 1 when every slot shows the sentinel, else 0.
 */
int ofi_amd_flush_buffer_fill(void *d_flush_buf, uint64_t sentinel, void *stream);
int ofi_amd_flush_post(const void *d_flush_buf, void *slots_dev, uint32_t num_rails, void *stream);
int ofi_amd_flush_test(const void *slots_host, uint32_t num_rails, uint64_t sentinel);

/* nccl_ofi_device_copy, include/nccl_ofi_device_copy.h:14-69: register a device region, then
 * small synchronous host<->device copies at an offset, done by the CPU through a mapping of
 * the device memory as GDRCopy does (src/nccl_ofi_gdrcopy.cpp:108-179).  On a large-BAR
 * system (hipDeviceAttributeIsLargeBar) device memory is CPU-addressable at its device
 * address, which is the mapping.  copy_to_device up to 2 MiB is then CPU stores plus a store
 * fence (0.2-0.4 us up to a page, 20 GB/s beyond), copy_from_device up to 256 bytes CPU loads
 * (2.5 us per 64 bytes); larger copies, where the copy engine wins, go through it.  Where the
 * device has no large BAR, or the runtime has not mapped the registered range into the
 * process, the region registers all the same and every copy takes the copy engine
 * (11-14 us at the least).  As with GDRCopy, neither call
 * waits for GPU work: a store is seen by work submitted after the call returns, a load sees
 * the results of work that has completed. */
typedef struct ofi_amd_devcopy_region ofi_amd_devcopy_region_t;
int ofi_amd_devcopy_register(void *device_ptr, size_t size, ofi_amd_devcopy_region_t **out);
/* 1: small copies of this region are CPU stores / loads through the mapping; 0: every copy takes
 * the copy engine (no large BAR, or the range is not mapped into the process) */
int ofi_amd_devcopy_cpu_mapped(const ofi_amd_devcopy_region_t *region);
int ofi_amd_devcopy_to_device(const void *host_ptr, ofi_amd_devcopy_region_t *h, size_t offset,
			      size_t size);
int ofi_amd_devcopy_from_device(ofi_amd_devcopy_region_t *h, size_t offset, void *host_ptr,
				size_t size);
int ofi_amd_devcopy_forced_pcie_copy(void); /* 0: no alternative path to force */
int ofi_amd_devcopy_deregister(ofi_amd_devcopy_region_t *h);

/* ======================================================================
 * 4. GIN put / put-signal descriptors: GPU producers, pinned-host rings,
 *    host proxy.  Ring protocol of include/nccl_ofi_mpsc_ring.h:56-163; the
 *    descriptor is the argument tuple of iputSignal
 *    (include/nccl_ofi_gin_base.h:83-91); what the proxy derives from it
 *    follows src/rdma/gin/nccl_ofi_gin.cpp:568-864.
 * ====================================================================== */

typedef struct {
	uint64_t src_off;
	uint64_t dst_off;
	uint64_t size;
	uint64_t signal_off;
	uint64_t signal_value;
	uint32_t rank;
	uint32_t signal_op;  /* 0 none, 1 INC, 2 ADD (nccl/net.h:28-29) */
	uint32_t opt_flags;  /* bit 0: aggregate (nccl/rma_v15.h:19-21) */
	uint32_t context;
	uint16_t src_mr;
	uint16_t dst_mr;
	uint16_t sig_mr;     /* 0xffff: no signal handle */
	uint16_t kind;       /* 1 put, 2 put-signal, 3 get */
} ofi_amd_gin_desc_t;    /* 64 bytes */

/* A get (iget, include/nccl_ofi_gin_base.h; src/rdma/gin/nccl_ofi_gin.cpp:879-939) moves data
 * the other way: src_off / src_mr are remoteOff / remoteMhandle (where the bytes are read),
 * dst_off / dst_mr are localOff / localMhandle (where they land); the signal fields are 0. */
#define OFI_AMD_GIN_KIND_PUT 1
#define OFI_AMD_GIN_KIND_PUT_SIGNAL 2
#define OFI_AMD_GIN_KIND_GET 3

typedef struct ofi_amd_gin_rings ofi_amd_gin_rings_t;

/* n_contexts rings of `capacity` descriptors each (a power of two, 256 .. 2^24: a workgroup of
 * the seeded producer reserves 256 slots at a time; -EINVAL otherwise), in pinned host memory:
 * record array (64 B each) + sequence array (u32 each). */
int ofi_amd_gin_rings_create(uint32_t n_contexts, uint32_t capacity, ofi_amd_gin_rings_t **out);
int ofi_amd_gin_rings_destroy(ofi_amd_gin_rings_t *rings);
/*
 * Recovery after a producer gave up on a full ring (ofi_amd_gin_producer_status -ETIMEDOUT;
 * the reference never gives up: await_tx_window, src/rdma/gin/nccl_ofi_gin.cpp:518-537, blocks
 * and carries on, which a kernel that must end cannot).  To be called by the consumer's thread
 * once every producing kernel has ended (the streams are synchronised) and no push or drain is
 * running: the ring of `context` -- or every ring, OFI_AMD_GIN_ALL_CONTEXTS -- restarts at the
 * consumer's position: records published but not popped are dropped (*dropped, optional, counts
 * them), slots reserved by producers that gave up are free again, and the cursors of GPU and
 * host producers and the GPU producers' horizon are set accordingly.  Which ring a producer
 * gave up on is not recorded, so after a reported time-out reset all of them; only that form
 * clears the status ofi_amd_gin_producer_status reports.  The producers re-issue what they
 * could not put; what the consumer had popped before stays delivered.
 */
#define OFI_AMD_GIN_ALL_CONTEXTS 0xffffffffu
int ofi_amd_gin_rings_reset(ofi_amd_gin_rings_t *rings, uint32_t context, uint64_t *dropped);
/* Raw views for tests / external consumers (host addresses of pinned memory). */
int ofi_amd_gin_rings_view(ofi_amd_gin_rings_t *rings, void **records, uint32_t **sequences,
			   uint32_t *n_contexts, uint32_t *capacity);

/*
 * Launches the synthetic producer: one workgroup per context, each emitting
 * ops_per_context descriptors of the seeded stream in op order (slot =
 * position & (capacity-1), publication by release-store of position+1 to the
 * slot's sequence word).  Returns right after the launch; a host proxy must be
 * draining concurrently or the kernel gives up after spin_limit polls of a
 * still-occupied slot (0 = default) and ofi_amd_gin_producer_status reports
 * -ETIMEDOUT.
 */
int ofi_amd_gin_produce_seeded(ofi_amd_gin_rings_t *rings, uint64_t seed,
			       uint64_t ops_per_context, uint32_t peer_rank,
			       uint32_t signal_every, uint32_t signal_op, uint32_t aggregate_mask,
			       uint64_t spin_limit, void *stream);
/* After the stream has been synchronised: 0, or -ETIMEDOUT if any producer gave up. */
int ofi_amd_gin_producer_status(ofi_amd_gin_rings_t *rings);

/*
 * What device code needs to put descriptors into the ring of one context from any number
 * of wavefronts at once (the multi-producer side of nccl_ofi_mpsc_ring,
 * include/nccl_ofi_mpsc_ring.h:79-118): device addresses of the record and sequence arrays,
 * the producers' reservation cursor (device memory: only producers touch it, the consumer
 * goes by the sequence words) and the status word.  Passed to kernels by value; the
 * wave-collective put itself is ofi_amd_gin_dev_put() in include/ofi_amd_gin_device.h.
 * A ring takes GPU producers (this cursor) or host producers (ofi_amd_gin_ring_push), not both.
 */
typedef struct {
	void *records;       /* 64-byte records, [capacity] */
	uint32_t *sequences; /* [capacity] */
	uint32_t *reserve;   /* [0] next position to hand out, [1] positions below it are known free */
	uint32_t *status;
	uint32_t capacity;
	uint32_t context;
} ofi_amd_gin_dev_ring_t;
int ofi_amd_gin_rings_device_view(ofi_amd_gin_rings_t *rings, uint32_t context,
				  ofi_amd_gin_dev_ring_t *out);

/*
 * Multi-producer launch: waves_per_context wavefronts per context (1..1024, each its own
 * workgroup) put the descriptors of a device-resident table d_table[context][ops_per_context]
 * through ofi_amd_gin_dev_put().  Wave g of a context takes the 64-descriptor groups g,
 * g + waves, g + 2*waves, ...; each group lands in 64 consecutive slots, a wave's groups
 * land in order (per-producer FIFO), the interleaving between waves is up to the hardware.
 * With one wave per context the ring order is the table order.
 */
int ofi_amd_gin_produce_table(ofi_amd_gin_rings_t *rings, const ofi_amd_gin_desc_t *d_table,
			      uint64_t ops_per_context, uint32_t waves_per_context,
			      uint64_t spin_limit, void *stream);

/* Host-side push with the same protocol (CPU producer threads; CAS claim as in
 * nccl_ofi_mpsc_ring::push).  1 pushed, 0 full. */
int ofi_amd_gin_ring_push(ofi_amd_gin_rings_t *rings, uint32_t context,
			  const ofi_amd_gin_desc_t *desc);
/* Single pop (nccl_ofi_mpsc_ring::pop).  1 popped, 0 empty. */
int ofi_amd_gin_ring_pop(ofi_amd_gin_rings_t *rings, uint32_t context, ofi_amd_gin_desc_t *desc);

/* Memory registration table entry the proxy resolves descriptor handles with
 * (gin_remote_mr, include/rdma/gin/nccl_ofi_gin.h:168-183). */
typedef struct {
	uint64_t local_base;
	uint64_t remote_address;
	uint64_t remote_address_offset;
	uint64_t key[OFI_AMD_MAX_NUM_RAILS];
} ofi_amd_gin_mr_t;

/* One RDMA write the proxy would post (fi_writemsg arguments minus libfabric handles), or one
 * RDMA read of a get (fi_read arguments): src is the local buffer -- read from by a write,
 * filled by a read -- and dest the offset in the peer's registration. */
typedef struct {
	uint64_t src;
	uint64_t len;
	uint64_t dest;
	uint64_t key;
	uint32_t rail;
	uint32_t more; /* FI_MORE */
} ofi_amd_gin_write_t;

/* Everything iputSignal derives from one descriptor (224 bytes). */
typedef struct {
	uint32_t seq;
	uint32_t nseg;
	uint32_t imm;        /* GIN_IMM_SEG_DATA, include/rdma/gin/nccl_ofi_gin_types.h:76-79 */
	uint32_t num_writes;
	uint32_t has_meta;
	uint32_t meta_rail;
	uint32_t meta_more;
	uint32_t ack_req;
	ofi_amd_gin_write_t writes[OFI_AMD_MAX_NUM_RAILS];
	uint64_t meta[4];    /* nccl_net_ofi_gin_signal_metadata_msg_t, :150-159 */
} ofi_amd_gin_wire_t;

/* Initiator-side comm state (nccl_ofi_gin_peer_rank_info,
 * include/rdma/gin/nccl_ofi_gin.h:111-163, plus pin state). */
typedef struct {
	ofi_amd_sched_state_t sched;
	uint32_t comm_id;
	uint32_t num_rails;
	uint32_t tx_head;
	uint32_t tx_tail;
	uint32_t consecutive_puts_without_ack;
	uint32_t last_ack_requested_seq;
	uint32_t has_pending_ack_request;
	int32_t pinned_rail_id;
	uint32_t pinned_rail_run;
	uint32_t next_rail_id;
	uint32_t ack_model; /* 0: ACKs only via ofi_amd_gin_apply_ack; 1: immediate ACK on request */
	uint32_t pad;
} ofi_amd_gin_comm_t;

int ofi_amd_gin_comm_init(ofi_amd_gin_comm_t *c, uint32_t comm_id, uint32_t num_rails,
			  uint64_t min_stripe, uint64_t max_small, uint32_t ack_model);
/* iputSignal's derivation for one descriptor.  mrs[0..n_mrs) is the registration table the
 * descriptor's 16-bit handles index.  0; -EINVAL (a NULL argument, a signal op other than
 * 0/INC/ADD, a handle >= n_mrs -- sig_mr 0xffff means "no signal handle"); -EAGAIN (TX window
 * full; the reference blocks in await_tx_window).  *out is all-zero on failure. */
int ofi_amd_gin_iput_signal(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
			    const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out);
/* iget's derivation (src/rdma/gin/nccl_ofi_gin.cpp:879-939): the schedule of d->size from the
 * same scheduler as the puts, one read per stripe in out->writes[0..num_writes), never FI_MORE.
 * A get has no sequence number, takes no room in the TX window and tells the target nothing:
 * seq, nseg, imm, ack_req and the metadata fields of *out are 0 (nseg == 0 marks a get's
 * record), and of *c only the scheduler's counters change.  A size of 0 is one read of length
 * 0, as the reference posts it.  0; -EINVAL (a NULL argument, a descriptor of another kind, a
 * handle >= n_mrs; *out all-zero). */
int ofi_amd_gin_iget(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
		     const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out);
/* Either of the two by the descriptor's kind: what a proxy runs per popped descriptor. */
int ofi_amd_gin_derive(ofi_amd_gin_comm_t *c, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
		       const ofi_amd_gin_desc_t *d, ofi_amd_gin_wire_t *out);
/* apply_rx_consumed, include/rdma/gin/nccl_ofi_gin.h:535-543 */
void ofi_amd_gin_apply_ack(ofi_amd_gin_comm_t *c, uint32_t wire_rx_consumed);
/* Wire encoders, include/rdma/gin/nccl_ofi_gin_types.h:39-181 */
uint32_t ofi_amd_gin_imm(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req);
uint64_t ofi_amd_gin_meta_header(uint32_t comm_id, uint32_t seq, uint32_t nseg, uint32_t ack_req);
uint64_t ofi_amd_gin_ack_msg(uint32_t comm_id, uint32_t rx_consumed);

typedef struct {
	uint64_t descriptors;   /* drained in this call */
	uint64_t signals;       /* of which put-signal */
	uint64_t writes;        /* RDMA writes derived (mode 2) */
	uint64_t checksum;      /* order-sensitive per context, summed over contexts */
	double seconds;         /* wall time from first poll to last descriptor */
	uint64_t empty_polls;
} ofi_amd_gin_proxy_stats_t;

/*
 * The host proxy loop, on the calling thread: drains all rings round-robin until
 * each has delivered ops_per_context descriptors, or timeout_ms passes without
 * progress (-ETIMEDOUT).
 *   mode 0: pop + fold every descriptor into the checksum;
 *   mode 1: also store the descriptors: out_desc[c * ops_per_context + i];
 *   mode 2: also run the derivation per context (comms[c], mrs[0..n_mrs); ofi_amd_gin_derive:
 *           iputSignal's for puts, iget's for gets).  out_wire receives the wire records at
 *           [c * ops_per_context + i]; with out_wire NULL they go round a 64-record array of the
 *           proxy thread's own and are complete in memory there (a post step would read them
 *           from it), so the timed work is the whole derivation either way.  The checksum is
 *           that of mode 0, the descriptors alone: what a proxy does with a record (the posts)
 *           is not this call's, and folding every record into the checksum is checking, not
 *           proxy work.  (Before mode 3 existed, mode 2 folded the records in: a caller that
 *           compared mode 2 checksums gets the mode 0 value now and the former value from mode 3.)
 *   mode 3: mode 2, and every wire record is folded into the checksum after its
 *           descriptor (the parity check of the derived stream at any size).
 * A descriptor whose handles lie outside mrs ends the call with -EINVAL.
 */
int ofi_amd_gin_proxy_drain(ofi_amd_gin_rings_t *rings, uint64_t ops_per_context, int mode,
			    ofi_amd_gin_desc_t *out_desc, ofi_amd_gin_comm_t *comms,
			    const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs, ofi_amd_gin_wire_t *out_wire,
			    uint32_t timeout_ms, ofi_amd_gin_proxy_stats_t *stats);

/*
 * The same loop on n_threads proxy threads (the caller's included), each owning a contiguous
 * range of contexts -- NCCL runs up to NCCL_GIN_MAX_CONNECTIONS = 4 GIN proxy threads
 * (nccl/net.h:38).  Contexts are independent (own ring, own comm state), so the per-context
 * results, and the checksum summed over contexts, do not depend on n_threads.  1..64.
 */
int ofi_amd_gin_proxy_drain_mt(ofi_amd_gin_rings_t *rings, uint64_t ops_per_context, int mode,
			       ofi_amd_gin_desc_t *out_desc, ofi_amd_gin_comm_t *comms,
			       const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs, ofi_amd_gin_wire_t *out_wire,
			       uint32_t timeout_ms, uint32_t n_threads, ofi_amd_gin_proxy_stats_t *stats);

/* ---- initiator side, below the derivation: request pool, posts, pending retry, bounded CQ drain ----
 *
 * What nccl_ofi_rdma_gin_put_comm::iputSignal does with the records it has derived
 * (src/rdma/gin/nccl_ofi_gin.cpp:737-864), send_ack (:267-315), and the progress engine of
 * nccl_ofi_gin_resources (src/rdma/gin/nccl_ofi_gin_resources.cpp:89-166 process_cq,
 * :574-599 progress / retry_pending_reqs): every RDMA write, metadata send and ACK send is a
 * request from one pool; a post that the fabric refuses with -EAGAIN (send queue full) goes
 * to the back of one pending list and is posted again, without FI_MORE, by the next progress
 * call; a progress call reads at most cq_read_count x cq_process_max_iter completions per
 * rail (OFI_NCCL_CQ_READ_COUNT and OFI_NCCL_GIN_CQ_PROCESS_MAX_ITER, both 4 by default,
 * include/nccl_ofi_param.h:104-109), then retries the pending list in order and stops at the
 * first request the fabric still refuses.  The fabric is reached through two callbacks, which
 * is where libfabric's fi_writemsg / fi_sendmsg / fi_send and fi_cq_readfrom go.
 */
#define OFI_AMD_GIN_POST_WRITE 1 /* fi_writemsg with FI_REMOTE_CQ_DATA */
#define OFI_AMD_GIN_POST_META 2  /* fi_sendmsg of the 32-byte metadata message */
#define OFI_AMD_GIN_POST_ACK 3   /* fi_send of the 8-byte ACK */
#define OFI_AMD_GIN_POST_READ 4  /* fi_read of one stripe of a get */

typedef struct {
	uint32_t kind;
	uint32_t rail;
	uint32_t more;    /* FI_MORE: this post does not ring the rail's doorbell */
	uint32_t context; /* completion context: the fabric returns it through cq_read */
	uint32_t peer;
	uint32_t imm;     /* write: immediate data */
	uint64_t src;     /* write: local source; read: local buffer the bytes land in */
	uint64_t len;
	uint64_t dest;
	uint64_t key;
	uint64_t msg[4];  /* metadata message, or msg[0] = the ACK word */
} ofi_amd_gin_post_t; /* 88 bytes */

typedef struct {
	/* 0, -EAGAIN (send queue full: the engine queues the request), any other negative errno */
	int (*post)(void *fabric, const ofi_amd_gin_post_t *post);
	/* completions of rail `rail`: writes up to `max` contexts, returns how many (0: none now) or a
	 * negative errno */
	int (*cq_read)(void *fabric, uint32_t rail, uint32_t *contexts, uint32_t max);
	void *fabric;
} ofi_amd_gin_fabric_ops_t;

typedef struct {
	uint64_t posts;          /* accepted by the fabric at the first attempt */
	uint64_t refused;        /* first attempts answered -EAGAIN (queued) */
	uint64_t retries;        /* posts of queued requests, accepted or not */
	uint64_t retried_ok;     /* of which accepted */
	uint64_t completions;    /* read from the CQs */
	uint32_t pending;        /* queued now */
	uint32_t pending_max;
	uint32_t requests;       /* pool entries in use now */
	uint32_t requests_max;
	uint32_t outstanding_acks;
	uint32_t pad;
} ofi_amd_gin_tx_stats_t;

typedef struct ofi_amd_gin_tx ofi_amd_gin_tx_t;

/* max_requests: size of the request pool (an operation takes one entry plus one per write and
 * one for its metadata message until each completes; an ACK takes one). */
int ofi_amd_gin_tx_create(uint32_t num_rails, uint32_t cq_read_count, uint32_t cq_process_max_iter,
			  uint32_t max_requests, const ofi_amd_gin_fabric_ops_t *ops,
			  ofi_amd_gin_tx_t **out);
int ofi_amd_gin_tx_destroy(ofi_amd_gin_tx_t *tx);
/* Posts the writes of *wire in stripe order and then its metadata message; *request is the
 * handle for ofi_amd_gin_tx_test.  0 also when posts were queued; -ENOMEM when the pool cannot
 * hold the operation (nothing is posted then); another negative errno when the fabric fails a
 * post (the operation is given up as the reference does: what was posted completes unobserved). */
int ofi_amd_gin_tx_iput_signal(ofi_amd_gin_tx_t *tx, uint32_t peer, const ofi_amd_gin_wire_t *wire,
			       int32_t *request);
/* iget below its derivation (:879-939): one read per stripe of *wire (a record of
 * ofi_amd_gin_iget), each a request of the pool, refused posts queued like any other; *request
 * is done once every read has completed.  Return values as ofi_amd_gin_tx_iput_signal. */
int ofi_amd_gin_tx_iget(ofi_amd_gin_tx_t *tx, uint32_t peer, const ofi_amd_gin_wire_t *wire,
			int32_t *request);
/* iflush (src/rdma/gin/nccl_ofi_gin.cpp:941-1003): fences the reads of earlier gets on every
 * rail.  host_slots: num_rails slots of 64 bytes in host memory the fabric can write (the
 * engine clears the first 8 bytes of each); device_flush_buffer: the device buffer that holds
 * `sentinel` (ofi_amd_flush_buffer_fill).  One read of 64 bytes per rail, peer
 * OFI_AMD_GIN_PEER_SELF, src = the rail's slot, dest = device_flush_buffer.
 * ofi_amd_gin_tx_test on the returned request reports done once every slot holds the sentinel
 * (the reads' own completions only return their requests to the pool).  One flush at a time per
 * host_slots, as in the reference. */
#define OFI_AMD_GIN_PEER_SELF 0xffffffffu
int ofi_amd_gin_tx_iflush(ofi_amd_gin_tx_t *tx, void *host_slots, uint64_t device_flush_buffer,
			  uint64_t sentinel, int32_t *request);
/* send_ack: one ACK send on rail 0. */
int ofi_amd_gin_tx_send_ack(ofi_amd_gin_tx_t *tx, uint32_t peer, uint64_t ack_msg);
/* nccl_ofi_gin_resources::progress. */
int ofi_amd_gin_tx_progress(ofi_amd_gin_tx_t *tx);
/* nccl_ofi_rdma_gin_iputsignal_req::test / nccl_ofi_gin_iget_req::test: *done = 1 (and the
 * request is freed) once every post of the operation has completed; for a flush request, once
 * every slot holds the sentinel.  It does not progress. */
int ofi_amd_gin_tx_test(ofi_amd_gin_tx_t *tx, int32_t request, int *done);
int ofi_amd_gin_tx_stats(const ofi_amd_gin_tx_t *tx, ofi_amd_gin_tx_stats_t *out);

/* The in-process fabric of the loop-back runs: per rail a send queue of sq_depth entries and a
 * completion queue.  A post is refused with -EAGAIN while the rail's send queue is full; an
 * entry leaves the send queue when its completion is read.  Entries are transmitted in post
 * order per rail once the rail's doorbell rings: by a post without FI_MORE, or by the queue
 * filling up.  ofi_amd_loopfab_take_transmitted hands the transmitted posts, in the order
 * their doorbells rang, to the caller, who plays the wire and the target; a taken post's
 * completion becomes readable at once. */
typedef struct ofi_amd_loopfab ofi_amd_loopfab_t;
int ofi_amd_loopfab_create(uint32_t num_rails, uint32_t sq_depth, ofi_amd_loopfab_t **out);
int ofi_amd_loopfab_destroy(ofi_amd_loopfab_t *f);
int ofi_amd_loopfab_ops(ofi_amd_loopfab_t *f, ofi_amd_gin_fabric_ops_t *ops);
uint32_t ofi_amd_loopfab_take_transmitted(ofi_amd_loopfab_t *f, ofi_amd_gin_post_t *out, uint32_t cap);
/* The same, one post at a time and in place: the next transmitted post as it stands in its rail's
 * send queue, or NULL when none is waiting.  The pointer is good until completions are next read
 * from the fabric (reading a completion frees the send-queue entry). */
const ofi_amd_gin_post_t *ofi_amd_loopfab_next_transmitted(ofi_amd_loopfab_t *f);
/* Rings every rail's doorbell: posts still waiting behind FI_MORE are transmitted. */
int ofi_amd_loopfab_ring_all(ofi_amd_loopfab_t *f);

/* ---- receiver side: completions -> in-order retire -> signal counters in HBM ---- */

/* One folded signal delivery: add `value` to the 8-byte counter at base + offset
 * (gin_signal_work_entry, include/rdma/gin/nccl_ofi_gin.h:257-299, reduced to what the
 * update needs).  32 bytes. */
typedef struct {
	uint64_t base;     /* signal_base_address: the VA the initiator knows the signal MR by */
	uint64_t offset;
	uint64_t value;
	uint32_t peer;
	uint16_t gate_seq; /* sequence number of the last op folded in */
	uint16_t run_len;  /* number of consecutive ops folded in */
} ofi_amd_gin_signal_work_t;

/* Standalone ACK to send back (gin_ack_msg_t in `msg`). */
typedef struct {
	uint32_t peer;
	uint32_t rx_consumed;
	uint64_t msg;
} ofi_amd_gin_ack_t;

typedef struct ofi_amd_gin_rx ofi_amd_gin_rx_t;

/*
 * Receiver state of one put-comm for n_peers initiators (peer_comm_ids[p] = the comm id
 * peer p expects in ACKs).  Feed it the completions the CQ delivers, in arrival order:
 * handle_signal_write_completion / handle_signal_metadata_completion,
 * src/rdma/gin/nccl_ofi_gin.cpp:1792-1924.  Ops retire strictly in sequence order per
 * peer; consecutive ready signals to the same (base, offset) fold into one work item
 * (retire_completed_peer_iput_ops, :1622-1790); an ACK is queued when a retired op asked
 * for one.  The hand-off of a work item is synchronous here (the reference's closing-path
 * behaviour, :1298-1304), so the output depends only on the arrival order.
 */
int ofi_amd_gin_rx_create(uint32_t n_peers, const uint32_t *peer_comm_ids, ofi_amd_gin_rx_t **out);
int ofi_amd_gin_rx_destroy(ofi_amd_gin_rx_t *rx);
int ofi_amd_gin_rx_write_completion(ofi_amd_gin_rx_t *rx, uint32_t peer, uint32_t imm);
int ofi_amd_gin_rx_metadata(ofi_amd_gin_rx_t *rx, uint32_t peer, const uint64_t meta[4]);
/* Move queued work items / ACKs out (returns how many were written). */
uint32_t ofi_amd_gin_rx_take_work(ofi_amd_gin_rx_t *rx, ofi_amd_gin_signal_work_t *out, uint32_t cap);
uint32_t ofi_amd_gin_rx_take_acks(ofi_amd_gin_rx_t *rx, ofi_amd_gin_ack_t *out, uint32_t cap);
int ofi_amd_gin_rx_cursors(const ofi_amd_gin_rx_t *rx, uint32_t peer, uint32_t *rx_consumed,
			   uint32_t *next_seq);

/* A registered signal region: initiators address it as `base`; its counters live at
 * d_counters (device memory), `size` bytes.  A window backed by several allocations (the
 * reference finds the segment of a counter by its address, ensure_signal_seg,
 * src/rdma/gin/nccl_ofi_gin.cpp:1038-1122) is listed as consecutive regions, each beginning
 * where the one before it ends: an item addressed by the first one's base and an offset beyond
 * its size lands in the region that holds base + offset.  A counter never straddles two. */
typedef struct {
	uint64_t base;
	uint64_t size;
	void *d_counters;
} ofi_amd_gin_signal_region_t;

/*
 * Applies a batch of work items to the signal counters in HBM, replacing the reference's
 * GDRCopy read-modify-write over PCIe (apply_signal_work, nccl_ofi_gin.cpp:1193-1256) and
 * its per-batch same-slot fold (apply_and_complete, :1425-1479): one thread per item, one
 * 64-bit device-scope atomic add each, so items hitting one slot combine in the L2.
 * d_work is device-accessible (pinned host or HBM); regions is a host array (<= 16).
 * Items that match no region or are misaligned are skipped and counted in *d_rejected
 * (device-accessible u32, may be NULL).
 */
int ofi_amd_gin_signal_apply(const ofi_amd_gin_signal_work_t *d_work, uint32_t n,
			     const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
			     uint32_t *d_rejected, void *stream);
/* ofi_amd_gin_signal_apply and, behind it, ofi_amd_flush_post in one launch of one workgroup (a
 * launch costs the host more than either does on the device): all n adds have been performed at
 * device scope before the flush buffer is read back into the slots.  n may be 0 (the flush read
 * alone); -E2BIG beyond 65,536 items: use the two calls.  Arguments as of the two calls. */
int ofi_amd_gin_signal_apply_post(const ofi_amd_gin_signal_work_t *d_work, uint32_t n,
				  const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
				  uint32_t *d_rejected, const void *d_flush_buf, void *slots_dev,
				  uint32_t num_rails, void *stream);

/*
 * A fabric for the transmit engine (and for ofi_amd_rma_ctx_create) that moves the bytes: the
 * initiator and its targets are this process, the wire is device copies on `stream`.  It stands
 * where the reference has libfabric endpoints, the target's progress thread and GDRCopy
 * (what tests/functional/rma.cpp sets up with two ranks).  Send queues and doorbells as
 * ofi_amd_loopfab_*.  Transmitted posts travel in launch groups: a write or a read is one entry
 * of ofi_amd_copy_table_pieces (a read of peer OFI_AMD_GIN_PEER_SELF lands in pinned host
 * memory from ofi_amd_gpu_host_alloc), a group ends in a sentinel read-back, and when that is
 * seen -- inside cq_read, i.e. inside the engine's progress call -- the group's posts complete
 * and the target hears of them in transmission order: write completions and metadata
 * messages go to a receiver (ofi_amd_gin_rx_* with n_peers peers: the state of target rank
 * `peer` towards this initiator), the signal work it releases is applied to `regions` by
 * ofi_amd_gin_signal_apply in the next group's launch, and its ACKs go to on_ack (an ACK post
 * of the engine itself is delivered there too).  Signals therefore land one progress call after
 * the completion that released them: keep calling progress (NCCL's proxy does), or call
 * ofi_amd_devfab_quiesce, which runs the fabric until nothing is in flight or waiting and then
 * waits for the stream (-ETIMEDOUT after timeout_ms, 0 = 10,000).  One thread.  -ENODEV without a
 * GPU.
 */
typedef struct ofi_amd_devfab ofi_amd_devfab_t;
typedef struct {
	uint64_t groups;       /* launch groups */
	uint64_t launches;     /* kernel launches: copies, signal applies, sentinels */
	uint64_t copy_entries;
	uint64_t bytes;        /* payload of writes and reads */
	uint64_t writes;
	uint64_t reads;
	uint64_t flush_reads;
	uint64_t metas;
	uint64_t acks;         /* handed to on_ack */
	uint64_t work_items;   /* folded signal updates applied */
} ofi_amd_devfab_stats_t;
int ofi_amd_devfab_create(uint32_t num_rails, uint32_t sq_depth, uint32_t n_peers, const uint32_t *peer_comm_ids,
			  const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions, void *stream,
			  ofi_amd_devfab_t **out);
int ofi_amd_devfab_destroy(ofi_amd_devfab_t *f);
int ofi_amd_devfab_ops(ofi_amd_devfab_t *f, ofi_amd_gin_fabric_ops_t *ops);
int ofi_amd_devfab_on_ack(ofi_amd_devfab_t *f, int (*on_ack)(void *arg, uint32_t peer, uint64_t ack_msg), void *arg);
/* Rings every rail's doorbell: posts still waiting behind FI_MORE are transmitted. */
int ofi_amd_devfab_ring_all(ofi_amd_devfab_t *f);
int ofi_amd_devfab_quiesce(ofi_amd_devfab_t *f, uint32_t timeout_ms);
int ofi_amd_devfab_stats(const ofi_amd_devfab_t *f, ofi_amd_devfab_stats_t *out);

/*
 * In-process loop-back of the whole GIN path on one GPU: initiator and target are the same
 * device, the "network" is this call.  For every descriptor drained from the rings it
 *   1. derives the wire record (ofi_amd_gin_derive on comms[context], ack_model 0),
 *   2. posts it through the progress engine (ofi_amd_gin_tx_*) into the in-process fabric
 *      (ofi_amd_loopfab_*, sq_depth entries per rail; 0 = 4096): refused posts are queued and
 *      retried by the engine's progress calls -- one every progress_interval operations (0
 *      or 1: after each), as NCCL's proxy alternates between submitting and ginProgress --
 *      and completions are drained 16 per rail and call,
 *   3. executes what the fabric transmits: each RDMA write as a (source, destination, length)
 *      copy -- source mrs[src_mr].local_base + src_off, destination the write's `dest` (give
 *      the destination MR's remote_address_offset the device address of the target buffer) --
 *      one table entry per write; the write completions and the metadata message go
 *      to a receiver (ofi_amd_gin_rx_*, one peer per context), up to reorder_window events
 *      out of order; each RDMA read of a get as the copy the other way -- from the read's
 *      `dest` (the remote MR's remote_address_offset + offset) into the local buffer -- of
 *      which the receiver hears nothing; a stream with gets ends with a flush
 *      (ofi_amd_gin_tx_iflush) whose reads are copies of the sentinel into host slots,
 *   4. sends the receiver's ACKs back through the same engine and fabric; an ACK that arrives
 *      moves the sender's window (ofi_amd_gin_apply_ack),
 * and every batch_writes queued copies (and at the end) launches, in this order on `stream`,
 * ofi_amd_copy_table_pieces for the copies and, as one launch with the sentinel read-back that
 * tells the call when the batch is done, the adds of the signals the receiver has released
 * (ofi_amd_gin_signal_apply_post): a signal is applied after the payloads it covers.  `stream`
 * should be another stream than the one the producing kernel runs on: that kernel waits for this
 * call to drain its rings, and work queued behind it starts only when it has ended.  Two
 * different streams can still share a hardware queue (a process has a few, and streams are dealt
 * onto them), and then the launches on `stream` wait for the producing kernel all the same.  The
 * call does not wait with them: when no launched table set comes back within 20 ms while
 * descriptors are still owed, it allocates another set (up to 256 sets or 256 MiB) and goes on
 * draining, and the launches run once the producers are through (`table_sets_added`; the results
 * are the same, the overlap of copies and draining is lost).  What the
 * reference does with two processes, libfabric and GDRCopy (tests/functional/rma.cpp), runs
 * here as GPU producer -> host proxy -> GPU copy and atomics.
 */
typedef struct {
	uint64_t descriptors;
	uint64_t writes;          /* RDMA writes derived */
	uint64_t copy_entries;    /* copy-table entries: one per write and per read */
	uint64_t bytes;           /* payload bytes moved */
	uint64_t signals;         /* put-signal operations */
	uint64_t work_items;      /* folded signal deliveries applied */
	uint64_t acks;            /* ACKs returned to the senders */
	uint64_t launches;        /* copy + apply launch pairs */
	double seconds;
	uint64_t posts_refused;   /* posts the fabric answered -EAGAIN (send queue full) */
	uint64_t post_retries;    /* posts of queued requests by progress calls */
	uint64_t tx_completions;  /* initiator completions read from the CQs */
	uint32_t pending_max;     /* longest the pending list got */
	uint32_t requests_max;    /* most request-pool entries in use */
	uint64_t reads;           /* RDMA reads of gets */
	uint64_t flush_reads;     /* reads of the flush that fences them (one per rail), 0 without gets */
	/* where the calling thread's time went, nanoseconds over the whole run (the first five from
	 * time stamps around the stages of every 16th operation, scaled up) */
	uint64_t ns_pop_derive;   /* ring pop + ofi_amd_gin_derive */
	uint64_t ns_tx_post;      /* ofi_amd_gin_tx_iput_signal / _iget: pool entries, posts into the fabric */
	uint64_t ns_wire;         /* taking transmitted posts off the fabric, copy-table entries, events */
	uint64_t ns_progress;     /* ofi_amd_gin_tx_progress (CQ drain, retries) + test of the oldest operations */
	uint64_t ns_rx;           /* receiver: completions, metadata, ACKs back into the engine, signal work */
	uint64_t ns_launch_wait;  /* copy / signal launches and the wait for the other table pair's sentinel */
	uint64_t table_sets_added; /* 0 in the ordinary case; see the note on `stream` below */
} ofi_amd_gin_loopback_stats_t;

int ofi_amd_gin_loopback_run(ofi_amd_gin_rings_t *rings, uint64_t ops_per_context,
			     ofi_amd_gin_comm_t *comms, const ofi_amd_gin_mr_t *mrs, uint32_t n_mrs,
			     const ofi_amd_gin_signal_region_t *regions, uint32_t n_regions,
			     uint32_t reorder_window, uint32_t batch_writes, uint32_t sq_depth,
			     uint32_t progress_interval, uint32_t timeout_ms, void *stream,
			     ofi_amd_gin_loopback_stats_t *stats);

/* ======================================================================
 * 5. Tuner: batched cost model and region lookup.
 *    Model: nccl_ofi_tuner_compute_cost + model_get_coll_info_internal_v3,
 *    src/tuner/nccl_ofi_model.cpp:46-234.  Regions:
 *    region_get_coll_info_internal_v3, src/tuner/nccl_ofi_regions.cpp:2070-2157.
 * ====================================================================== */

enum {
	OFI_AMD_PLATFORM_P5_P5E = 0, /* enum nccl_ofi_tuner_platform, */
	OFI_AMD_PLATFORM_P5EN = 1,   /* include/tuner/nccl_ofi_tuner_common.h:18-25 */
	OFI_AMD_PLATFORM_P6 = 2,
	OFI_AMD_PLATFORM_P6_B300 = 3,
};

/* One grid variant: everything that is fixed per tuner context / call. */
typedef struct {
	int32_t platform;
	int32_t pipe_ops;          /* numPipeOps */
	int32_t num_channels;      /* OFI_NCCL_TUNER_NUM_CHANNELS, default 8 */
	int32_t net_comp_overhead; /* OFI_NCCL_TUNER_NET_COMP_OVERHEAD, default 3 */
} ofi_amd_tuner_variant_t;

typedef struct ofi_amd_tuner_plan ofi_amd_tuner_plan_t;

/*
 * A plan fixes the grid axes (host arrays, copied): collectives (ncclFunc_t
 * values), message sizes, node counts, ranks-per-node values, and the
 * algorithm list whose cost cells are emitted (all three protocols each).
 * Point index = ((coll * n_sizes + size) * n_nodes + node) * n_ppn + ppn.
 */
int ofi_amd_tuner_plan_create(const int32_t *colls, uint32_t n_colls, const uint64_t *sizes,
			      uint32_t n_sizes, const uint64_t *nodes, uint32_t n_nodes,
			      const uint32_t *ppn, uint32_t n_ppn, const int32_t *algos,
			      uint32_t n_algos, ofi_amd_tuner_plan_t **out);
int ofi_amd_tuner_plan_destroy(ofi_amd_tuner_plan_t *plan);
uint64_t ofi_amd_tuner_plan_points(const ofi_amd_tuner_plan_t *plan);
uint64_t ofi_amd_tuner_plan_cells(const ofi_amd_tuner_plan_t *plan); /* points * n_algos * 3 */

/*
 * Model grid for n_variants variants in one launch.
 *   d_cost[v * cells + point * n_algos * 3 + a * 3 + proto]  (fp64 of the fp32 cost, -1 = no model)
 *   d_choice[(v * points + point) * 2 + {0,1}] = chosen {algo, proto} or {-1,-1}
 * Either output may be NULL.
 */
int ofi_amd_tuner_model_grid(ofi_amd_tuner_plan_t *plan, const ofi_amd_tuner_variant_t *variants,
			     uint32_t n_variants, double *d_cost, int8_t *d_choice, void *stream);

/*
 * Region grid for n_platforms platforms in one launch.
 *   d_choice[(p * points + point) * 4 + {0,1}] = {algo, proto} or {-1,-1} (fall back to NCCL),
 *   bytes 2..3 = int16 nChannels override, or -1 when the tuner leaves nChannels alone.
 *   d_choice is 4-byte aligned (one record per store).
 */
int ofi_amd_tuner_region_grid(ofi_amd_tuner_plan_t *plan, const int32_t *platforms,
			      uint32_t n_platforms, int8_t *d_choice, void *stream);

/*
 * Point queries: a list of independent tuner questions answered in one launch.
 * This is the form behind the plugin's per-collective calls
 * (nccl_ofi_tuner_get_coll_info / _v2 / _v6 and nccl_ofi_tuner_get_chunk_size,
 * src/tuner/nccl_ofi_tuner.cpp:162-272), which memoises the answers.
 *   kind 0  region decision (region_get_coll_info_internal_v3 / _v2)
 *   kind 1  model decision  (model_get_coll_info_internal_v3 / _v2)
 *   kind 2  region chunk size for a given algo / proto (region_get_chunk_size_internal)
 * allowed_mask bit (algo*3 + proto): for kind 0 a region with a clear bit is passed
 * over (NCCL marked the cell -1, or it lies beyond numAlgo / numProto; v2: PAT, and NVLS
 * tree without NVLS support); for kind 1 only the NVLS-tree/Simple bit is looked at.
 */
typedef struct {
	int32_t platform;
	int32_t kind;
	int32_t coll;
	int32_t pipe_ops;
	int32_t num_channels;
	int32_t net_comp_overhead;
	int32_t algo;
	int32_t proto;
	uint32_t allowed_mask;
	uint32_t pad;
	uint64_t nbytes;
	uint64_t num_ranks;
	uint64_t num_nodes;
} ofi_amd_tuner_query_t; /* 64 bytes */

typedef struct {
	int8_t algo;        /* -1: no decision, fall back to NCCL */
	int8_t proto;
	int16_t nchannels;  /* -1: left alone */
	uint32_t pad;
	uint64_t chunk_size; /* kind 2; 0: left alone */
} ofi_amd_tuner_answer_t; /* 16 bytes */

/* Synchronous: queries and answers are host arrays.  The first call creates what the launches
 * need (a private stream, pinned staging for the questions and answers, the region tables in
 * device memory); ofi_amd_tuner_query_prepare(capacity) does that ahead of time, after which
 * a call with n <= capacity allocates nothing (a launch and a wait on the private stream). */
int ofi_amd_tuner_query_prepare(uint32_t capacity);
int ofi_amd_tuner_query(const ofi_amd_tuner_query_t *queries, uint32_t n,
			ofi_amd_tuner_answer_t *answers);

/* Counters of the tuner plugin's per-communicator answer table (context = what the plugin's
 * init returned): questions answered from the table, questions that went to the GPU, entries
 * evaluated ahead of time by init. */
typedef struct {
	uint64_t hits;
	uint64_t misses;
	uint64_t preloaded;
} ofi_amd_tuner_ctx_stats_t;
int ofi_amd_tuner_ctx_stats(const void *context, ofi_amd_tuner_ctx_stats_t *out);

/*
 * NCCL tuner plugin symbols, same names and struct layouts as the reference exports
 * (src/tuner/nccl_ofi_tuner.cpp:185,242,274; nccl/tuner.h:46-87, tuner_v2.h, tuner_v6.h):
 *   ncclTunerPlugin_v2, ncclTunerPlugin_v3, ncclTunerPlugin_v6
 * They are data symbols of this library; their types are declared in
 * aws_ofi_nccl_amd/csrc/nccl_tuner_abi.h.
 */

#ifdef __cplusplus
}
#endif
#endif /* OFI_AMD_HOTPATH_H_ */

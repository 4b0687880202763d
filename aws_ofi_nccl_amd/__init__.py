"""Python bindings (ctypes) onto libofi_amd_hotpath.so for tests and benchmarks.

The product is the C-ABI library declared in include/ofi_amd_hotpath.h; this
module only loads it and sets argument types.  There is no CPU implementation
behind these bindings: if the library has not been built, loading raises.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libofi_amd_hotpath.so")

_lib = None

c_u8p = ctypes.c_void_p
c_u32 = ctypes.c_uint32
c_u64 = ctypes.c_uint64
c_i32 = ctypes.c_int32
c_vp = ctypes.c_void_p


class SchedState(ctypes.Structure):
    """ofi_amd_sched_state_t"""
    _fields_ = [("rr_small_counter", c_u32), ("rr_counter", c_u32),
                ("max_small_msg_size", c_u64), ("min_stripe_size", c_u64),
                ("num_rails", c_i32), ("pad", c_i32)]


class XferInfo(ctypes.Structure):
    """ofi_amd_xfer_info_t (24 bytes)"""
    _fields_ = [("rail_id", ctypes.c_uint16), ("pad0", ctypes.c_uint16), ("pad1", c_u32),
                ("offset", c_u64), ("msg_size", c_u64)]


class GinDesc(ctypes.Structure):
    """ofi_amd_gin_desc_t (64 bytes)"""
    _fields_ = [("src_off", c_u64), ("dst_off", c_u64), ("size", c_u64), ("signal_off", c_u64),
                ("signal_value", c_u64), ("rank", c_u32), ("signal_op", c_u32),
                ("opt_flags", c_u32), ("context", c_u32), ("src_mr", ctypes.c_uint16),
                ("dst_mr", ctypes.c_uint16), ("sig_mr", ctypes.c_uint16),
                ("kind", ctypes.c_uint16)]


class GinMr(ctypes.Structure):
    """ofi_amd_gin_mr_t"""
    _fields_ = [("local_base", c_u64), ("remote_address", c_u64),
                ("remote_address_offset", c_u64), ("key", c_u64 * 4)]


class GinWrite(ctypes.Structure):
    _fields_ = [("src", c_u64), ("len", c_u64), ("dest", c_u64), ("key", c_u64),
                ("rail", c_u32), ("more", c_u32)]


class GinWire(ctypes.Structure):
    """ofi_amd_gin_wire_t (224 bytes)"""
    _fields_ = [("seq", c_u32), ("nseg", c_u32), ("imm", c_u32), ("num_writes", c_u32),
                ("has_meta", c_u32), ("meta_rail", c_u32), ("meta_more", c_u32),
                ("ack_req", c_u32), ("writes", GinWrite * 4), ("meta", c_u64 * 4)]


class GinPost(ctypes.Structure):
    """ofi_amd_gin_post_t (88 bytes)"""
    _fields_ = [("kind", c_u32), ("rail", c_u32), ("more", c_u32), ("context", c_u32), ("peer", c_u32),
                ("imm", c_u32), ("src", c_u64), ("len", c_u64), ("dest", c_u64), ("key", c_u64),
                ("msg", c_u64 * 4)]


FABRIC_POST_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(GinPost))
FABRIC_CQ_READ_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, c_u32, ctypes.POINTER(c_u32), c_u32)


class GinFabricOps(ctypes.Structure):
    """ofi_amd_gin_fabric_ops_t"""
    _fields_ = [("post", FABRIC_POST_FN), ("cq_read", FABRIC_CQ_READ_FN), ("fabric", ctypes.c_void_p)]


class GinTxStats(ctypes.Structure):
    """ofi_amd_gin_tx_stats_t"""
    _fields_ = [("posts", c_u64), ("refused", c_u64), ("retries", c_u64), ("retried_ok", c_u64),
                ("completions", c_u64), ("pending", c_u32), ("pending_max", c_u32), ("requests", c_u32),
                ("requests_max", c_u32), ("outstanding_acks", c_u32), ("pad", c_u32)]


class GinComm(ctypes.Structure):
    """ofi_amd_gin_comm_t"""
    _fields_ = [("sched", SchedState), ("comm_id", c_u32), ("num_rails", c_u32),
                ("tx_head", c_u32), ("tx_tail", c_u32),
                ("consecutive_puts_without_ack", c_u32), ("last_ack_requested_seq", c_u32),
                ("has_pending_ack_request", c_u32), ("pinned_rail_id", c_i32),
                ("pinned_rail_run", c_u32), ("next_rail_id", c_u32), ("ack_model", c_u32),
                ("pad", c_u32)]


class GinProxyStats(ctypes.Structure):
    _fields_ = [("descriptors", c_u64), ("signals", c_u64), ("writes", c_u64),
                ("checksum", c_u64), ("seconds", ctypes.c_double), ("empty_polls", c_u64)]


class GinDevRing(ctypes.Structure):
    """ofi_amd_gin_dev_ring_t"""
    _fields_ = [("records", c_vp), ("sequences", c_vp), ("reserve", c_vp), ("status", c_vp),
                ("capacity", c_u32), ("context", c_u32)]


class GinLoopbackStats(ctypes.Structure):
    """ofi_amd_gin_loopback_stats_t"""
    _fields_ = [("descriptors", c_u64), ("writes", c_u64), ("copy_entries", c_u64), ("bytes", c_u64),
                ("signals", c_u64), ("work_items", c_u64), ("acks", c_u64), ("launches", c_u64),
                ("seconds", ctypes.c_double), ("posts_refused", c_u64), ("post_retries", c_u64),
                ("tx_completions", c_u64), ("pending_max", c_u32), ("requests_max", c_u32), ("reads", c_u64),
                ("flush_reads", c_u64), ("ns_pop_derive", c_u64), ("ns_tx_post", c_u64), ("ns_wire", c_u64),
                ("ns_progress", c_u64), ("ns_rx", c_u64), ("ns_launch_wait", c_u64), ("table_sets_added", c_u64)]


class GinSignalWork(ctypes.Structure):
    """ofi_amd_gin_signal_work_t (32 bytes)"""
    _fields_ = [("base", c_u64), ("offset", c_u64), ("value", c_u64), ("peer", c_u32),
                ("gate_seq", ctypes.c_uint16), ("run_len", ctypes.c_uint16)]


class GinAck(ctypes.Structure):
    """ofi_amd_gin_ack_t (16 bytes)"""
    _fields_ = [("peer", c_u32), ("rx_consumed", c_u32), ("msg", c_u64)]


class GinSignalRegion(ctypes.Structure):
    """ofi_amd_gin_signal_region_t"""
    _fields_ = [("base", c_u64), ("size", c_u64), ("d_counters", c_vp)]


class EagerHdr(ctypes.Structure):
    """ofi_amd_eager_hdr_t (8 bytes)"""
    _fields_ = [("eager_offset", ctypes.c_uint8), ("prev_batch_count", ctypes.c_uint8),
                ("eager_seq", ctypes.c_uint16), ("tag", c_i32)]


class CtrlEntry(ctypes.Structure):
    """ofi_amd_ctrl_entry_t (64 bytes)"""
    _fields_ = [("buff_offset", c_u64), ("mr_key", c_u64 * 4), ("buff_len", c_u32),
                ("tag", ctypes.c_int16), ("flags", ctypes.c_uint16), ("num_recvs", ctypes.c_uint16),
                ("recv_idx", ctypes.c_uint8), ("entry_used", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 10), ("msg_seq_num", ctypes.c_uint16)]


class CtrlMsg(ctypes.Structure):
    """ofi_amd_ctrl_msg_t (512 bytes)"""
    _fields_ = [("entries", CtrlEntry * 8)]


class EagerEntry(ctypes.Structure):
    """ofi_amd_eager_entry_t (24 bytes)"""
    _fields_ = [("eager_offset", ctypes.c_uint8), ("prev_batch_count", ctypes.c_uint8),
                ("eager_seq", ctypes.c_uint16), ("msg_seq_num", ctypes.c_uint16),
                ("pad", ctypes.c_uint16), ("tag", c_i32), ("recv_len", c_u32), ("cookie", c_u64)]


class EagerTx(ctypes.Structure):
    """ofi_amd_eager_tx_t"""
    _fields_ = [("eager_seq_next", ctypes.c_uint16), ("cur_eager_seq", ctypes.c_uint16),
                ("eager_offset_next", ctypes.c_uint8), ("prev_eager_batch_count", ctypes.c_uint8),
                ("pad", ctypes.c_uint16)]


class SendAction(ctypes.Structure):
    """ofi_amd_send_action_t"""
    _fields_ = [("kind", c_i32), ("req", c_i32), ("msg_seq_num", ctypes.c_uint16),
                ("recv_idx", ctypes.c_uint8), ("no_target_completion", ctypes.c_uint8), ("imm", c_u32),
                ("hdr", EagerHdr), ("size", c_u64), ("remote_buff_offset", c_u64), ("mr_key", c_u64 * 4),
                ("num_xfers", c_u32), ("pad", c_u32), ("xfers", XferInfo * 4)]


class SendState(ctypes.Structure):
    """ofi_amd_send_state_t"""
    _fields_ = [("next_msg_seq_num", ctypes.c_uint16), ("group_sends_remaining", ctypes.c_uint16),
                ("group_num_recvs", ctypes.c_uint16), ("cur_eager_seq", ctypes.c_uint16),
                ("eager_seq_next", ctypes.c_uint16), ("eager_queue_count", ctypes.c_uint8),
                ("eager_offset_next", ctypes.c_uint8), ("prev_eager_batch_count", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 3), ("num_inflight_reqs", c_u32), ("num_inflight_writes", c_u32),
                ("n_ctrl_received", c_u64)]


class EagerCopyItem(ctypes.Structure):
    """ofi_amd_eager_copy_item_t"""
    _fields_ = [("rx_cookie", c_u64), ("dst", c_u64), ("dst_len", c_u64), ("recv_len", c_u32),
                ("req", c_i32), ("sub_idx", c_i32), ("needs_copy", c_i32)]


class RecvState(ctypes.Structure):
    """ofi_amd_recv_state_t"""
    _fields_ = [("next_msg_seq_num", ctypes.c_uint16), ("eager_drain_recv_seq", ctypes.c_uint16),
                ("last_eager_seq", ctypes.c_uint16), ("last_completed_seq", ctypes.c_uint16),
                ("last_eager_offset", ctypes.c_uint8), ("has_processed_eager", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 2), ("num_inflight_reqs", c_u32), ("eager_pending", c_u32),
                ("pad2", c_u32), ("n_ctrl_sent", c_u64)]


DEVFAB_ACK_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, c_u32, c_u64)


class DevfabStats(ctypes.Structure):
    """ofi_amd_devfab_stats_t"""
    _fields_ = [(k, c_u64) for k in ("groups", "launches", "copy_entries", "bytes", "writes", "reads", "flush_reads",
                                     "metas", "acks", "work_items")]


class NetLinkStats(ctypes.Structure):
    """ofi_amd_net_link_stats_t"""
    _fields_ = [(k, c_u64) for k in ("isend_calls", "isend_again", "eager_sends", "write_sends", "rdma_writes",
                                     "payload_bytes", "irecv_calls", "flushes", "launches", "copy_entries",
                                     "eager_copies", "progress_calls", "posts_refused")]


class NetPost(ctypes.Structure):
    """ofi_amd_net_post_t"""
    _fields_ = [("kind", c_u32), ("rail", c_u32), ("context", c_u32), ("imm", c_u32), ("src", c_u64), ("len", c_u64),
                ("dest", c_u64), ("key", c_u64), ("hdr", ctypes.c_uint8 * 8)]


class NetCqe(ctypes.Structure):
    """ofi_amd_net_cqe_t"""
    _fields_ = [("kind", c_u32), ("context", c_u32), ("imm", c_u32), ("pad", c_u32), ("len", c_u64), ("rx_cookie", c_u64),
                ("hdr", ctypes.c_uint8 * 8)]


NET_POST_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(NetPost))
NET_CQ_READ_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(NetCqe), c_u32)
NET_REPOST_RX_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, c_u64)


class NetFabricOps(ctypes.Structure):
    """ofi_amd_net_fabric_ops_t"""
    _fields_ = [("post", NET_POST_FN), ("cq_read", NET_CQ_READ_FN), ("repost_rx", NET_REPOST_RX_FN),
                ("end", ctypes.c_void_p)]


class SendrecvLoopbackStats(ctypes.Structure):
    """ofi_amd_sendrecv_loopback_stats_t"""
    _fields_ = [("messages", c_u64), ("payload_bytes", c_u64), ("eager_messages", c_u64),
                ("write_messages", c_u64), ("rdma_writes", c_u64), ("copy_entries", c_u64),
                ("rounds", c_u64), ("launches", c_u64), ("send_again", c_u64), ("flushes", c_u64),
                ("seconds", ctypes.c_double)]


class TunerQuery(ctypes.Structure):
    """ofi_amd_tuner_query_t (64 bytes)"""
    _fields_ = [("platform", c_i32), ("kind", c_i32), ("coll", c_i32), ("pipe_ops", c_i32),
                ("num_channels", c_i32), ("net_comp_overhead", c_i32), ("algo", c_i32),
                ("proto", c_i32), ("allowed_mask", c_u32), ("pad", c_u32), ("nbytes", c_u64),
                ("num_ranks", c_u64), ("num_nodes", c_u64)]


class TunerAnswer(ctypes.Structure):
    """ofi_amd_tuner_answer_t (16 bytes)"""
    _fields_ = [("algo", ctypes.c_int8), ("proto", ctypes.c_int8), ("nchannels", ctypes.c_int16),
                ("pad", c_u32), ("chunk_size", c_u64)]


class NcclTunerV2(ctypes.Structure):
    """ncclTuner_v2_t"""
    _fields_ = [("name", ctypes.c_char_p),
                ("init", ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t, c_vp,
                                          ctypes.POINTER(c_vp))),
                ("getCollInfo", ctypes.CFUNCTYPE(ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_size_t,
                                                 ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 ctypes.POINTER(ctypes.c_int),
                                                 ctypes.POINTER(ctypes.c_int),
                                                 ctypes.POINTER(ctypes.c_int))),
                ("destroy", ctypes.CFUNCTYPE(ctypes.c_int, c_vp))]


class TunerCtxStats(ctypes.Structure):
    """ofi_amd_tuner_ctx_stats_t"""
    _fields_ = [("hits", c_u64), ("misses", c_u64), ("preloaded", c_u64)]


class NcclTunerV3(ctypes.Structure):
    """ncclTuner_v3_t"""
    _fields_ = [("name", ctypes.c_char_p),
                ("init", ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t, c_vp,
                                          ctypes.POINTER(c_vp))),
                ("getCollInfo", ctypes.CFUNCTYPE(ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_size_t,
                                                 ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_int,
                                                 ctypes.POINTER(ctypes.c_int))),
                ("destroy", ctypes.CFUNCTYPE(ctypes.c_int, c_vp))]


class NcclTunerV6(ctypes.Structure):
    """ncclTuner_v6_t"""
    _fields_ = [("name", ctypes.c_char_p),
                ("init", ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(c_vp), c_u64, ctypes.c_size_t,
                                          ctypes.c_size_t, c_vp, c_vp, c_vp)),
                ("getCollInfo", ctypes.CFUNCTYPE(ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_size_t,
                                                 ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_int, ctypes.POINTER(ctypes.c_int))),
                ("finalize", ctypes.CFUNCTYPE(ctypes.c_int, c_vp)),
                ("getChunkSize", ctypes.CFUNCTYPE(ctypes.c_int, c_vp, ctypes.c_int, ctypes.c_size_t,
                                                  ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                  ctypes.POINTER(ctypes.c_size_t)))]


class TunerVariant(ctypes.Structure):
    _fields_ = [("platform", c_i32), ("pipe_ops", c_i32), ("num_channels", c_i32),
                ("net_comp_overhead", c_i32)]


# name -> (restype, argtypes); every symbol the headers under include/ declare
PROTOTYPES = {
    "ofi_amd_gpu_init": (ctypes.c_int, []),
    "ofi_amd_gpu_get_device_for_addr": (ctypes.c_int, [c_vp, ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_gpu_flush_gpudirect_rdma_writes": (ctypes.c_int, []),
    "ofi_amd_gpu_mem_alloc": (ctypes.c_int, [ctypes.POINTER(c_vp), ctypes.c_size_t]),
    "ofi_amd_gpu_mem_free": (ctypes.c_int, [c_vp]),
    "ofi_amd_gpu_mem_copy_host_to_device": (ctypes.c_int, [c_vp, c_vp, ctypes.c_size_t]),
    "ofi_amd_gpu_mem_copy_device_to_host": (ctypes.c_int, [c_vp, c_vp, ctypes.c_size_t]),
    "ofi_amd_gpu_stream_synchronize": (ctypes.c_int, [c_vp]),
    "ofi_amd_async_error_fetch": (ctypes.c_int, [ctypes.POINTER(c_u32)]),
    "ofi_amd_gpu_get_dma_buf_fd": (ctypes.c_int, [c_vp, ctypes.c_size_t,
                                                  ctypes.POINTER(ctypes.c_int),
                                                  ctypes.POINTER(ctypes.c_size_t)]),
    "ofi_amd_gpu_have_dma_buf_attr": (ctypes.c_int, []),
    "ofi_amd_gpu_have_gdr_support_attr": (ctypes.c_int, []),
    "ofi_amd_gpu_set_current_device": (ctypes.c_int, [ctypes.c_int]),
    "ofi_amd_gpu_get_current_device": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_gpu_get_address_range": (ctypes.c_int, [c_vp, ctypes.POINTER(c_vp),
                                                     ctypes.POINTER(ctypes.c_size_t)]),
    "ofi_amd_gpu_seg_is_host": (ctypes.c_int, [c_vp, ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_gpu_host_alloc": (ctypes.c_int, [ctypes.POINTER(c_vp), ctypes.c_size_t]),
    "ofi_amd_gpu_host_free": (ctypes.c_int, [c_vp]),
    "ofi_amd_gpu_host_get_device_pointer": (ctypes.c_int, [ctypes.POINTER(c_vp), c_vp]),
    "ofi_amd_sched_batch": (ctypes.c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, c_vp, c_vp]),
    "ofi_amd_sched_stream_release": (ctypes.c_int, [c_vp]),
    "ofi_amd_sched_batch_noalloc": (ctypes.c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, c_vp, c_vp]),
    "ofi_amd_sched_get_schedule": (ctypes.c_int, [ctypes.POINTER(SchedState), c_u64, c_u64,
                                                  ctypes.POINTER(XferInfo)]),
    "ofi_amd_bounce_scatter": (ctypes.c_int, [c_vp, c_u64, c_vp, c_u64, c_vp, c_vp, c_vp, c_u32, c_vp,
                                              c_vp]),
    "ofi_amd_eager_copy_batch": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_u32, c_vp, c_vp,
                                                c_vp]),
    "ofi_amd_copy_table": (ctypes.c_int, [c_vp, c_vp, c_vp, c_u32, c_vp]),
    "ofi_amd_copy_table_pieces": (ctypes.c_int, [c_vp, c_vp, c_vp, c_u32, c_u32, c_vp]),
    "ofi_amd_gin_loopback_run": (ctypes.c_int, [c_vp, c_u64, c_vp, c_vp, c_u32, ctypes.POINTER(GinSignalRegion), c_u32,
                                                c_u32, c_u32, c_u32, c_u32, c_u32, c_vp,
                                                ctypes.POINTER(GinLoopbackStats)]),
    "ofi_amd_loopfab_ring_all": (ctypes.c_int, [c_vp]),
    "ofi_amd_flush_buffer_fill": (ctypes.c_int, [c_vp, c_u64, c_vp]),
    "ofi_amd_flush_post": (ctypes.c_int, [c_vp, c_vp, c_u32, c_vp]),
    "ofi_amd_flush_test": (ctypes.c_int, [c_vp, c_u32, c_u64]),
    "ofi_amd_flush_read": (ctypes.c_int, [c_vp, c_vp, c_u32, c_vp, c_vp]),
    "ofi_amd_devcopy_register": (ctypes.c_int, [c_vp, ctypes.c_size_t, ctypes.POINTER(c_vp)]),
    "ofi_amd_devcopy_cpu_mapped": (ctypes.c_int, [c_vp]),
    "ofi_amd_devcopy_to_device": (ctypes.c_int, [c_vp, c_vp, ctypes.c_size_t, ctypes.c_size_t]),
    "ofi_amd_devcopy_from_device": (ctypes.c_int, [c_vp, ctypes.c_size_t, c_vp,
                                                   ctypes.c_size_t]),
    "ofi_amd_devcopy_forced_pcie_copy": (ctypes.c_int, []),
    "ofi_amd_devcopy_deregister": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_rings_create": (ctypes.c_int, [c_u32, c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_rings_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_rings_view": (ctypes.c_int, [c_vp, ctypes.POINTER(c_vp), ctypes.POINTER(c_vp),
                                              ctypes.POINTER(c_u32), ctypes.POINTER(c_u32)]),
    "ofi_amd_gin_produce_seeded": (ctypes.c_int, [c_vp, c_u64, c_u64, c_u32, c_u32, c_u32, c_u32,
                                                  c_u64, c_vp]),
    "ofi_amd_gin_rings_device_view": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinDevRing)]),
    "ofi_amd_gin_produce_table": (ctypes.c_int, [c_vp, c_vp, c_u64, c_u32, c_u64, c_vp]),
    "ofi_amd_gin_producer_status": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_rings_reset": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(c_u64)]),
    "ofi_amd_gin_ring_push": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinDesc)]),
    "ofi_amd_gin_ring_pop": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinDesc)]),
    "ofi_amd_gin_comm_init": (ctypes.c_int, [ctypes.POINTER(GinComm), c_u32, c_u32, c_u64, c_u64,
                                             c_u32]),
    "ofi_amd_gin_iput_signal": (ctypes.c_int, [ctypes.POINTER(GinComm), ctypes.POINTER(GinMr), c_u32,
                                               ctypes.POINTER(GinDesc), ctypes.POINTER(GinWire)]),
    "ofi_amd_gin_iget": (ctypes.c_int, [ctypes.POINTER(GinComm), ctypes.POINTER(GinMr), c_u32,
                                        ctypes.POINTER(GinDesc), ctypes.POINTER(GinWire)]),
    "ofi_amd_gin_derive": (ctypes.c_int, [ctypes.POINTER(GinComm), ctypes.POINTER(GinMr), c_u32,
                                          ctypes.POINTER(GinDesc), ctypes.POINTER(GinWire)]),
    "ofi_amd_gin_apply_ack": (None, [ctypes.POINTER(GinComm), c_u32]),
    "ofi_amd_gin_imm": (c_u32, [c_u32, c_u32, c_u32, c_u32]),
    "ofi_amd_gin_meta_header": (c_u64, [c_u32, c_u32, c_u32, c_u32]),
    "ofi_amd_gin_ack_msg": (c_u64, [c_u32, c_u32]),
    "ofi_amd_gin_proxy_drain": (ctypes.c_int, [c_vp, c_u64, ctypes.c_int, c_vp, c_vp, c_vp, c_u32, c_vp,
                                               c_u32, ctypes.POINTER(GinProxyStats)]),
    "ofi_amd_gin_proxy_drain_mt": (ctypes.c_int, [c_vp, c_u64, ctypes.c_int, c_vp, c_vp, c_vp, c_u32, c_vp,
                                                  c_u32, c_u32, ctypes.POINTER(GinProxyStats)]),
    "ofi_amd_gin_tx_create": (ctypes.c_int, [c_u32, c_u32, c_u32, c_u32, ctypes.POINTER(GinFabricOps),
                                             ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_tx_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_tx_iput_signal": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinWire),
                                                  ctypes.POINTER(c_i32)]),
    "ofi_amd_gin_tx_iget": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinWire), ctypes.POINTER(c_i32)]),
    "ofi_amd_gin_tx_iflush": (ctypes.c_int, [c_vp, c_vp, c_u64, c_u64, ctypes.POINTER(c_i32)]),
    "ofi_amd_gin_tx_send_ack": (ctypes.c_int, [c_vp, c_u32, c_u64]),
    "ofi_amd_gin_tx_progress": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_tx_test": (ctypes.c_int, [c_vp, c_i32, ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_gin_tx_stats": (ctypes.c_int, [c_vp, ctypes.POINTER(GinTxStats)]),
    # include/ofi_amd_rma_abi.h: set-up, then the data-path members of ncclRma_v15_t (int = ncclResult_t)
    "ofi_amd_rma_ctx_create": (ctypes.c_int, [c_u32, c_u32, c_u64, c_u64, ctypes.POINTER(GinFabricOps), c_u32,
                                              c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_ctx_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_rma_mr_create": (ctypes.c_int, [c_vp, c_u64, c_vp, c_vp, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_mr_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_rma_set_flush_buffers": (ctypes.c_int, [c_vp, c_vp, c_u64, c_u64]),
    "ofi_amd_rma_ack_received": (ctypes.c_int, [c_vp, c_u32, c_u64]),
    "ofi_amd_rma_peer_state": (ctypes.POINTER(GinComm), [c_vp, c_u32]),
    "ofi_amd_rma_tx_stats": (ctypes.c_int, [c_vp, ctypes.POINTER(GinTxStats)]),
    "ofi_amd_rma_iput": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32, c_u32,
                                        ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_iputSignal": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32,
                                              c_u64, c_vp, c_u64, c_u32, ctypes.c_bool, c_u32,
                                              ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_iget": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32, c_u32,
                                        ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_iflush": (ctypes.c_int, [c_vp, ctypes.c_int, c_vp, c_u32, ctypes.POINTER(c_vp)]),
    # the same operations as the older op-tables spell them (no optFlags; v13 / v11 no isStrongSignal;
    # v11 no context number)
    "ofi_amd_rma_iput_v14": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32,
                                            ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_iputSignal_v14": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp,
                                                  c_u32, c_u64, c_vp, c_u64, c_u32, ctypes.c_bool,
                                                  ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_iget_v14": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32,
                                            ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_iputSignal_v13": (ctypes.c_int, [c_vp, ctypes.c_int, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp,
                                                  c_u32, c_u64, c_vp, c_u64, c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_iput_v11": (ctypes.c_int, [c_vp, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32,
                                            ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_iputSignal_v11": (ctypes.c_int, [c_vp, c_u64, c_vp, ctypes.c_size_t, c_u64, c_vp, c_u32, c_u64, c_vp,
                                                  c_u64, c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_rma_test": (ctypes.c_int, [c_vp, c_vp, ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_rma_rmaProgress": (ctypes.c_int, [c_vp]),
    # include/ofi_amd_net_abi.h: an in-process link, then the data-path members of ncclNet_vN_t
    "ofi_amd_net_send_comm_create": (ctypes.c_int, [c_u32, ctypes.c_int64, c_u64, c_u64, ctypes.POINTER(NetFabricOps),
                                                    ctypes.POINTER(c_vp)]),
    "ofi_amd_net_send_comm_mailbox": (c_vp, [c_vp]),
    "ofi_amd_net_recv_comm_create": (ctypes.c_int, [c_u32, ctypes.POINTER(NetFabricOps), c_vp, c_vp,
                                                    ctypes.POINTER(c_vp)]),
    "ofi_amd_net_comm_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_netfab_create": (ctypes.c_int, [c_u32, c_u32, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_netfab_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_netfab_ops": (ctypes.c_int, [c_vp, ctypes.POINTER(NetFabricOps), ctypes.POINTER(NetFabricOps)]),
    "ofi_amd_netfab_rx_pool": (c_vp, [c_vp]),
    "ofi_amd_netfab_connect": (ctypes.c_int, [c_vp, c_vp]),
    "ofi_amd_netfab_counts": (ctypes.c_int, [c_vp, ctypes.POINTER(c_u64), ctypes.POINTER(c_u64)]),
    "ofi_amd_net_link_create": (ctypes.c_int, [c_u32, ctypes.c_int64, c_u64, c_u64, c_u32, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_net_link_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_net_link_send_comm": (c_vp, [c_vp]),
    "ofi_amd_net_link_recv_comm": (c_vp, [c_vp]),
    "ofi_amd_net_link_stats": (ctypes.c_int, [c_vp, ctypes.POINTER(NetLinkStats)]),
    "ofi_amd_net_link_state": (ctypes.c_int, [c_vp, ctypes.POINTER(SendState), ctypes.POINTER(RecvState)]),
    "ofi_amd_net_isend": (ctypes.c_int, [c_vp, c_vp, ctypes.c_size_t, ctypes.c_int, c_vp, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_net_irecv": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(c_vp), ctypes.POINTER(ctypes.c_size_t),
                                         ctypes.POINTER(ctypes.c_int), ctypes.POINTER(c_vp), ctypes.POINTER(c_vp),
                                         ctypes.POINTER(c_vp)]),
    "ofi_amd_net_iflush": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(c_vp), ctypes.POINTER(ctypes.c_int),
                                          ctypes.POINTER(c_vp), ctypes.POINTER(c_vp)]),
    "ofi_amd_net_test": (ctypes.c_int, [c_vp, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_net_isend_v5": (ctypes.c_int, [c_vp, c_vp, ctypes.c_int, ctypes.c_int, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_net_irecv_v5": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(c_vp), ctypes.POINTER(ctypes.c_int),
                                            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(c_vp), ctypes.POINTER(c_vp)]),
    "ofi_amd_net_isend_v9": (ctypes.c_int, [c_vp, c_vp, ctypes.c_size_t, ctypes.c_int, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_net_irecv_v9": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(c_vp), ctypes.POINTER(ctypes.c_size_t),
                                            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(c_vp), ctypes.POINTER(c_vp)]),
    "ofi_amd_devfab_create": (ctypes.c_int, [c_u32, c_u32, c_u32, ctypes.POINTER(c_u32), ctypes.POINTER(GinSignalRegion),
                                             c_u32, c_vp, ctypes.POINTER(c_vp)]),
    "ofi_amd_devfab_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_devfab_ops": (ctypes.c_int, [c_vp, ctypes.POINTER(GinFabricOps)]),
    "ofi_amd_devfab_on_ack": (ctypes.c_int, [c_vp, DEVFAB_ACK_FN, c_vp]),
    "ofi_amd_devfab_ring_all": (ctypes.c_int, [c_vp]),
    "ofi_amd_devfab_quiesce": (ctypes.c_int, [c_vp, c_u32]),
    "ofi_amd_devfab_stats": (ctypes.c_int, [c_vp, ctypes.POINTER(DevfabStats)]),
    "ofi_amd_loopfab_create": (ctypes.c_int, [c_u32, c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_loopfab_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_loopfab_ops": (ctypes.c_int, [c_vp, ctypes.POINTER(GinFabricOps)]),
    "ofi_amd_loopfab_take_transmitted": (c_u32, [c_vp, ctypes.POINTER(GinPost), c_u32]),
    "ofi_amd_loopfab_next_transmitted": (ctypes.POINTER(GinPost), [c_vp]),
    "ofi_amd_gin_rx_create": (ctypes.c_int, [c_u32, ctypes.POINTER(c_u32), ctypes.POINTER(c_vp)]),
    "ofi_amd_gin_rx_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_gin_rx_write_completion": (ctypes.c_int, [c_vp, c_u32, c_u32]),
    "ofi_amd_gin_rx_metadata": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(c_u64)]),
    "ofi_amd_gin_rx_take_work": (c_u32, [c_vp, ctypes.POINTER(GinSignalWork), c_u32]),
    "ofi_amd_gin_rx_take_acks": (c_u32, [c_vp, ctypes.POINTER(GinAck), c_u32]),
    "ofi_amd_gin_rx_cursors": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(c_u32),
                                              ctypes.POINTER(c_u32)]),
    "ofi_amd_gin_signal_apply": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinSignalRegion),
                                                c_u32, c_vp, c_vp]),
    "ofi_amd_gin_signal_apply_post": (ctypes.c_int, [c_vp, c_u32, ctypes.POINTER(GinSignalRegion),
                                                     c_u32, c_vp, c_vp, c_vp, c_u32, c_vp]),
    "ofi_amd_rdma_imm": (c_u32, [c_u32, c_u32, c_u32, c_u32]),
    "ofi_amd_rdma_imm_decode": (None, [c_u32] + [ctypes.POINTER(c_u32)] * 4),
    "ofi_amd_ctrl_mailbox_slot": (c_u32, [ctypes.c_uint16]),
    "ofi_amd_ctrl_msg_fill": (ctypes.c_int, [ctypes.POINTER(CtrlMsg), ctypes.c_uint16, ctypes.c_uint16,
                                             ctypes.POINTER(c_u64), ctypes.POINTER(c_u32),
                                             ctypes.POINTER(ctypes.c_int), ctypes.POINTER(c_u64), c_u32,
                                             ctypes.c_int]),
    "ofi_amd_ctrl_msg_ready": (ctypes.c_int, [ctypes.POINTER(CtrlMsg), ctypes.c_uint16, ctypes.c_int,
                                              ctypes.c_int]),
    "ofi_amd_ctrl_msg_find_tag": (ctypes.c_int, [ctypes.POINTER(CtrlMsg), ctypes.c_int]),
    "ofi_amd_seq_before": (ctypes.c_int, [ctypes.c_uint16, ctypes.c_uint16]),
    "ofi_amd_eager_seq_before": (ctypes.c_int, [ctypes.c_uint16, ctypes.c_uint16]),
    "ofi_amd_eager_entry_less": (ctypes.c_int, [ctypes.POINTER(EagerEntry), ctypes.POINTER(EagerEntry)]),
    "ofi_amd_eager_entry_can_process": (ctypes.c_int, [ctypes.c_int, ctypes.c_uint16, ctypes.c_uint8,
                                                       ctypes.POINTER(EagerEntry)]),
    "ofi_amd_eager_rxq_create": (ctypes.c_int, [ctypes.POINTER(c_vp)]),
    "ofi_amd_eager_rxq_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_eager_rxq_insert": (ctypes.c_int, [c_vp, ctypes.POINTER(EagerEntry)]),
    "ofi_amd_eager_rxq_drain": (c_u32, [c_vp, ctypes.POINTER(EagerEntry), c_u32]),
    "ofi_amd_eager_rxq_pending": (c_u32, [c_vp]),
    "ofi_amd_eager_rxq_peek": (c_u32, [c_vp, ctypes.POINTER(EagerEntry), c_u32]),
    "ofi_amd_eager_tx_init": (None, [ctypes.POINTER(EagerTx)]),
    "ofi_amd_eager_tx_assign": (None, [ctypes.POINTER(EagerTx), c_i32, ctypes.POINTER(EagerHdr)]),
    "ofi_amd_eager_tx_advance": (None, [ctypes.POINTER(EagerTx)]),
    "ofi_amd_eager_fits": (ctypes.c_int, [c_u64, ctypes.c_int64]),
    "ofi_amd_msgbuff_create": (ctypes.c_int, [ctypes.c_uint16, ctypes.c_uint16, ctypes.c_uint16,
                                              ctypes.POINTER(c_vp)]),
    "ofi_amd_msgbuff_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_msgbuff_insert": (ctypes.c_int, [c_vp, ctypes.c_uint16, c_vp, ctypes.c_int,
                                              ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_msgbuff_replace": (ctypes.c_int, [c_vp, ctypes.c_uint16, c_vp, ctypes.c_int,
                                               ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_msgbuff_retrieve": (ctypes.c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(c_vp),
                                                ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_msgbuff_complete": (ctypes.c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_send_comm_create": (ctypes.c_int, [c_u32, c_u32, ctypes.c_int64, c_u64, c_u64,
                                                ctypes.POINTER(c_vp)]),
    "ofi_amd_send_comm_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_send_comm_mailbox": (ctypes.POINTER(CtrlMsg), [c_vp]),
    "ofi_amd_send_comm_send": (ctypes.c_int, [c_vp, c_u64, c_i32, ctypes.POINTER(SendAction)]),
    "ofi_amd_send_comm_completion": (ctypes.c_int, [c_vp, c_i32]),
    "ofi_amd_send_comm_test": (ctypes.c_int, [c_vp, c_i32, ctypes.POINTER(ctypes.c_int),
                                              ctypes.POINTER(c_u64)]),
    "ofi_amd_send_comm_state": (None, [c_vp, ctypes.POINTER(SendState)]),
    "ofi_amd_recv_comm_create": (ctypes.c_int, [c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_recv_comm_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_recv_comm_recv": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(c_u64),
                                              ctypes.POINTER(c_u64), ctypes.POINTER(ctypes.c_int),
                                              ctypes.POINTER(c_u64), ctypes.c_int, ctypes.POINTER(CtrlMsg),
                                              ctypes.POINTER(c_i32), ctypes.POINTER(ctypes.c_uint16)]),
    "ofi_amd_recv_comm_eager_arrival": (ctypes.c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(EagerHdr),
                                                       c_u32, c_u64]),
    "ofi_amd_recv_comm_write_arrival": (ctypes.c_int, [c_vp, c_u32, c_u64]),
    "ofi_amd_recv_comm_ctrl_sent": (ctypes.c_int, [c_vp, c_i32]),
    "ofi_amd_recv_comm_take_copies": (c_u32, [c_vp, ctypes.POINTER(EagerCopyItem), c_u32]),
    "ofi_amd_recv_comm_copy_done": (ctypes.c_int, [c_vp, c_i32, c_i32]),
    "ofi_amd_recv_comm_test": (ctypes.c_int, [c_vp, c_i32, ctypes.POINTER(ctypes.c_int),
                                              ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_recv_comm_state": (None, [c_vp, ctypes.POINTER(RecvState)]),
    "ofi_amd_recv_comm_flush": (ctypes.c_int, [c_vp, ctypes.c_int, ctypes.POINTER(ctypes.c_int),
                                               ctypes.POINTER(c_i32)]),
    "ofi_amd_recv_comm_flush_test": (ctypes.c_int, [c_vp, c_i32, c_vp, c_u32, c_u64,
                                                    ctypes.POINTER(ctypes.c_int)]),
    "ofi_amd_sendrecv_loopback_run": (ctypes.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_u64, c_u32, c_u32, c_u32,
                                                     c_vp, c_u64, c_u32, c_vp,
                                                     ctypes.POINTER(SendrecvLoopbackStats)]),
    "ofi_amd_tuner_plan_create": (ctypes.c_int, [c_vp, c_u32, c_vp, c_u32, c_vp, c_u32, c_vp,
                                                 c_u32, c_vp, c_u32, ctypes.POINTER(c_vp)]),
    "ofi_amd_tuner_plan_destroy": (ctypes.c_int, [c_vp]),
    "ofi_amd_tuner_plan_points": (c_u64, [c_vp]),
    "ofi_amd_tuner_plan_cells": (c_u64, [c_vp]),
    "ofi_amd_tuner_model_grid": (ctypes.c_int, [c_vp, c_vp, c_u32, c_vp, c_vp, c_vp]),
    "ofi_amd_tuner_region_grid": (ctypes.c_int, [c_vp, c_vp, c_u32, c_vp, c_vp]),
    "ofi_amd_tuner_query": (ctypes.c_int, [c_vp, c_u32, c_vp]),
    "ofi_amd_tuner_query_prepare": (ctypes.c_int, [c_u32]),
    "ofi_amd_tuner_ctx_stats": (ctypes.c_int, [c_vp, ctypes.POINTER(TunerCtxStats)]),
}


def load(path=None):
    """Load the product library; raises if it is missing (there is no fallback)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise RuntimeError(
            "%s not built: run `python -m aws_ofi_nccl_amd.build` (hipcc, gfx950)" % p)
    lib = ctypes.CDLL(p)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def check(rc, what="call"):
    if rc != 0:
        raise RuntimeError("%s failed: %d (%s)" % (what, rc, os.strerror(-rc) if rc < 0 else rc))

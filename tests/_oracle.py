"""ctypes bindings onto the CPU oracle (oracle/liboracle.so) and, where built, the
reference's self-contained headers (oracle/_ref/libref.so).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

c_u32 = ctypes.c_uint32
c_u64 = ctypes.c_uint64
c_i32 = ctypes.c_int32
c_vp = ctypes.c_void_p
c_int = ctypes.c_int


class Sched(ctypes.Structure):
    _fields_ = [("rr_small_counter", c_u32), ("rr_counter", c_u32), ("max_small_msg_size", c_u64),
                ("min_stripe_size", c_u64), ("num_rails", c_i32), ("pad", c_i32)]


class Xfer(ctypes.Structure):
    _fields_ = [("rail_id", ctypes.c_uint16), ("pad0", ctypes.c_uint16), ("pad1", c_u32),
                ("offset", c_u64), ("msg_size", c_u64)]


class GinDesc(ctypes.Structure):
    _fields_ = [("src_off", c_u64), ("dst_off", c_u64), ("size", c_u64), ("signal_off", c_u64),
                ("signal_value", c_u64), ("rank", c_u32), ("signal_op", c_u32),
                ("opt_flags", c_u32), ("context", c_u32), ("src_mr", ctypes.c_uint16),
                ("dst_mr", ctypes.c_uint16), ("sig_mr", ctypes.c_uint16),
                ("kind", ctypes.c_uint16)]


class GinWrite(ctypes.Structure):
    _fields_ = [("src", c_u64), ("len", c_u64), ("dest", c_u64), ("key", c_u64),
                ("rail", c_u32), ("more", c_u32)]


class GinWire(ctypes.Structure):
    _fields_ = [("seq", c_u32), ("nseg", c_u32), ("imm", c_u32), ("num_writes", c_u32),
                ("has_meta", c_u32), ("meta_rail", c_u32), ("meta_more", c_u32),
                ("ack_req", c_u32), ("writes", GinWrite * 4), ("meta", c_u64 * 4)]


class GinPost(ctypes.Structure):
    _fields_ = [("kind", c_u32), ("rail", c_u32), ("more", c_u32), ("context", c_u32), ("peer", c_u32),
                ("imm", c_u32), ("src", c_u64), ("len", c_u64), ("dest", c_u64), ("key", c_u64),
                ("msg", c_u64 * 4)]


FABRIC_POST_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(GinPost))
FABRIC_CQ_READ_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, c_u32, ctypes.POINTER(c_u32), c_u32)


class GinFabricOps(ctypes.Structure):
    _fields_ = [("post", FABRIC_POST_FN), ("cq_read", FABRIC_CQ_READ_FN), ("fabric", ctypes.c_void_p)]


class GinTxStats(ctypes.Structure):
    _fields_ = [("posts", c_u64), ("refused", c_u64), ("retries", c_u64), ("retried_ok", c_u64),
                ("completions", c_u64), ("pending", c_u32), ("pending_max", c_u32), ("requests", c_u32),
                ("requests_max", c_u32), ("outstanding_acks", c_u32), ("pad", c_u32)]


class GinMr(ctypes.Structure):
    _fields_ = [("local_base", c_u64), ("remote_address", c_u64),
                ("remote_address_offset", c_u64), ("key", c_u64 * 4)]


class GinComm(ctypes.Structure):
    _fields_ = [("sched", Sched), ("comm_id", c_u32), ("num_rails", c_u32), ("tx_head", c_u32),
                ("tx_tail", c_u32), ("consecutive_puts_without_ack", c_u32),
                ("last_ack_requested_seq", c_u32), ("has_pending_ack_request", c_u32),
                ("pinned_rail_id", c_i32), ("pinned_rail_run", c_u32), ("next_rail_id", c_u32),
                ("ack_model", c_u32), ("pad", c_u32)]


class GinSignalWork(ctypes.Structure):
    _fields_ = [("base", c_u64), ("offset", c_u64), ("value", c_u64), ("peer", c_u32),
                ("gate_seq", ctypes.c_uint16), ("run_len", ctypes.c_uint16)]


class GinAck(ctypes.Structure):
    _fields_ = [("peer", c_u32), ("rx_consumed", c_u32), ("msg", c_u64)]


class EagerHdr(ctypes.Structure):
    _fields_ = [("eager_offset", ctypes.c_uint8), ("prev_batch_count", ctypes.c_uint8),
                ("eager_seq", ctypes.c_uint16), ("tag", c_i32)]


class CtrlEntry(ctypes.Structure):
    _fields_ = [("buff_offset", c_u64), ("mr_key", c_u64 * 4), ("buff_len", c_u32),
                ("tag", ctypes.c_int16), ("flags", ctypes.c_uint16), ("num_recvs", ctypes.c_uint16),
                ("recv_idx", ctypes.c_uint8), ("entry_used", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 10), ("msg_seq_num", ctypes.c_uint16)]


class CtrlMsg(ctypes.Structure):
    _fields_ = [("entries", CtrlEntry * 8)]


class EagerEntry(ctypes.Structure):
    _fields_ = [("eager_offset", ctypes.c_uint8), ("prev_batch_count", ctypes.c_uint8),
                ("eager_seq", ctypes.c_uint16), ("msg_seq_num", ctypes.c_uint16),
                ("pad", ctypes.c_uint16), ("tag", c_i32), ("recv_len", c_u32), ("cookie", c_u64)]


class EagerTx(ctypes.Structure):
    _fields_ = [("eager_seq_next", ctypes.c_uint16), ("cur_eager_seq", ctypes.c_uint16),
                ("eager_offset_next", ctypes.c_uint8), ("prev_eager_batch_count", ctypes.c_uint8),
                ("pad", ctypes.c_uint16)]


class SendAction(ctypes.Structure):
    _fields_ = [("kind", c_i32), ("req", c_i32), ("msg_seq_num", ctypes.c_uint16),
                ("recv_idx", ctypes.c_uint8), ("no_target_completion", ctypes.c_uint8), ("imm", c_u32),
                ("hdr", EagerHdr), ("size", c_u64), ("remote_buff_offset", c_u64), ("mr_key", c_u64 * 4),
                ("num_xfers", c_u32), ("pad", c_u32), ("xfers", Xfer * 4)]


class SendState(ctypes.Structure):
    _fields_ = [("next_msg_seq_num", ctypes.c_uint16), ("group_sends_remaining", ctypes.c_uint16),
                ("group_num_recvs", ctypes.c_uint16), ("cur_eager_seq", ctypes.c_uint16),
                ("eager_seq_next", ctypes.c_uint16), ("eager_queue_count", ctypes.c_uint8),
                ("eager_offset_next", ctypes.c_uint8), ("prev_eager_batch_count", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 3), ("num_inflight_reqs", c_u32), ("num_inflight_writes", c_u32),
                ("n_ctrl_received", c_u64)]


class EagerCopyItem(ctypes.Structure):
    _fields_ = [("rx_cookie", c_u64), ("dst", c_u64), ("dst_len", c_u64), ("recv_len", c_u32),
                ("req", c_i32), ("sub_idx", c_i32), ("needs_copy", c_i32)]


class RecvState(ctypes.Structure):
    _fields_ = [("next_msg_seq_num", ctypes.c_uint16), ("eager_drain_recv_seq", ctypes.c_uint16),
                ("last_eager_seq", ctypes.c_uint16), ("last_completed_seq", ctypes.c_uint16),
                ("last_eager_offset", ctypes.c_uint8), ("has_processed_eager", ctypes.c_uint8),
                ("pad", ctypes.c_uint8 * 2), ("num_inflight_reqs", c_u32), ("eager_pending", c_u32),
                ("pad2", c_u32), ("n_ctrl_sent", c_u64)]


class Point(ctypes.Structure):
    _fields_ = [("x", ctypes.c_double), ("y", ctypes.c_double)]


_ORACLE_PROTOS = {
    "oracle_gin_tx_create": (ctypes.c_void_p, [c_u32, c_u32, c_u32, c_u32, ctypes.POINTER(GinFabricOps)]),
    "oracle_gin_tx_destroy": (None, [ctypes.c_void_p]),
    "oracle_gin_tx_iput_signal": (c_int, [ctypes.c_void_p, c_u32, ctypes.POINTER(GinWire),
                                          ctypes.POINTER(c_i32)]),
    "oracle_gin_tx_iget": (c_int, [ctypes.c_void_p, c_u32, ctypes.POINTER(GinWire), ctypes.POINTER(c_i32)]),
    "oracle_gin_tx_iflush": (c_int, [ctypes.c_void_p, ctypes.c_void_p, c_u64, c_u64, ctypes.POINTER(c_i32)]),
    "oracle_gin_tx_send_ack": (c_int, [ctypes.c_void_p, c_u32, c_u64]),
    "oracle_gin_tx_progress": (c_int, [ctypes.c_void_p]),
    "oracle_gin_tx_test": (c_int, [ctypes.c_void_p, c_i32, ctypes.POINTER(c_int)]),
    "oracle_gin_tx_stats": (None, [ctypes.c_void_p, ctypes.POINTER(GinTxStats)]),
    "oracle_sched_init": (None, [ctypes.POINTER(Sched), c_int, c_u64, c_u64]),
    "oracle_sched_num_stripes": (c_int, [ctypes.POINTER(Sched), c_u64]),
    "oracle_sched_get_schedule": (c_int, [ctypes.POINTER(Sched), c_u64, c_u64, ctypes.POINTER(Xfer)]),
    "oracle_sched_batch": (None, [ctypes.POINTER(Sched), c_vp, c_u64, c_u64, c_vp, c_vp]),
    "oracle_sched_batch_alloc": (None, [ctypes.POINTER(Sched), c_vp, c_u64, c_u64, c_vp, c_vp]),
    "oracle_bounce_scatter": (None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_u32, c_vp]),
    "oracle_mpsc_create": (c_vp, [c_u32, c_u32]),
    "oracle_mpsc_destroy": (None, [c_vp]),
    "oracle_mpsc_push": (c_int, [c_vp, c_vp]),
    "oracle_mpsc_pop": (c_int, [c_vp, c_vp]),
    "oracle_mpsc_set_positions": (None, [c_vp, c_u32]),
    "oracle_mpsc_stress": (c_int, [c_u32, c_u32, c_u32]),
    "oracle_spsc_create": (c_vp, [c_u32, c_u32]),
    "oracle_spsc_destroy": (None, [c_vp]),
    "oracle_spsc_push": (c_int, [c_vp, c_vp]),
    "oracle_spsc_pop": (c_int, [c_vp, c_vp]),
    "oracle_gin_imm": (c_u32, [c_u32, c_u32, c_u32, c_u32]),
    "oracle_gin_meta_header": (c_u64, [c_u32, c_u32, c_u32, c_u32]),
    "oracle_gin_ack_msg": (c_u64, [c_u32, c_u32]),
    "oracle_gin_gen_desc": (None, [c_u64, c_u32, c_u64, c_u32, c_u32, c_u32, c_u32,
                                   ctypes.POINTER(GinDesc)]),
    "oracle_gin_comm_init": (None, [ctypes.POINTER(GinComm), c_u32, c_u32, c_u64, c_u64, c_u32]),
    "oracle_gin_iput_signal": (c_int, [ctypes.POINTER(GinComm), ctypes.POINTER(GinMr),
                                       ctypes.POINTER(GinDesc), ctypes.POINTER(GinWire)]),
    "oracle_gin_iget": (c_int, [ctypes.POINTER(GinComm), ctypes.POINTER(GinMr), ctypes.POINTER(GinDesc),
                                ctypes.POINTER(GinWire)]),
    "oracle_gin_apply_ack": (None, [ctypes.POINTER(GinComm), c_u32]),
    "oracle_gin_rx_create": (c_vp, [c_u32, ctypes.POINTER(c_u32)]),
    "oracle_gin_rx_destroy": (None, [c_vp]),
    "oracle_gin_rx_write": (c_int, [c_vp, c_u32, c_u32]),
    "oracle_gin_rx_metadata": (c_int, [c_vp, c_u32, ctypes.POINTER(c_u64)]),
    "oracle_gin_rx_take_work": (c_u32, [c_vp, ctypes.POINTER(GinSignalWork), c_u32]),
    "oracle_gin_rx_take_acks": (c_u32, [c_vp, ctypes.POINTER(GinAck), c_u32]),
    "oracle_gin_rx_cursors": (None, [c_vp, c_u32, ctypes.POINTER(c_u32), ctypes.POINTER(c_u32)]),
    "oracle_gin_signal_apply": (c_int, [ctypes.POINTER(GinSignalWork), c_u32, ctypes.POINTER(c_u64),
                                        ctypes.POINTER(c_u64), ctypes.POINTER(c_vp), c_u32]),
    "oracle_gin_fold": (c_u64, [c_u64, c_vp, c_int]),
    "oracle_rdma_imm": (c_u32, [c_u32, c_u32, c_u32, c_u32]),
    "oracle_rdma_imm_decode": (None, [c_u32] + [ctypes.POINTER(c_u32)] * 4),
    "oracle_ctrl_mailbox_slot": (c_u32, [ctypes.c_uint16]),
    "oracle_ctrl_msg_fill": (c_int, [ctypes.POINTER(CtrlMsg), ctypes.c_uint16, ctypes.c_uint16,
                                     ctypes.POINTER(c_u64), ctypes.POINTER(c_u32), ctypes.POINTER(c_int),
                                     ctypes.POINTER(c_u64), c_u32, c_int]),
    "oracle_ctrl_msg_ready": (c_int, [ctypes.POINTER(CtrlMsg), ctypes.c_uint16, c_int, c_int]),
    "oracle_ctrl_msg_find_tag": (c_int, [ctypes.POINTER(CtrlMsg), c_int]),
    "oracle_seq_before": (c_int, [ctypes.c_uint16, ctypes.c_uint16]),
    "oracle_eager_seq_before": (c_int, [ctypes.c_uint16, ctypes.c_uint16]),
    "oracle_eager_entry_less": (c_int, [ctypes.POINTER(EagerEntry), ctypes.POINTER(EagerEntry)]),
    "oracle_eager_entry_can_process": (c_int, [c_int, ctypes.c_uint16, ctypes.c_uint8,
                                               ctypes.POINTER(EagerEntry)]),
    "oracle_eager_rxq_create": (c_vp, []),
    "oracle_eager_rxq_destroy": (None, [c_vp]),
    "oracle_eager_rxq_insert": (c_int, [c_vp, ctypes.POINTER(EagerEntry)]),
    "oracle_eager_rxq_drain": (c_u32, [c_vp, ctypes.POINTER(EagerEntry), c_u32]),
    "oracle_eager_rxq_pending": (c_u32, [c_vp]),
    "oracle_eager_rxq_peek": (c_u32, [c_vp, ctypes.POINTER(EagerEntry), c_u32]),
    "oracle_eager_tx_init": (None, [ctypes.POINTER(EagerTx)]),
    "oracle_eager_tx_assign": (None, [ctypes.POINTER(EagerTx), c_i32, ctypes.POINTER(EagerHdr)]),
    "oracle_eager_tx_advance": (None, [ctypes.POINTER(EagerTx)]),
    "oracle_eager_fits": (c_int, [c_u64, ctypes.c_int64]),
    "oracle_flush_post": (None, [c_vp, c_vp, c_u32]),
    "oracle_flush_completed": (c_int, [c_vp, c_u32, c_u64]),
    "oracle_eager_copy_batch": (None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_u32, c_vp]),
    "oracle_gin_stream_checksum": (c_u64, [c_u64, c_u32, c_u64, c_u32, c_u32, c_u32, c_u32, c_int,
                                           c_u32, c_u64, c_u64, c_u32, ctypes.POINTER(GinMr)]),
    "oracle_msgbuff_create": (c_vp, [ctypes.c_uint16, ctypes.c_uint16, ctypes.c_uint16]),
    "oracle_msgbuff_destroy": (None, [c_vp]),
    "oracle_msgbuff_insert": (c_int, [c_vp, ctypes.c_uint16, c_vp, c_int, ctypes.POINTER(c_int)]),
    "oracle_msgbuff_replace": (c_int, [c_vp, ctypes.c_uint16, c_vp, c_int, ctypes.POINTER(c_int)]),
    "oracle_msgbuff_retrieve": (c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(c_vp), ctypes.POINTER(c_int),
                                        ctypes.POINTER(c_int)]),
    "oracle_msgbuff_complete": (c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(c_int)]),
    "oracle_send_comm_create": (c_vp, [c_u32, c_u32, ctypes.c_int64, c_u64, c_u64]),
    "oracle_send_comm_destroy": (None, [c_vp]),
    "oracle_send_comm_mailbox": (ctypes.POINTER(CtrlMsg), [c_vp]),
    "oracle_send_comm_state": (None, [c_vp, ctypes.POINTER(SendState)]),
    "oracle_send_comm_send": (c_int, [c_vp, c_u64, c_i32, ctypes.POINTER(SendAction)]),
    "oracle_send_comm_completion": (c_int, [c_vp, c_i32]),
    "oracle_send_comm_test": (c_int, [c_vp, c_i32, ctypes.POINTER(c_int), ctypes.POINTER(c_u64)]),
    "oracle_recv_comm_create": (c_vp, [c_u32]),
    "oracle_recv_comm_destroy": (None, [c_vp]),
    "oracle_recv_comm_recv": (c_int, [c_vp, c_int, ctypes.POINTER(c_u64), ctypes.POINTER(c_u64),
                                      ctypes.POINTER(c_int), ctypes.POINTER(c_u64), c_int,
                                      ctypes.POINTER(CtrlMsg), ctypes.POINTER(c_i32),
                                      ctypes.POINTER(ctypes.c_uint16)]),
    "oracle_recv_comm_eager_arrival": (c_int, [c_vp, ctypes.c_uint16, ctypes.POINTER(EagerHdr), c_u32, c_u64]),
    "oracle_recv_comm_write_arrival": (c_int, [c_vp, c_u32, c_u64]),
    "oracle_recv_comm_ctrl_sent": (c_int, [c_vp, c_i32]),
    "oracle_recv_comm_take_copies": (c_u32, [c_vp, ctypes.POINTER(EagerCopyItem), c_u32]),
    "oracle_recv_comm_copy_done": (c_int, [c_vp, c_i32, c_i32]),
    "oracle_recv_comm_test": (c_int, [c_vp, c_i32, ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "oracle_recv_comm_state": (None, [c_vp, ctypes.POINTER(RecvState)]),
    "oracle_recv_comm_flush": (c_int, [c_vp, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_i32)]),
    "oracle_recv_comm_flush_test": (c_int, [c_vp, c_i32, c_vp, c_u32, c_u64, ctypes.POINTER(c_int)]),
    "oracle_gin_cpu_rings_run": (c_int, [c_u64, c_u32, c_u64, c_u32, c_u32, c_u32, c_u32, c_u32, c_u32,
                                         ctypes.POINTER(c_u64), ctypes.POINTER(ctypes.c_double)]),
    "oracle_model_cost": (ctypes.c_float, [c_int, c_int, c_int, c_int, c_int, c_u64, c_u64, c_u64,
                                           c_int, c_int]),
    "oracle_model_decide": (None, [c_int, c_int, c_int, c_u64, c_u64, c_u64, c_int, c_int,
                                   ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "oracle_region_extend": (Point, [Point, Point, Point]),
    "oracle_region_log2": (Point, [Point]),
    "oracle_region_inside": (c_int, [Point, ctypes.POINTER(Point), ctypes.c_size_t]),
    "oracle_region_decide": (None, [c_int, c_int, c_u64, c_u64, c_u64, ctypes.POINTER(c_int),
                                    ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "oracle_region_polys": (c_int, [c_int, c_u64, c_u64, c_int, ctypes.POINTER(c_int),
                                    ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                                    ctypes.POINTER(Point), c_int]),
    "oracle_region_chunk_size": (c_int, [c_int, c_int, c_u64, c_int, c_int, c_u64, c_u64,
                                         ctypes.POINTER(c_u64)]),
    "oracle_chunk_tree_ll128": (c_u64, [c_u64, c_int, c_int]),
    "oracle_best_nchannel_tree": (c_int, [c_u64, c_int]),
    "oracle_best_nchannel_pat": (c_int, [c_u64, c_u64]),
    "oracle_model_decide_v2": (None, [c_int, c_int, c_int, c_u64, c_u64, c_u64, c_int, c_int, c_int,
                                      ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "oracle_region_decide_masked": (None, [c_int, c_int, c_u64, c_u64, c_u64, c_u32,
                                           ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                                           ctypes.POINTER(c_int)]),
    "oracle_model_grid": (None, [c_int, c_int, c_int, c_int, c_vp, c_u32, c_vp, c_u32, c_vp, c_u32,
                                 c_vp, c_u32, c_vp, c_u32, c_vp, c_vp]),
    "oracle_region_grid": (None, [c_int, c_vp, c_u32, c_vp, c_u32, c_vp, c_u32, c_vp, c_u32, c_vp]),
}

_REF_PROTOS = {
    "ref_mpsc_create": (c_vp, [c_int]),
    "ref_mpsc_destroy": (None, [c_int, c_vp]),
    "ref_mpsc_push": (c_int, [c_int, c_vp, c_vp]),
    "ref_mpsc_pop": (c_int, [c_int, c_vp, c_vp]),
    "ref_spsc_create": (c_vp, []),
    "ref_spsc_destroy": (None, [c_vp]),
    "ref_spsc_push": (c_int, [c_vp, c_u64]),
    "ref_spsc_pop": (c_int, [c_vp, ctypes.POINTER(c_u64)]),
    "ref_gin_imm": (c_u32, [c_u32, c_u32, c_u32, c_u32]),
    "ref_gin_imm_decode": (None, [c_u32] + [ctypes.POINTER(c_u32)] * 4),
    "ref_gin_meta": (None, [c_u32, c_u32, c_u32, c_u32, c_u64, c_u64, c_u64, c_vp]),
    "ref_gin_ack": (c_u64, [c_u32, c_u32]),
    "ref_gin_const": (c_u64, [c_int]),
    "ref_div_ceil": (c_u64, [c_u64, c_u64]),
    "ref_round_up": (c_u64, [c_u64, c_u64]),
    "ref_round_down": (c_u64, [c_u64, c_u64]),
}

_oracle = None
_ref = None


def _bind(lib, protos):
    for name, (res, args) in protos.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def load_oracle():
    global _oracle
    if _oracle is None:
        path = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", ORACLE_DIR], check=True, stdout=subprocess.DEVNULL)
        _oracle = _bind(ctypes.CDLL(path), _ORACLE_PROTOS)
    return _oracle


def load_ref():
    global _ref
    if _ref is None:
        path = os.path.join(ORACLE_DIR, "_ref", "libref.so")
        if not os.path.exists(path):
            return None
        _ref = _bind(ctypes.CDLL(path), _REF_PROTOS)
    return _ref


def ptr(a):
    """numpy array -> void*"""
    return a.ctypes.data_as(c_vp)


def sched_batch(oracle, sizes, num_rails=4, min_stripe=131072, max_small=64, seeds=(0, 0), align=128):
    """Run the oracle scheduler over `sizes`; returns (num_xfers[n], xfers[n,4,3] as u64 words, state)."""
    st = Sched(seeds[0], seeds[1], max_small, min_stripe, num_rails, 0)
    n = len(sizes)
    num = np.zeros(n, dtype=np.uint32)
    xf = np.zeros((n, 4, 3), dtype=np.uint64)
    oracle.oracle_sched_batch(ctypes.byref(st), ptr(sizes), n, align, ptr(num), ptr(xf))
    return num, xf, st


def default_mrs(cls=GinMr):
    """Three registrations (source, destination, signal) with fixed addresses and keys."""
    mrs = (cls * 3)()
    for i in range(3):
        mrs[i].local_base = 0x7F0000000000 + (i << 32)
        mrs[i].remote_address = 0x7E0000000000 + (i << 32)
        mrs[i].remote_address_offset = (0x7E0000000000 + (i << 32)) if i != 1 else 0
        for r in range(4):
            mrs[i].key[r] = 0x1000 * (i + 1) + r
    return mrs

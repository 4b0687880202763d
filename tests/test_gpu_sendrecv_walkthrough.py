"""The send/receive protocol walked through with the library's own pieces, in protocol order,
on one GPU: no transport is claimed -- the test plays the wire -- but every step that the
reference performs around a message is done by the entry point that would do it in the
plugin.

  eager message   sender: eligibility + batch numbering (ofi_amd_eager_fits, _eager_tx_assign),
                  header + payload into a receiver rx buffer; receiver: arrival in any order
                  -> ordered queue (_eager_rxq_insert / _drain) -> batched copy into the posted
                  receive buffers (ofi_amd_eager_copy_batch), truncating to the buffer size
  rendezvous      receiver: control message into the sender's mailbox (_ctrl_msg_fill);
                  sender: mailbox poll (_ctrl_msg_ready, _find_tag), rail schedule
                  (ofi_amd_sched_get_schedule), one RDMA write per stripe executed as a device
                  copy (ofi_amd_copy_table) with the write's immediate data (ofi_amd_rdma_imm);
                  receiver: segment counting from the decoded immediate data

Reference: nccl_net_ofi_rdma_send_comm::send, src/nccl_ofi_rdma.cpp:5646-5860; recv :3545 with
allocate_recv_req :3398-3474 (mailbox update); handle_eager_recv :897-940; the receive side's
segment counting on write completions, handle_write_comp :1102-1150.
Sizes follow the configured sweep: powers of two from 8 B up (64 MiB here), 64 in flight."""
import ctypes

import numpy as np
import pytest
import torch

import _gpu
import aws_ofi_nccl_amd as m

pytestmark = pytest.mark.gpu

RX_STRIDE = 8320
EAGER_SEND_SIZE = 8192
COMM_ID = 77


def test_sixty_four_messages_in_flight_arrive_bit_exact(lib, gpu):
    rng = np.random.default_rng(64)
    sizes = [8 << k for k in range(0, 24)]                     # 8 B .. 64 MiB
    sizes = (sizes * 3)[:64]
    rng.shuffle(sizes)
    n = len(sizes)
    tags = [int(t) for t in rng.integers(1, 1000, n)]
    payload = [rng.integers(0, 256, s, dtype=np.uint8) for s in sizes]
    # every sixth receive buffer is smaller than the message: eager copies truncate to it
    recv_len = [s // 2 if (i % 6 == 5 and s <= EAGER_SEND_SIZE - 8) else s for i, s in enumerate(sizes)]

    d_send = [_gpu.to_dev(p) for p in payload]                 # sender's registered buffers
    d_recv = [torch.full((max(r, 1) + 32,), 0xAB, dtype=torch.uint8, device="cuda") for r in recv_len]
    recv_ptr = [t.data_ptr() + 3 for t in d_recv]              # receive buffers at odd addresses

    # ---- receiver posts all 64 receives: one control message each into the sender's mailbox ----
    mailbox = (m.CtrlMsg * 256)()
    for i in range(n):
        seq = 1 + i                                            # sequence numbers start at 1
        offs = (ctypes.c_uint64 * 1)(recv_ptr[i])
        lens = (ctypes.c_uint32 * 1)(recv_len[i])
        tg = (ctypes.c_int * 1)(tags[i])
        keys = (ctypes.c_uint64 * 4)(*[0xA000 + i * 4 + r for r in range(4)])
        assert lib.ofi_amd_ctrl_msg_fill(mailbox, seq, 1, offs, lens, tg, keys, 4, 0) == 0

    # ---- sender: eager for what fits, rendezvous for the rest ----
    tx = m.EagerTx()
    lib.ofi_amd_eager_tx_init(ctypes.byref(tx))
    sched = m.SchedState(0, 0, 64, 131072, 4, 0)
    rx_pool = np.zeros(n * RX_STRIDE, dtype=np.uint8)          # receiver's posted rx buffers
    eager_arrivals = []                                        # (entry, rx slot)
    copy_src, copy_dst, copy_len = [], [], []
    write_completions = []                                     # immediate data of every RDMA write
    expected_segments = {}
    for i in range(n):
        seq = 1 + i
        if lib.ofi_amd_eager_fits(sizes[i], EAGER_SEND_SIZE):
            hdr = m.EagerHdr()
            lib.ofi_amd_eager_tx_assign(ctypes.byref(tx), tags[i], ctypes.byref(hdr))
            slot = len(eager_arrivals)
            rx_pool[slot * RX_STRIDE:slot * RX_STRIDE + 8] = np.frombuffer(bytes(hdr), dtype=np.uint8)
            rx_pool[slot * RX_STRIDE + 8:slot * RX_STRIDE + 8 + sizes[i]] = payload[i]
            eager_arrivals.append((m.EagerEntry(hdr.eager_offset, hdr.prev_batch_count, hdr.eager_seq,
                                                seq, 0, hdr.tag, sizes[i], slot), i))
            if rng.random() < 0.4:                             # the message sequence moves on: batch closed
                lib.ofi_amd_eager_tx_advance(ctypes.byref(tx))
            continue
        lib.ofi_amd_eager_tx_advance(ctypes.byref(tx))
        # rendezvous: the control message must be there and carry our tag
        assert lib.ofi_amd_ctrl_msg_ready(mailbox, seq, tags[i], 0) == 1
        ctrl = mailbox[lib.ofi_amd_ctrl_mailbox_slot(seq)]
        k = lib.ofi_amd_ctrl_msg_find_tag(ctypes.byref(ctrl), tags[i])
        assert k == 0 and ctrl.entries[k].buff_len >= sizes[i]
        xfers = (m.XferInfo * 4)()
        nseg = lib.ofi_amd_sched_get_schedule(ctypes.byref(sched), sizes[i], 128, xfers)
        assert nseg in (1, 2, 4) and sum(xfers[s].msg_size for s in range(nseg)) == sizes[i]
        expected_segments[seq] = nseg
        for s in range(nseg):
            assert ctrl.entries[k].mr_key[xfers[s].rail_id] == 0xA000 + i * 4 + xfers[s].rail_id
            copy_src.append(d_send[i].data_ptr() + xfers[s].offset)
            copy_dst.append(ctrl.entries[k].buff_offset + xfers[s].offset)
            copy_len.append(xfers[s].msg_size)
            write_completions.append(lib.ofi_amd_rdma_imm(COMM_ID, seq & 0x3FF, ctrl.entries[k].recv_idx, nseg))
    assert len(eager_arrivals) >= 20 and len(copy_src) >= 40

    # ---- the wire: rendezvous writes as device copies, pieces of at most 1 MiB per wavefront ----
    pieces = [(s + o, d + o, min(1 << 20, l - o)) for s, d, l in zip(copy_src, copy_dst, copy_len)
              for o in range(0, l, 1 << 20)]
    a_src = _gpu.to_dev(np.array([p[0] for p in pieces], dtype=np.uint64))
    a_dst = _gpu.to_dev(np.array([p[1] for p in pieces], dtype=np.uint64))
    a_len = _gpu.to_dev(np.array([p[2] for p in pieces], dtype=np.uint32))
    assert lib.ofi_amd_copy_table(a_src.data_ptr(), a_dst.data_ptr(), a_len.data_ptr(), len(pieces),
                                  _gpu.stream()) == 0

    # ---- receiver: write completions arrive in any order; a message is done at its segment count ----
    got_segments = {}
    order = rng.permutation(len(write_completions))
    comm, seq_, ridx, nseg_ = (ctypes.c_uint32() for _ in range(4))
    for j in order:
        lib.ofi_amd_rdma_imm_decode(write_completions[j], ctypes.byref(comm), ctypes.byref(seq_),
                                    ctypes.byref(ridx), ctypes.byref(nseg_))
        assert comm.value == COMM_ID and ridx.value == 0
        got_segments[seq_.value] = got_segments.get(seq_.value, 0) + 1
        assert got_segments[seq_.value] <= nseg_.value == expected_segments[seq_.value]
    assert got_segments == expected_segments

    # ---- receiver: eager arrivals in any order -> chain order -> one batched copy ----
    q = ctypes.c_void_p()
    assert lib.ofi_amd_eager_rxq_create(ctypes.byref(q)) == 0
    ready = []
    buf = (m.EagerEntry * 64)()
    for j in rng.permutation(len(eager_arrivals)):
        assert lib.ofi_amd_eager_rxq_insert(q, ctypes.byref(eager_arrivals[j][0])) == 0
        k = lib.ofi_amd_eager_rxq_drain(q, buf, 64)
        ready += [(buf[x].cookie, buf[x].msg_seq_num, buf[x].tag, buf[x].recv_len) for x in range(k)]
    assert lib.ofi_amd_eager_rxq_pending(q) == 0 and lib.ofi_amd_eager_rxq_destroy(q) == 0
    assert [r[1] for r in ready] == [e[0].msg_seq_num for e in eager_arrivals]     # send order restored
    msg_of_slot = {e[0].cookie: e[1] for e in eager_arrivals}
    for slot, seq, tag, _l in ready:                           # matches the receive posted for that sequence
        assert tags[msg_of_slot[slot]] == tag and msg_of_slot[slot] == seq - 1
    d_pool = _gpu.to_dev(rx_pool)
    rx_off = _gpu.to_dev(np.array([r[0] * RX_STRIDE for r in ready], dtype=np.uint64))
    e_len = _gpu.to_dev(np.array([r[3] for r in ready], dtype=np.uint32))
    e_dst = _gpu.to_dev(np.array([recv_ptr[msg_of_slot[r[0]]] for r in ready], dtype=np.uint64))
    e_cap = _gpu.to_dev(np.array([recv_len[msg_of_slot[r[0]]] for r in ready], dtype=np.uint32))
    d_copied = torch.zeros(len(ready), dtype=torch.int32, device="cuda")
    assert lib.ofi_amd_eager_copy_batch(d_pool.data_ptr(), rx_off.data_ptr(), e_len.data_ptr(), None,
                                        e_dst.data_ptr(), e_cap.data_ptr(), len(ready), d_copied.data_ptr(),
                                        None, _gpu.stream()) == 0
    _gpu.sync()

    # ---- what the application sees ----
    copied = _gpu.to_host(d_copied, np.uint32)
    for (slot, _s, _t, _l), c in zip(ready, copied):
        i = msg_of_slot[slot]
        assert c == min(sizes[i], recv_len[i])
    for i in range(n):
        got = d_recv[i].cpu().numpy()
        k = min(sizes[i], recv_len[i])
        assert np.array_equal(got[3:3 + k], payload[i][:k]), (i, sizes[i])
        assert np.all(got[:3] == 0xAB) and np.all(got[3 + k:] == 0xAB)             # nothing beyond the buffer

"""The sending end of the net entry points (ofi_amd_net_send_comm_create) over a fabric played by this
test, on the CPU: what isend posts, what it does when the fabric says -EAGAIN, and how completions
finish a request.  The fabric is three callbacks (include/ofi_amd_net_abi.h); behind the reference's
send() they are fi_senddata / fi_writedata and the completion queue.

Worked by hand from the reference: an eager send is one post of header + payload with the sequence
number in its immediate data (post_eager, src/nccl_ofi_rdma.cpp:2368-2427); a rendezvous send is one
write per stripe of the schedule, each to the control message's address plus the stripe's offset under
that rail's key, each with the same immediate data (rdma_send_req::post, :2429-2496); a refused post is
queued and retried in order by the next progress, and while posts wait isend answers "call again"
(post_with_pending_retry :1375-1387, process_cq_if_pending :3523-3545)."""
import ctypes
import errno

import aws_ofi_nccl_amd as m

ncclSuccess, ncclInternalError = 0, 3
EAGER, WRITE = 1, 2
POSTED = 1
CTX_SEND = 1 << 28
vp = ctypes.c_void_p


class Fabric:
    """Records posts; refuses them while `refuse` is positive; hands back the completions queued in `cq`."""

    def __init__(self):
        self.posts, self.cq, self.refuse, self.cq_reads = [], [], 0, 0

        def post(end, p):
            if self.refuse > 0:
                self.refuse -= 1
                return -errno.EAGAIN
            q = p.contents
            self.posts.append((q.kind, q.rail, q.context, q.imm, q.src, q.len, q.dest, q.key, bytes(q.hdr)))
            return 0

        def cq_read(end, out, cap):
            self.cq_reads += 1
            n = 0
            while self.cq and n < cap:
                out[n].kind, out[n].context = POSTED, self.cq.pop(0)
                n += 1
            return n

        self.ops = m.NetFabricOps(m.NET_POST_FN(post), m.NET_CQ_READ_FN(cq_read), m.NET_REPOST_RX_FN(lambda e, c: 0), None)


def make(lib, fabric, rails=4, eager=8192):
    comm = vp()
    assert lib.ofi_amd_net_send_comm_create(rails, eager, 0, 0, ctypes.byref(fabric.ops), ctypes.byref(comm)) == 0
    return comm


def isend(lib, comm, addr, size, tag):
    req = vp(1)
    assert lib.ofi_amd_net_isend(comm, vp(addr), size, tag, None, None, ctypes.byref(req)) == ncclSuccess
    return req if req.value else None


def poll(lib, req):
    done, size = ctypes.c_int(-1), (ctypes.c_int * 1)(-1)
    assert lib.ofi_amd_net_test(req, ctypes.byref(done), size) == ncclSuccess
    return done.value, size[0]


def post_receive(lib, comm, seq, bufs, sizes, tags, keys_per_recv):
    """What the peer's irecv makes arrive in this end's mailbox: the control message of sequence number seq."""
    mailbox = ctypes.cast(vp(lib.ofi_amd_net_send_comm_mailbox(comm)), ctypes.POINTER(m.CtrlMsg))
    n = len(bufs)
    keys = (ctypes.c_uint64 * (4 * n))(*[k for ks in keys_per_recv for k in ks])
    assert lib.ofi_amd_ctrl_msg_fill(mailbox, seq, n, (ctypes.c_uint64 * n)(*bufs), (ctypes.c_uint32 * n)(*sizes),
                                     (ctypes.c_int * n)(*tags), keys, 4, 0) == 0


def test_an_eager_send_is_one_post_and_completes_with_its_control_message(lib):
    fab = Fabric()
    comm = make(lib, fab)
    req = isend(lib, comm, 0x10000, 1000, 7)
    assert req is not None and len(fab.posts) == 1
    kind, rail, context, imm, src, length, dest, key, hdr = fab.posts[0]
    assert (kind, src, length) == (EAGER, 0x10000, 1000) and rail < 4 and context & ~0xFFFFFFF == CTX_SEND
    # header: eager_offset 0, prev_batch_count 0, eager_seq 0, tag 7 (nccl_ofi_eager_msg_header_t)
    assert hdr == bytes([0, 0, 0, 0]) + (7).to_bytes(4, "little")
    # immediate data: comm id 1, sequence number 1 (the first message), receive 0, one segment
    assert imm == lib.ofi_amd_rdma_imm(1, 1, 0, 1)
    assert poll(lib, req) == (0, -1)
    fab.cq.append(context)                              # the send's own completion
    assert poll(lib, req) == (0, -1)                    # ... is not enough: the match is still to come
    post_receive(lib, comm, 1, [0x900000], [4096], [7], [[11, 12, 13, 14]])
    assert poll(lib, req) == (1, 1000)
    assert lib.ofi_amd_net_test(req, ctypes.byref(ctypes.c_int()), None) == ncclInternalError     # freed
    assert lib.ofi_amd_net_comm_destroy(comm) == 0


def test_a_rendezvous_send_is_one_write_per_stripe(lib):
    fab = Fabric()
    comm = make(lib, fab)
    size = 1 << 20
    assert isend(lib, comm, 0x4000000, size, 3) is None and not fab.posts       # too large for eager, no receive yet
    assert fab.cq_reads == 1                                                    # "call again" after a look at the fabric
    post_receive(lib, comm, 1, [0x90000000], [size], [3], [[0xA0, 0xA1, 0xA2, 0xA3]])
    req = isend(lib, comm, 0x4000000, size, 3)
    assert req is not None and len(fab.posts) == 4
    imm = lib.ofi_amd_rdma_imm(1, 1, 0, 4)
    offset, rails = 0, set()
    for kind, rail, context, got_imm, src, length, dest, key, _hdr in fab.posts:
        assert kind == WRITE and got_imm == imm and key == 0xA0 + rail
        assert src == 0x4000000 + offset and dest == 0x90000000 + offset and length == size // 4
        offset += length
        rails.add(rail)
    assert offset == size and rails == {0, 1, 2, 3}
    for k in range(4):
        assert poll(lib, req)[0] == 0
        fab.cq.append(fab.posts[k][2])
    assert poll(lib, req) == (1, size)
    # a receive buffer smaller than the message cuts it (update_send_data_from_remote, :574-640)
    fab.posts.clear()
    post_receive(lib, comm, 2, [0x91000000], [5000], [3], [[1, 2, 3, 4]])
    req = isend(lib, comm, 0x4000000, 300000, 3)
    assert [(p[0], p[5]) for p in fab.posts] == [(WRITE, 5000)]
    fab.cq.append(fab.posts[0][2])
    assert poll(lib, req) == (1, 5000)
    assert lib.ofi_amd_net_comm_destroy(comm) == 0


def test_refused_posts_wait_in_order_and_isend_says_call_again_meanwhile(lib):
    fab = Fabric()
    comm = make(lib, fab)
    size = 1 << 20
    post_receive(lib, comm, 1, [0x90000000], [size], [3], [[0xA0, 0xA1, 0xA2, 0xA3]])
    post_receive(lib, comm, 2, [0x98000000], [64 << 10], [3], [[0xB0, 0xB1, 0xB2, 0xB3]])
    fab.refuse = 1
    r1 = isend(lib, comm, 0x4000000, size, 3)
    assert r1 is not None and len(fab.posts) == 0        # the first write was refused: all four wait, in order
    fab.refuse = 10
    assert isend(lib, comm, 0x5000000, 64 << 10, 3) is None and len(fab.posts) == 0      # network busy
    fab.refuse = 0
    r2 = isend(lib, comm, 0x5000000, 64 << 10, 3)        # progress first: the four go, then this one
    assert r2 is not None
    assert [(p[0], p[4] - 0x4000000) for p in fab.posts[:4]] == [(WRITE, k * (size // 4)) for k in range(4)]
    assert [(p[0], p[4], p[5], p[6]) for p in fab.posts[4:]] == [(WRITE, 0x5000000, 64 << 10, 0x98000000)]
    for p in fab.posts:
        fab.cq.append(p[2])
    assert poll(lib, r2) == (1, 64 << 10) and poll(lib, r1) == (1, size)
    # anything but -EAGAIN from the fabric is the call's error: -EIO -> ncclSystemError
    post_receive(lib, comm, 3, [0x98000000], [8], [3], [[1, 2, 3, 4]])
    fab.ops.post = m.NET_POST_FN(lambda e, p: -errno.EIO)
    bad = make(lib, fab)
    post_receive(lib, bad, 1, [0x98000000], [1 << 20], [3], [[1, 2, 3, 4]])
    req = vp(1)
    assert lib.ofi_amd_net_isend(bad, vp(0x1000), 1 << 20, 3, None, None, ctypes.byref(req)) == 2 and req.value is None
    assert lib.ofi_amd_net_comm_destroy(bad) == 0 and lib.ofi_amd_net_comm_destroy(comm) == 0


def test_arguments(lib):
    fab = Fabric()
    comm = vp()
    for rails, eager in ((0, 8192), (5, 8192), (4, 8193)):
        assert lib.ofi_amd_net_send_comm_create(rails, eager, 0, 0, ctypes.byref(fab.ops), ctypes.byref(comm)) == -errno.EINVAL
    assert lib.ofi_amd_net_send_comm_create(4, 8192, 0, 0, None, ctypes.byref(comm)) == -errno.EINVAL
    assert lib.ofi_amd_net_comm_destroy(None) == -errno.EINVAL
    assert lib.ofi_amd_net_send_comm_mailbox(None) is None
    comm = make(lib, fab, eager=-1)                         # no eager protocol: a small message waits for its receive
    assert isend(lib, comm, 0x1000, 8, 1) is None and not fab.posts
    assert lib.ofi_amd_net_comm_destroy(comm) == 0

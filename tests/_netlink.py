"""The two ends of an in-process net link (ofi_amd_net_link_create) behind small Python wrappers of the
net entry points, for the GPU tests: one call each, results as Python values."""
import ctypes

import _gpu
import aws_ofi_nccl_amd as m

ncclSuccess = 0
TAG = 1
vp = ctypes.c_void_p


class Link:
    def __init__(self, lib, rails=4, eager=8192, rx_buffers=0):
        self.lib = lib
        self.h = vp()
        rc = lib.ofi_amd_net_link_create(rails, eager, 0, 0, rx_buffers, _gpu.stream(), ctypes.byref(self.h))
        assert rc == 0, rc
        self.s = vp(lib.ofi_amd_net_link_send_comm(self.h))
        self.r = vp(lib.ofi_amd_net_link_recv_comm(self.h))
        self.mh = vp(0x1000)     # a registration handle: opaque to the data path

    def isend(self, tensor, size, tag=TAG, offset=0):
        """One call: the request, or None for "call again"."""
        req = vp()
        rc = self.lib.ofi_amd_net_isend(self.s, vp(tensor.data_ptr() + offset), size, tag, self.mh, None,
                                        ctypes.byref(req))
        assert rc == ncclSuccess, rc
        return req if req.value else None

    def irecv(self, tensors, sizes, tags=None, offset=0):
        n = len(tensors)
        data = (vp * n)(*[t.data_ptr() + offset for t in tensors])
        a_sizes = (ctypes.c_size_t * n)(*sizes)
        a_tags = (ctypes.c_int * n)(*(tags or [TAG] * n))
        mhs = (vp * n)(*[self.mh.value] * n)
        req = vp()
        rc = self.lib.ofi_amd_net_irecv(self.r, n, data, a_sizes, a_tags, mhs, None, ctypes.byref(req))
        assert rc == ncclSuccess and req.value, rc
        return req

    def test(self, req, n=1):
        done = ctypes.c_int(0)
        sizes = (ctypes.c_int * 8)(*[-1] * 8)
        rc = self.lib.ofi_amd_net_test(req, ctypes.byref(done), sizes)
        assert rc == ncclSuccess, rc
        return bool(done.value), list(sizes)[:n]

    def flush(self, tensors, sizes):
        """iflush and poll, as poll_and_validate does after each completed receive."""
        n = len(tensors)
        data = (vp * n)(*[t.data_ptr() for t in tensors])
        a_sizes = (ctypes.c_int * n)(*sizes)
        mhs = (vp * n)(*[self.mh.value] * n)
        req = vp()
        assert self.lib.ofi_amd_net_iflush(self.r, n, data, a_sizes, mhs, ctypes.byref(req)) == ncclSuccess
        if not req.value:
            return False
        for _ in range(1_000_000):
            done, _ = self.test(req)
            if done:
                return True
        raise AssertionError("flush never completed")

    def stats(self):
        st = m.NetLinkStats()
        assert self.lib.ofi_amd_net_link_stats(self.h, ctypes.byref(st)) == 0
        return st

    def close(self):
        assert self.lib.ofi_amd_net_link_destroy(self.h) == 0

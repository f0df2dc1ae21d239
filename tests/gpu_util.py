"""Helpers for the GPU parity tests: numpy in/out around the C-ABI calls."""
import numpy as np
import torch


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def stream_ptr():
    return torch.cuda.current_stream().cuda_stream


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def assert_bits_equal(a, b, what=""):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    ua = a.view(np.uint32) if a.dtype == np.float32 else a
    ub = b.view(np.uint32) if b.dtype == np.float32 else b
    if not np.array_equal(ua, ub):
        bad = np.flatnonzero(ua != ub)
        raise AssertionError(f"{what}: {bad.size} of {ua.size} differ, first at {bad[:5]}: "
                             f"{a.ravel()[bad[:5]]} vs {b.ravel()[bad[:5]]}")


class Tbq:
    def __init__(self, capi):
        self.c = capi
        self.L = capi.load()

    def encode(self, gs, rs, thrs, outs=None):
        """gs, rs: lists of cuda float tensors (rs updated in place). Returns list of packed cuda tensors."""
        c = self.c
        if outs is None:
            outs = [torch.full(((g.numel() + 3) // 4,), 0xAA, dtype=torch.uint8, device="cuda") for g in gs]
        rc = self.L.hpx_tbq_encode(len(gs), c.ptr_array([g.data_ptr() for g in gs]), c.i32_array([g.numel() for g in gs]),
                                   c.ptr_array([r.data_ptr() for r in rs]), c.ptr_array([o.data_ptr() for o in outs]),
                                   c.f32_array(thrs), stream_ptr())
        assert rc == 0, c.last_error()
        return outs

    def decode(self, packed, outs, thrs, adds):
        c = self.c
        rc = self.L.hpx_tbq_decode(len(outs), c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                   c.ptr_array([p.data_ptr() for p in packed]), c.f32_array(thrs), c.i32_array(adds), stream_ptr())
        assert rc == 0, c.last_error()
        return outs


class Terngrad:
    def __init__(self, capi):
        self.c = capi
        self.L = capi.load()

    @staticmethod
    def packed_size(n, b):
        dpb = 8 // b
        return 10 + (n + dpb - 1) // dpb

    def encode(self, xs, bits_, randoms, seeds, outs=None, expect_rc=0):
        c = self.c
        if outs is None:
            outs = [torch.zeros(self.packed_size(x.numel(), b), dtype=torch.uint8, device="cuda") for x, b in zip(xs, bits_)]
        rc = self.L.hpx_terngrad_encode(len(xs), c.ptr_array([x.data_ptr() for x in xs]), c.i32_array([x.numel() for x in xs]),
                                        c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                        c.u8_array(bits_), c.i32_array(randoms),
                                        c.u64_array(seeds) if seeds is not None else None, stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())
        return outs

    def decode(self, packed, outs, adds, in_sizes=None):
        c = self.c
        if in_sizes is None:
            in_sizes = [p.numel() for p in packed]
        rc = self.L.hpx_terngrad_decode(len(outs), c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                        c.ptr_array([p.data_ptr() for p in packed]), c.i32_array(in_sizes), c.i32_array(adds), stream_ptr())
        assert rc == 0, c.last_error()
        return outs

    def status(self):
        return self.L.hpx_terngrad_decode_status(stream_ptr())

    def encode_status(self):
        return self.L.hpx_terngrad_encode_status(stream_ptr())

    def repaired(self):
        return self.L.hpx_terngrad_repaired(stream_ptr())

    def encode_noalloc(self, xs, bits_, randoms, seeds, outs=None, expect_rc=0):
        c = self.c
        if outs is None:
            outs = [torch.zeros(self.packed_size(x.numel(), b), dtype=torch.uint8, device="cuda") for x, b in zip(xs, bits_)]
        rc = self.L.hpx_terngrad_encode_noalloc(len(xs), c.ptr_array([x.data_ptr() for x in xs]), c.i32_array([x.numel() for x in xs]),
                                                c.ptr_array([o.data_ptr() for o in outs]), c.i32_array([o.numel() for o in outs]),
                                                c.u8_array(bits_), c.i32_array(randoms),
                                                c.u64_array(seeds) if seeds is not None else None, stream_ptr())
        assert rc == expect_rc, (rc, c.last_error())
        return outs

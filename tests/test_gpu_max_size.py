"""GPU parity at the largest tensors the reference's int32 sizes allow (N = 2^31 - 1 elements, or the
largest N whose message size still fits an int32).

At this size the CPU oracle is only run on windows of the tensor (TBQ, TernGrad: both are element-wise
once the per-tensor scalars are fixed, so a window encodes to the same bytes as it does inside the
whole tensor) or once on the whole tensor (GradDrop); everything else is checked through properties
that do not depend on the size, computed on the device in chunks.
"""
import numpy as np
import pytest
import torch

from gpu_util import Tbq, Terngrad, assert_bits_equal, host, stream_ptr

pytestmark = pytest.mark.gpu

N_MAX = 2**31 - 1
WIN = 1 << 20
CHUNK = 1 << 27


def _windows(n):
    """(start, end) pairs: the head, a stretch across the 2^30 element mark and the ragged end; starts are multiples of 16."""
    mid = (1 << 30) - WIN // 2
    return [(0, WIN), (mid, mid + WIN), ((n - WIN) & ~15, n)]


def _need_memory(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2**30:
        pytest.skip(f"needs {gib} GiB of free device memory")


def test_tbq_two_to_31_minus_1(capi, oracle_cpu):
    _need_memory(48)
    tbq = Tbq(capi)
    n, thr = N_MAX, 1e-2                       # n % 4 == 3: the last byte holds three codes and one pad field
    gen = torch.Generator(device="cuda").manual_seed(11)
    g = torch.randn(n, device="cuda", generator=gen) * 5e-3
    r0 = torch.randn(n, device="cuda", generator=gen) * 2e-3
    r = r0.clone()
    packed = tbq.encode([g], [r], [thr])[0]
    assert packed.numel() == 2**29
    out = torch.empty(n, device="cuda")
    tbq.decode([packed], [out], [thr], [0])
    torch.cuda.synchronize()
    for s, e in _windows(n):
        gh, rh = host(g[s:e]), host(r0[s:e])
        p_ref = oracle_cpu.tbq_encode(gh, rh, thr)
        assert_bits_equal(host(packed[s // 4:(e + 3) // 4]), p_ref, f"packed, window {s}")
        assert_bits_equal(host(r[s:e]), rh, f"residual, window {s}")
        assert_bits_equal(host(out[s:e]), oracle_cpu.tbq_decode(p_ref, e - s, thr), f"decoded, window {s}")
    assert int(packed[-1]) >> 6 == 1           # pad field of the last byte stays 01 (tbq_body.h:114-155)
    # size-independent: decode takes the values {-thr, 0, thr}; decode + new residual == old residual + gradient
    t = torch.tensor(thr, dtype=torch.float32, device="cuda")
    for c0 in range(0, n, CHUNK):
        sl = slice(c0, min(n, c0 + CHUNK))
        o = out[sl]
        assert bool(((o == 0) | (o == t) | (o == -t)).all())
        err = (o.double() + r[sl].double()) - (r0[sl].double() + g[sl].double())
        assert float(err.abs().max()) < 4e-9
        del o, err


@pytest.mark.parametrize("bits,rnd,n", [(2, 1, N_MAX), (8, 0, N_MAX - 10)])
def test_terngrad_largest_tensor(capi, oracle_cpu, bits, rnd, n):
    # (8, 0, 2^31 - 11): the message is 10 + n = 2^31 - 1 bytes, the largest an int32 size can name
    _need_memory(40)
    tg = Terngrad(capi)
    dpb = 8 // bits
    seed = 0xFFFFFFF0                          # seed + byte index wraps past 2^32 inside the tensor
    gen = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn(n, device="cuda", generator=gen) * 1e-2
    wins = _windows(n)
    for s, _ in wins:                          # the tensor's extremes sit in every window: a window then
        x[s] = -1.0                            # quantises with the scalars of the whole tensor
        x[s + 1] = 1.0
    msg = tg.encode([x], [bits], [rnd], [seed])[0]
    assert msg.numel() == 10 + (n + dpb - 1) // dpb
    out = torch.empty(n, device="cuda")
    tg.decode([msg], [out], [0])
    torch.cuda.synchronize()
    assert tg.status() == 0
    head = host(msg[:10])
    assert head[0] == bits and head[1] == (-n) % dpb
    assert head[2:6].view(np.float32)[0] == -1.0 and head[6:10].view(np.float32)[0] == 1.0
    for s, e in wins:
        rc, ref = oracle_cpu.terngrad_encode(host(x[s:e]), bits, rnd, seed + s // dpb)
        assert rc == 0
        assert_bits_equal(host(msg[10 + s // dpb:10 + (e + dpb - 1) // dpb]), ref[10:], f"payload, window {s}")
        rc, dec = oracle_cpu.terngrad_decode(ref, e - s)
        assert rc == 0
        assert_bits_equal(host(out[s:e]), dec, f"decoded, window {s}")
    # size-independent: a decoded value is within one level (half a level without random rounding) of its input
    gap = 2.0 / ((1 << bits) - 1)
    bound = gap * (1.0 if rnd else 0.5) * (1 + 2e-3) + 1e-6   # the quantiser scales by 1 / (gap + 1e-8)
    for c0 in range(0, n, CHUNK):
        sl = slice(c0, min(n, c0 + CHUNK))
        assert float((out[sl] - x[sl]).abs().max()) <= bound


def test_graddrop_two_to_31_minus_1(capi, oracle_cpu):
    _need_memory(40)
    c, L = capi, capi.load()
    n, sr, dr, seed = N_MAX, 0.01, 0.999, 2**32 - 5
    gen = torch.Generator(device="cuda").manual_seed(13)
    u = torch.rand(n, device="cuda", generator=gen) - 0.5
    g = -1e-3 * torch.sign(u) * torch.log1p(-2 * u.abs())
    del u
    r = torch.randn(n, device="cuda", generator=gen) * 1e-4
    gh, rh = host(g), host(r)
    sample_cnt, expected, thr_index = oracle_cpu.gd_sizes(n, sr, dr)
    out = torch.zeros(4 + 8 * expected, dtype=torch.uint8, device="cuda")
    rc = L.hpx_gd_encode(1, c.ptr_array([g.data_ptr()]), c.i32_array([n]), c.ptr_array([r.data_ptr()]),
                         c.ptr_array([out.data_ptr()]), c.f64_array([sr]), c.f64_array([dr]), c.u64_array([seed]), stream_ptr())
    assert rc == 0, c.last_error()
    torch.cuda.synchronize()
    msg, info = oracle_cpu.gd_encode(gh, rh, sr, dr, seed)
    got = host(out)
    assert int(got[:4].view(np.int32)[0]) == msg.size, info
    assert_bits_equal(got[:msg.size], msg, f"message {info}")
    idx, val = oracle_cpu.gd_split(msg)
    assert idx.size > 0 and int(idx.max()) > 2**30          # indices beyond 2^30 are in play
    # the residual after the encode, compared in chunks on the device
    rd = torch.from_numpy(rh)
    for c0 in range(0, n, CHUNK):
        sl = slice(c0, min(n, c0 + CHUNK))
        assert torch.equal(r[sl].view(torch.int32), rd[sl].cuda().view(torch.int32)), f"residual chunk {c0}"
    # decode(add) into the residual restores R + G at the selected positions
    rc = L.hpx_gd_decode(1, c.ptr_array([out.data_ptr()]), c.i32_array([msg.size]), c.ptr_array([r.data_ptr()]),
                         c.i32_array([n]), c.i32_array([1]), stream_ptr())
    assert rc == 0, c.last_error()
    torch.cuda.synchronize()
    pos = torch.from_numpy(idx.astype(np.int64)).cuda()
    assert_bits_equal(host(r[pos]), val, "decode(add) puts the values back")

"""Host-side mirror of the reference's kernel-driver layer.

The nine functions below carry the names, argument order and argument meaning
of the `hp_cuda_*` free functions the reference declares in hp_cuda.cpp:18-102
and defines in hp_cuda_kernel.cu; each forwards to the C-ABI entry point of
libhpx.so that replaces it.  Where the reference takes std::vector<float*> a
list of CUDA-device torch tensors (or raw device addresses) is taken, and the
trailing `stream` is a torch.cuda.Stream, a raw hipStream_t address, or None
for the current stream.

Like the reference drivers they report a body failure by printing and carry on
(hp_cuda_kernel.cu:63, :90-92, :115-117, :153-155); unlike them they also
return the code.  `seeds` is an addition: the reference draws its RNG seed from
the wall clock inside the body and cannot be seeded from outside.
"""
import torch

from . import _capi


def _addr(t):
    return t.data_ptr() if isinstance(t, torch.Tensor) else int(t)


def _stream(stream):
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def _check_cuda(ts, what):
    # CHECK_CUDA_INPUT, hp_cuda.cpp:107-111
    for t in ts:
        if isinstance(t, torch.Tensor):
            if not t.is_cuda:
                raise RuntimeError(f"{what} must be a CUDA tensor")
            if not t.is_contiguous():
                raise RuntimeError(f"{what} must be contiguous")


def _report(rc, what):
    if rc:
        print(f"Call {what} failed, ret = {rc}. {_capi.last_error()}", flush=True)
    return rc


def _sync(stream):
    s = _stream(stream)
    torch.cuda.ExternalStream(s).synchronize() if s else torch.cuda.default_stream().synchronize()


def hp_cuda_tbq(to_compress_floats, to_compress_float_sizes, residual_floats, residual_float_sizes,
                out_uint8_ts, out_uint8_t_sizes, thresholds, stream=None):
    """hp_cuda_kernel.cu:120-158; waits for the stream like the reference (:157)."""
    _check_cuda(to_compress_floats, "tensor"); _check_cuda(residual_floats, "residual"); _check_cuda(out_uint8_ts, "B")
    L = _capi.load()
    n = len(to_compress_floats)
    rc = L.hpx_tbq_encode(n, _capi.ptr_array([_addr(t) for t in to_compress_floats]),
                          _capi.i32_array(to_compress_float_sizes),
                          _capi.ptr_array([_addr(t) for t in residual_floats]),
                          _capi.ptr_array([_addr(t) for t in out_uint8_ts]),
                          _capi.f32_array(thresholds), _stream(stream))
    _sync(stream)
    return _report(rc, "tbq_body")


def hp_cuda_tbqr(out_floats, out_float_sizes, in_uint8_ts, in_uint8_t_sizes, thresholds, is_add_tos, stream=None):
    """hp_cuda_kernel.cu:161-198; waits for the stream like the reference (:197)."""
    _check_cuda(out_floats, "tensor"); _check_cuda(in_uint8_ts, "B")
    L = _capi.load()
    n = len(out_floats)
    rc = L.hpx_tbq_decode(n, _capi.ptr_array([_addr(t) for t in out_floats]), _capi.i32_array(out_float_sizes),
                          _capi.ptr_array([_addr(t) for t in in_uint8_ts]), _capi.f32_array(thresholds),
                          _capi.i32_array(is_add_tos), _stream(stream))
    _sync(stream)
    return _report(rc, "tbq_r_body")


def hp_cuda_terngrad(in_floats, in_float_sizes, out_uint8_ts, out_uint8_t_sizes, bitwidths, enable_randoms,
                     stream=None, seeds=None):
    """hp_cuda_kernel.cu:30-65."""
    _check_cuda(in_floats, "tensor"); _check_cuda(out_uint8_ts, "B")
    L = _capi.load()
    n = len(in_floats)
    rc = L.hpx_terngrad_encode(n, _capi.ptr_array([_addr(t) for t in in_floats]), _capi.i32_array(in_float_sizes),
                               _capi.ptr_array([_addr(t) for t in out_uint8_ts]), _capi.i32_array(out_uint8_t_sizes),
                               _capi.u8_array(bitwidths), _capi.i32_array(enable_randoms),
                               _capi.u64_array(seeds) if seeds is not None else None, _stream(stream))
    return _report(rc, "terngrad_body")


def hp_cuda_terngradr(out_floats, out_float_sizes, in_uint8_ts, in_uint8_t_sizes, is_add_tos, stream=None):
    """hp_cuda_kernel.cu:200-230."""
    _check_cuda(out_floats, "tensor"); _check_cuda(in_uint8_ts, "B")
    L = _capi.load()
    n = len(out_floats)
    rc = L.hpx_terngrad_decode(n, _capi.ptr_array([_addr(t) for t in out_floats]), _capi.i32_array(out_float_sizes),
                               _capi.ptr_array([_addr(t) for t in in_uint8_ts]), _capi.i32_array(in_uint8_t_sizes),
                               _capi.i32_array(is_add_tos), _stream(stream))
    return _report(rc, "terngrad_r_body")


def hp_cuda_gd(in_floats, Ns, residuals, residual_sizes, out_uint8_ts, sample_rates, drop_ratios,
               stream=None, seeds=None):
    """hp_cuda_kernel.cu:67-94."""
    _check_cuda(in_floats, "tensor"); _check_cuda(residuals, "residual"); _check_cuda(out_uint8_ts, "B")
    L = _capi.load()
    n = len(in_floats)
    rc = L.hpx_gd_encode(n, _capi.ptr_array([_addr(t) for t in in_floats]), _capi.i32_array(Ns),
                         _capi.ptr_array([_addr(t) for t in residuals]),
                         _capi.ptr_array([_addr(t) for t in out_uint8_ts]), _capi.f64_array(sample_rates),
                         _capi.f64_array(drop_ratios), _capi.u64_array(seeds) if seeds is not None else None,
                         _stream(stream))
    return _report(rc, "gd_body")


def hp_cuda_gdr(in_uint8_ts, in_uint8_t_sizes, out_floats, out_float_sizes, is_add_tos, stream=None):
    """hp_cuda_kernel.cu:96-118."""
    _check_cuda(in_uint8_ts, "B"); _check_cuda(out_floats, "tensor")
    L = _capi.load()
    n = len(in_uint8_ts)
    rc = L.hpx_gd_decode(n, _capi.ptr_array([_addr(t) for t in in_uint8_ts]), _capi.i32_array(in_uint8_t_sizes),
                         _capi.ptr_array([_addr(t) for t in out_floats]), _capi.i32_array(out_float_sizes),
                         _capi.i32_array(is_add_tos), _stream(stream))
    return _report(rc, "gdr_body")


def _dims(Ms, Qs):
    ns, ms, rs = [], [], []
    for M, Q in zip(Ms, Qs):
        if M.dim() != 2 or Q.dim() != 2 or Q.shape[0] != M.shape[1]:
            raise RuntimeError("M must be n x m and Q m x r")
        ns.append(M.shape[0]); ms.append(M.shape[1]); rs.append(Q.shape[1])
    return ns, ms, rs


def hp_cuda_powersgd_encode1(grads, residuals, Qs, Ms, Ps, stream=None):
    """hp_cuda_kernel.cu:232-255: M[:N] = grad + residual, P = M Q."""
    for ts, w in ((grads, "tensor"), (residuals, "residual"), (Qs, "Q"), (Ms, "M"), (Ps, "P")):
        _check_cuda(ts, w)
    L = _capi.load()
    ns, ms, rs = _dims(Ms, Qs)
    rc = L.hpx_powersgd_encode1(len(grads), _capi.ptr_array([_addr(t) for t in grads]),
                                _capi.i64_array([g.numel() for g in grads]),
                                _capi.ptr_array([_addr(t) for t in residuals]),
                                _capi.ptr_array([_addr(t) for t in Qs]), _capi.ptr_array([_addr(t) for t in Ms]),
                                _capi.ptr_array([_addr(t) for t in Ps]), _capi.i32_array(ns), _capi.i32_array(ms),
                                _capi.i32_array(rs), _stream(stream))
    return _report(rc, "powersgd encode1")


def hp_cuda_powersgd_encode2(Ps, Ms, Qs, stream=None):
    """hp_cuda_kernel.cu:257-276: P = orth(P), Q = M^T P."""
    for ts, w in ((Ps, "P"), (Ms, "M"), (Qs, "Q")):
        _check_cuda(ts, w)
    L = _capi.load()
    ns, ms, rs = _dims(Ms, Qs)
    rc = L.hpx_powersgd_encode2(len(Ps), _capi.ptr_array([_addr(t) for t in Ps]),
                                _capi.ptr_array([_addr(t) for t in Ms]), _capi.ptr_array([_addr(t) for t in Qs]),
                                _capi.i32_array(ns), _capi.i32_array(ms), _capi.i32_array(rs), _stream(stream))
    return _report(rc, "powersgd encode2")


def hp_cuda_powersgd_decode(Ps, Qs, Ms, residuals, grads, stream=None):
    """hp_cuda_kernel.cu:278-301: M = P Q^T, residual = grad - M[:N], grad = M[:N]."""
    for ts, w in ((Ps, "P"), (Qs, "Q"), (Ms, "M"), (residuals, "residual"), (grads, "tensor")):
        _check_cuda(ts, w)
    L = _capi.load()
    ns, ms, rs = _dims(Ms, Qs)
    rc = L.hpx_powersgd_decode(len(Ps), _capi.ptr_array([_addr(t) for t in Ps]),
                               _capi.ptr_array([_addr(t) for t in Qs]), _capi.ptr_array([_addr(t) for t in Ms]),
                               _capi.ptr_array([_addr(t) for t in residuals]),
                               _capi.ptr_array([_addr(t) for t in grads]),
                               _capi.i64_array([g.numel() for g in grads]), _capi.i32_array(ns),
                               _capi.i32_array(ms), _capi.i32_array(rs), _stream(stream))
    return _report(rc, "powersgd decode")

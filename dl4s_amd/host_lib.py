"""ctypes binding of libdl4s_host.so: whole layers of the C++ host layer (include/dl4s_host.h), driven with
numpy arrays.  No CPU fallback: a missing library or a failing call raises."""
import ctypes as C
import os

import numpy as np

from . import lib as _hip

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libdl4s_host.so")
_f = C.POINTER(C.c_float)
_i64 = C.c_int64


class MhaParams(C.Structure):
    _fields_ = [(n, _f) for n in ("qDense", "kDense", "vDense", "fc", "norm_scale", "norm_shift")]


class FfnParams(C.Structure):
    _fields_ = [(n, _f) for n in ("w1", "b1", "w2", "b2", "norm_scale", "norm_shift")]


_lib = None


def load():
    global _lib
    if _lib is None:
        _hip.load()
        if not os.path.exists(HOST_LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m dl4s_amd.build`" % HOST_LIB_PATH)
        _lib = C.CDLL(HOST_LIB_PATH)
        _lib.dl4s_host_last_error.restype = C.c_char_p
    return _lib


class HostError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise HostError(load().dl4s_host_last_error().decode())


def _a(x):
    return np.ascontiguousarray(x, np.float32)


def _p(x):
    return x.ctypes.data_as(_f) if x is not None else None


def _mask(mask):
    if mask is None:
        return None, None, 0, None
    m = _a(mask)
    return _p(m), (_i64 * max(1, m.ndim))(*m.shape), m.ndim, m


def _mha(p, keep):
    st = MhaParams()
    for dst, src in (("qDense", "Wq"), ("kDense", "Wk"), ("vDense", "Wv"), ("fc", "Wo"), ("norm_scale", "ln_scale"),
                     ("norm_shift", "ln_shift")):
        a = _a(p[src])
        keep.append(a)
        setattr(st, dst, _p(a))
    return st


def _ffn(p, keep):
    st = FfnParams()
    for dst, src in (("w1", "W1"), ("b1", "b1"), ("w2", "W2"), ("b2", "b2"), ("norm_scale", "ln_scale"), ("norm_shift", "ln_shift")):
        a = _a(p[src])
        keep.append(a)
        setattr(st, dst, _p(a))
    return st


def _timing(iters):
    ms = C.c_float()
    return (C.byref(ms) if iters else None), ms


def sdpa(ctx, q, k, v, mask=None, temperature=None, fused=True, iters=0):
    q, k, v = _a(q), _a(k), _a(v)
    B, H, Lq, dk = q.shape
    Lk, dv = v.shape[2], v.shape[3]
    if temperature is None:
        temperature = float(np.sqrt(np.float32(dk)))
    out = np.empty((B, H, Lq, dv), np.float32)
    mp, ms, md, keep = _mask(mask)
    tp, t = _timing(iters)
    _check(load().dl4s_host_sdpa(ctx.handle, int(fused), _p(q), _p(k), _p(v), mp, ms, md, _i64(B), _i64(H), _i64(Lq), _i64(Lk),
                                 _i64(dk), _i64(dv), C.c_float(temperature), _p(out), max(1, iters), tp))
    return (out, t.value) if iters else out


def mha(ctx, q, k, v, mask, params, heads, dk, dv, fused=True, iters=0):
    q = _a(q)
    k = q if k is q else _a(k)
    v = q if v is q else (k if v is k else _a(v))
    B, Lq, D = q.shape
    Lk = k.shape[1]
    keep = []
    st = _mha(params, keep)
    out = np.empty((B, Lq, D), np.float32)
    mp, ms, md, mk = _mask(mask)
    tp, t = _timing(iters)
    _check(load().dl4s_host_mha(ctx.handle, int(fused), _p(q), _p(k), _p(v), mp, ms, md, _i64(B), _i64(Lq), _i64(Lk), _i64(D),
                                _i64(heads), _i64(dk), _i64(dv), C.byref(st), _p(out), max(1, iters), tp))
    return (out, t.value) if iters else out


def encoder_block(ctx, x, mask, attn, ffn, heads, dk, dv, fused=True, iters=0):
    x = _a(x)
    B, L, D = x.shape
    F = np.asarray(ffn["W1"]).shape[1]
    keep = []
    a, f = _mha(attn, keep), _ffn(ffn, keep)
    out = np.empty_like(x)
    mp, ms, md, mk = _mask(mask)
    tp, t = _timing(iters)
    _check(load().dl4s_host_encoder_block(ctx.handle, int(fused), _p(x), mp, ms, md, _i64(B), _i64(L), _i64(D), _i64(heads),
                                          _i64(dk), _i64(dv), _i64(F), C.byref(a), C.byref(f), _p(out), max(1, iters), tp))
    return (out, t.value) if iters else out


def decoder_block(ctx, dec, enc, enc_mask, dec_mask, self_attn, enc_attn, ffn, heads, dk, dv, fused=True, iters=0):
    dec, enc = _a(dec), _a(enc)
    B, Ld, D = dec.shape
    Le = enc.shape[1]
    F = np.asarray(ffn["W1"]).shape[1]
    keep = []
    sa, ea, f = _mha(self_attn, keep), _mha(enc_attn, keep), _ffn(ffn, keep)
    out = np.empty_like(dec)
    ep, es, ed, ek = _mask(enc_mask)
    dp, ds, dd, dk_ = _mask(dec_mask)
    tp, t = _timing(iters)
    _check(load().dl4s_host_decoder_block(ctx.handle, int(fused), _p(dec), _p(enc), ep, es, ed, dp, ds, dd, _i64(B), _i64(Ld),
                                          _i64(Le), _i64(D), _i64(heads), _i64(dk), _i64(dv), _i64(F), C.byref(sa), C.byref(ea),
                                          C.byref(f), _p(out), max(1, iters), tp))
    return (out, t.value) if iters else out


def _masks(fn, ctx, lengths):
    lens = np.ascontiguousarray(lengths, np.int64)
    L = _i64()
    lp = lens.ctypes.data_as(C.POINTER(_i64))
    _check(fn(ctx.handle, lp, _i64(len(lens)), None, C.byref(L)))
    return lens, lp, L.value


def make_encoder_masks(ctx, lengths):
    fn = load().dl4s_host_make_encoder_masks
    lens, lp, L = _masks(fn, ctx, lengths)
    out = np.empty((len(lens), 1, 1, L), np.float32)
    _check(fn(ctx.handle, lp, _i64(len(lens)), _p(out), None))
    return out


def make_decoder_masks(ctx, lengths):
    fn = load().dl4s_host_make_decoder_masks
    lens, lp, L = _masks(fn, ctx, lengths)
    out = np.empty((len(lens), 1, L, L), np.float32)
    _check(fn(ctx.handle, lp, _i64(len(lens)), _p(out), None))
    return out

"""ctypes binding of the CPU oracle (libdl4s_oracle.so).  TEST INFRASTRUCTURE.

Only tests, the smoke check and the benchmark's cpu_baseline leg import this module;
the GPU library and its Python host layer never do.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdl4s_oracle.so")

_f = C.POINTER(C.c_float)
_i64 = C.POINTER(C.c_int64)
_i32 = C.POINTER(C.c_int32)


class MhaParams(C.Structure):
    _fields_ = [(n, _f) for n in ("Wq", "Wk", "Wv", "Wo", "ln_scale", "ln_shift")]


class FfnParams(C.Structure):
    _fields_ = [(n, _f) for n in ("W1", "b1", "W2", "b2", "ln_scale", "ln_shift")]


def build():
    """Compile the oracle with gcc (idempotent)."""
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a):
    return a.ctypes.data_as(_f) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _shape(a):
    arr = (C.c_int64 * max(1, len(a)))(*a)
    return arr


def gemm(a, b, trans_a=False, trans_b=False, alpha=1.0, beta=0.0, c=None):
    a, b = _f32(a), _f32(b)
    M = a.shape[1] if trans_a else a.shape[0]
    K = a.shape[0] if trans_a else a.shape[1]
    N = b.shape[0] if trans_b else b.shape[1]
    assert K == (b.shape[1] if trans_b else b.shape[0])
    out = np.zeros((M, N), np.float32) if c is None else _f32(c).copy()
    lib().orc_gemm(int(trans_a), int(trans_b), C.c_int64(M), C.c_int64(N), C.c_int64(K),
                   C.c_float(alpha), _p(a), _p(b), C.c_float(beta), _p(out))
    return out


def bmm(a, b, trans_a=False, trans_b=False):
    a, b = _f32(a), _f32(b)
    dim = max(a.ndim, b.ndim)
    a = a.reshape((1,) * (dim - a.ndim) + a.shape)
    b = b.reshape((1,) * (dim - b.ndim) + b.shape)
    M = a.shape[-1] if trans_a else a.shape[-2]
    N = b.shape[-2] if trans_b else b.shape[-1]
    bs = tuple(max(x, y) for x, y in zip(a.shape[:-2], b.shape[:-2]))
    out = np.empty(bs + (M, N), np.float32)
    rc = lib().orc_bmm(_p(a), _shape(a.shape), _p(b), _shape(b.shape), dim, int(trans_a), int(trans_b), _p(out))
    if rc:
        raise ValueError("orc_bmm: shape error")
    return out


_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def broadcast(op, a, b):
    a, b = _f32(a), _f32(b)
    dim = max(a.ndim, b.ndim)
    oshape = (C.c_int64 * max(dim, 1))()
    out = np.empty(np.broadcast_shapes(a.shape, b.shape), np.float32)
    rc = lib().orc_broadcast(_OPS[op], _p(a), _shape(a.shape), a.ndim, _p(b), _shape(b.shape), b.ndim,
                             _p(out), oshape)
    if rc:
        raise ValueError("orc_broadcast: shape error")
    assert tuple(oshape[:dim]) == out.shape
    return out


def reduce_sum(x, axes):
    x = _f32(x)
    axes = sorted(int(a) for a in axes)
    oshape = tuple(s for i, s in enumerate(x.shape) if i not in axes)
    out = np.empty(oshape, np.float32)
    ax = (C.c_int * max(1, len(axes)))(*axes)
    rc = lib().orc_reduce_sum_axes(_p(x), _shape(x.shape), x.ndim, ax, len(axes), _p(out))
    if rc:
        raise ValueError("orc_reduce_sum_axes")
    return out


def reduce_max(x, axis):
    x = _f32(x)
    oshape = tuple(s for i, s in enumerate(x.shape) if i != axis)
    out = np.empty(oshape, np.float32)
    rc = lib().orc_reduce_max_axis(_p(x), _shape(x.shape), x.ndim, int(axis), _p(out))
    if rc:
        raise ValueError("orc_reduce_max_axis")
    return out


def _unary(name, x):
    x = _f32(x)
    out = np.empty_like(x)
    getattr(lib(), name)(_p(x), _p(out), C.c_int64(x.size))
    return out


def exp(x):
    return _unary("orc_exp", x)


def tanh(x):
    return _unary("orc_tanh", x)


def sqrt(x):
    return _unary("orc_sqrt", x)


def relu(x):
    return _unary("orc_relu", x)


def gelu(x):
    return _unary("orc_gelu", x)


def log(x):
    return _unary("orc_log", x)


def sin(x):
    return _unary("orc_sin", x)


def cos(x):
    return _unary("orc_cos", x)


def argmax(x):
    x = _f32(x).reshape(-1)
    v = C.c_float()
    f = lib().orc_argmax
    f.restype = C.c_int64
    i = f(_p(x), C.c_int64(x.size), C.byref(v))
    return int(i), float(v.value)


def embedding(table, tokens, ignore_index=-1):
    table = _f32(table)
    tok = np.ascontiguousarray(tokens, np.int32).reshape(-1)
    out = np.empty((tok.size, table.shape[1]), np.float32)
    rc = lib().orc_embedding(_p(table), C.c_int64(table.shape[0]), C.c_int64(table.shape[1]),
                             tok.ctypes.data_as(C.c_void_p), C.c_int64(tok.size), C.c_int32(ignore_index), _p(out))
    if rc:
        raise ValueError("orc_embedding: token out of range")
    return out


def permute(x, arrangement):
    x = _f32(x)
    dshape = [0] * x.ndim
    for i, a in enumerate(arrangement):
        dshape[a] = x.shape[i]
    out = np.empty(dshape, np.float32)
    arr = (C.c_int * x.ndim)(*arrangement)
    rc = lib().orc_permute(_p(x), _shape(x.shape), x.ndim, arr, _p(out), None)
    if rc:
        raise ValueError("orc_permute")
    return out


def band(x, below, above):
    x = _f32(x)
    out = np.empty_like(x)
    lib().orc_band(_p(x), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), int(below is not None),
                   C.c_int64(below or 0), int(above is not None), C.c_int64(above or 0), _p(out))
    return out


def make_encoder_masks(lens):
    lens = np.ascontiguousarray(lens, np.int32)
    fn = lib().orc_make_encoder_masks
    fn.restype = C.c_int64
    L = fn(lens.ctypes.data_as(_i32), C.c_int64(len(lens)), None)
    out = np.empty((len(lens), 1, 1, L), np.float32)
    fn(lens.ctypes.data_as(_i32), C.c_int64(len(lens)), _p(out))
    return out


def make_decoder_masks(lens):
    lens = np.ascontiguousarray(lens, np.int32)
    fn = lib().orc_make_decoder_masks
    fn.restype = C.c_int64
    L = fn(lens.ctypes.data_as(_i32), C.c_int64(len(lens)), None)
    out = np.empty((len(lens), 1, L, L), np.float32)
    fn(lens.ctypes.data_as(_i32), C.c_int64(len(lens)), _p(out))
    return out


def softmax_last(x):
    x = _f32(x)
    out = np.empty_like(x)
    n = x.shape[-1]
    lib().orc_softmax_last(_p(x), C.c_int64(x.size // max(n, 1)), C.c_int64(n), _p(out))
    return out


def _mask_args(mask):
    if mask is None:
        return None, None, 0, None
    m = _f32(mask)
    return _p(m), _shape(m.shape), m.ndim, m


def sdpa(q, k, v, mask=None, temperature=None):
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, Lq, dk = q.shape
    Lk, dv = v.shape[2], v.shape[3]
    assert k.shape == (B, H, Lk, dk) and v.shape[:2] == (B, H)
    if temperature is None:
        temperature = float(np.sqrt(np.float32(dk)))
    out = np.empty((B, H, Lq, dv), np.float32)
    mp, ms, md, keep = _mask_args(mask)
    rc = lib().orc_sdpa(_p(q), _p(k), _p(v), mp, ms, md, C.c_int64(B), C.c_int64(H), C.c_int64(Lq),
                        C.c_int64(Lk), C.c_int64(dk), C.c_int64(dv), C.c_float(temperature), _p(out))
    if rc:
        raise ValueError("orc_sdpa rc=%d" % rc)
    return out


def sdpa_backward(q, k, v, mask, dout, temperature=None):
    """(dq, dk, dv) for the upstream gradient dout of sdpa(q, k, v, mask)."""
    q, k, v, dout = _f32(q), _f32(k), _f32(v), _f32(dout)
    B, H, Lq, dk = q.shape
    Lk, dv = v.shape[2], v.shape[3]
    assert dout.shape == (B, H, Lq, dv)
    if temperature is None:
        temperature = float(np.sqrt(np.float32(dk)))
    dq, dkey, dval = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    mp, ms, md, keep = _mask_args(mask)
    rc = lib().orc_sdpa_backward(_p(q), _p(k), _p(v), mp, ms, md, C.c_int64(B), C.c_int64(H), C.c_int64(Lq), C.c_int64(Lk),
                                 C.c_int64(dk), C.c_int64(dv), C.c_float(temperature), _p(dout), _p(dq), _p(dkey), _p(dval))
    if rc:
        raise ValueError("orc_sdpa_backward rc=%d" % rc)
    return dq, dkey, dval


def sdpa_decode(q, kcache, vcache, T, temperature=None):
    q, kcache, vcache = _f32(q), _f32(kcache), _f32(vcache)
    B, H, Tcap, d = kcache.shape
    if temperature is None:
        temperature = float(np.sqrt(np.float32(d)))
    out = np.empty((B, H, 1, d), np.float32)
    rc = lib().orc_sdpa_decode(_p(q), _p(kcache), _p(vcache), C.c_int64(B), C.c_int64(H), C.c_int64(T),
                               C.c_int64(Tcap), C.c_int64(d), C.c_float(temperature), _p(out))
    if rc:
        raise ValueError("orc_sdpa_decode rc=%d" % rc)
    return out


def layernorm(x, scale, shift):
    """x: [B, ...]; scale/shift: [D] with D the last axis; normalises over all non-batch axes."""
    x, scale, shift = _f32(x), _f32(scale), _f32(shift)
    B, D = x.shape[0], x.shape[-1]
    rows = x.size // (B * D)
    out = np.empty_like(x)
    lib().orc_layernorm(_p(x), C.c_int64(B), C.c_int64(rows), C.c_int64(D), _p(scale), _p(shift), _p(out))
    return out


def _mha_params(p, keep):
    st = MhaParams()
    for n in ("Wq", "Wk", "Wv", "Wo", "ln_scale", "ln_shift"):
        a = _f32(p[n])
        keep.append(a)
        setattr(st, n, _p(a))
    return st


def _ffn_params(p, keep):
    st = FfnParams()
    for n in ("W1", "b1", "W2", "b2", "ln_scale", "ln_shift"):
        a = _f32(p[n])
        keep.append(a)
        setattr(st, n, _p(a))
    return st


def mha(q, k, v, mask, params, heads, dk, dv, return_attn=False):
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, Lq, D = q.shape
    Lk = k.shape[1]
    keep = []
    st = _mha_params(params, keep)
    out = np.empty((B, Lq, D), np.float32)
    attn = np.empty((B, heads, Lq, dv), np.float32) if return_attn else None
    mp, ms, md, mk = _mask_args(mask)
    rc = lib().orc_mha(_p(q), _p(k), _p(v), mp, ms, md, C.c_int64(B), C.c_int64(Lq), C.c_int64(Lk),
                       C.c_int64(D), C.c_int64(heads), C.c_int64(dk), C.c_int64(dv), st.Wq, st.Wk, st.Wv,
                       st.Wo, st.ln_scale, st.ln_shift, _p(out), _p(attn))
    if rc:
        raise ValueError("orc_mha rc=%d" % rc)
    return (out, attn) if return_attn else out


def ffn(x, params):
    x = _f32(x)
    D = x.shape[-1]
    F = np.asarray(params["W1"]).shape[1]
    keep = []
    st = _ffn_params(params, keep)
    out = np.empty_like(x)
    rc = lib().orc_ffn(_p(x), C.c_int64(x.size // D), C.c_int64(D), C.c_int64(F), st.W1, st.b1, st.W2,
                       st.b2, st.ln_scale, st.ln_shift, _p(out))
    if rc:
        raise ValueError("orc_ffn rc=%d" % rc)
    return out


def encoder_block(x, mask, attn_params, ffn_params, heads, dk, dv):
    x = _f32(x)
    B, L, D = x.shape
    F = np.asarray(ffn_params["W1"]).shape[1]
    keep = []
    a = _mha_params(attn_params, keep)
    f = _ffn_params(ffn_params, keep)
    out = np.empty_like(x)
    mp, ms, md, mk = _mask_args(mask)
    rc = lib().orc_encoder_block(_p(x), mp, ms, md, C.c_int64(B), C.c_int64(L), C.c_int64(D),
                                 C.c_int64(heads), C.c_int64(dk), C.c_int64(dv), C.c_int64(F),
                                 C.byref(a), C.byref(f), _p(out))
    if rc:
        raise ValueError("orc_encoder_block rc=%d" % rc)
    return out


def decoder_block(dec, enc, dec_mask, enc_mask, self_params, cross_params, ffn_params, heads, dk, dv):
    dec, enc = _f32(dec), _f32(enc)
    B, Ld, D = dec.shape
    Le = enc.shape[1]
    F = np.asarray(ffn_params["W1"]).shape[1]
    keep = []
    sa = _mha_params(self_params, keep)
    ca = _mha_params(cross_params, keep)
    f = _ffn_params(ffn_params, keep)
    out = np.empty_like(dec)
    dp, ds, dd, dk_ = _mask_args(dec_mask)
    ep, es, ed, ek_ = _mask_args(enc_mask)
    rc = lib().orc_decoder_block(_p(dec), _p(enc), dp, ds, dd, ep, es, ed, C.c_int64(B), C.c_int64(Ld),
                                 C.c_int64(Le), C.c_int64(D), C.c_int64(heads), C.c_int64(dk),
                                 C.c_int64(dv), C.c_int64(F), C.byref(sa), C.byref(ca), C.byref(f), _p(out))
    if rc:
        raise ValueError("orc_decoder_block rc=%d" % rc)
    return out

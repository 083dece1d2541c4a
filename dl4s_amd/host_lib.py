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


class TransformerConfig(C.Structure):
    _fields_ = [(n, _i64) for n in ("encoder_layers", "decoder_layers", "vocab_size", "hidden_dim", "heads", "key_dim",
                                    "value_dim", "forward_dim")]


class TransformerParams(C.Structure):
    _fields_ = [("embedding", _f), ("output_bias", _f), ("encoder_attention", C.POINTER(MhaParams)),
                ("encoder_ffn", C.POINTER(FfnParams)), ("decoder_self_attention", C.POINTER(MhaParams)),
                ("decoder_encoder_attention", C.POINTER(MhaParams)), ("decoder_ffn", C.POINTER(FfnParams))]


class Transformer:
    """Transformer (NN/Models/Transformer/Transformer.swift) with its weights resident on the device.  `params` is the
    dictionary oracle.transformer documents."""

    def __init__(self, ctx, params):
        self.ctx = ctx
        E = _a(params["embedding"])
        ne, nd = len(params["encoder"]), len(params["decoder"])
        first = (params["encoder"][0]["ffn"] if ne else params["decoder"][0]["ffn"])
        self.vocab = E.shape[0]
        cfg = TransformerConfig(ne, nd, E.shape[0], E.shape[1], params["heads"], params["dk"], params["dv"],
                                np.asarray(first["W1"]).shape[1])
        keep = [E, _a(params["output_bias"])]
        st = TransformerParams()
        st.embedding, st.output_bias = _p(keep[0]), _p(keep[1])
        ea = (MhaParams * max(1, ne))(*[_mha(l["attn"], keep) for l in params["encoder"]])
        ef = (FfnParams * max(1, ne))(*[_ffn(l["ffn"], keep) for l in params["encoder"]])
        ds = (MhaParams * max(1, nd))(*[_mha(l["self"], keep) for l in params["decoder"]])
        dc = (MhaParams * max(1, nd))(*[_mha(l["cross"], keep) for l in params["decoder"]])
        df = (FfnParams * max(1, nd))(*[_ffn(l["ffn"], keep) for l in params["decoder"]])
        st.encoder_attention, st.encoder_ffn = ea, ef
        st.decoder_self_attention, st.decoder_encoder_attention, st.decoder_ffn = ds, dc, df
        self.handle = C.c_void_p()
        _check(load().dl4s_host_transformer_create(ctx.handle, C.byref(cfg), C.byref(st), C.byref(self.handle)))

    def close(self):
        if self.handle:
            load().dl4s_host_transformer_destroy(self.handle)
            self.handle = None

    def forward(self, enc_tokens, dec_tokens, enc_lengths, dec_lengths, fused=True, iters=0):
        enc = np.ascontiguousarray(enc_tokens, np.int32)
        dec = np.ascontiguousarray(dec_tokens, np.int32)
        el, dl = np.ascontiguousarray(enc_lengths, np.int64), np.ascontiguousarray(dec_lengths, np.int64)
        B = enc.shape[0]
        out = np.empty((B, dec.shape[1], self.vocab), np.float32)
        tp, t = _timing(iters)
        i32, i64p = C.POINTER(C.c_int32), C.POINTER(_i64)
        _check(load().dl4s_host_transformer_forward(self.ctx.handle, int(fused), self.handle, enc.ctypes.data_as(i32),
                                                    _i64(enc.shape[1]), dec.ctypes.data_as(i32), _i64(dec.shape[1]),
                                                    el.ctypes.data_as(i64p), dl.ctypes.data_as(i64p), _i64(B), _p(out),
                                                    max(1, iters), tp))
        return (out, t.value) if iters else out

    def set_norm_per_token(self, per_token):
        """Every attention layer normalises per token (True) or over (length, hidden) jointly like the reference (False)."""
        _check(load().dl4s_host_transformer_set_norm_per_token(self.handle, int(bool(per_token))))

    def greedy(self, input_sequence, start_token, end_token, max_length, fused=True, return_logits=False, timing=False, cached=False):
        """cached=True: key / value caches, one new position per step (models set to normalise per token only), the step
        recorded into a HIP graph and replayed; cached="stepwise": the same calls issued one by one."""
        src = np.ascontiguousarray(input_sequence, np.int32)
        toks = np.empty(max(1, max_length), np.int32)
        n = _i64()
        logits = np.empty((max(1, max_length), self.vocab), np.float32) if return_logits else None
        ms = C.c_float()
        head = (self.ctx.handle, int(fused), self.handle, src.ctypes.data_as(C.POINTER(C.c_int32)), _i64(len(src)),
                C.c_int32(start_token), C.c_int32(end_token), _i64(max_length))
        tail = (toks.ctypes.data_as(C.POINTER(C.c_int32)), C.byref(n), _p(logits), C.byref(ms))
        if cached:
            _check(load().dl4s_host_transformer_greedy_cached(*head, C.c_int(0 if cached == "stepwise" else 1), *tail))
        else:
            _check(load().dl4s_host_transformer_greedy(*head, *tail))
        res = [[int(x) for x in toks[:n.value]]]
        if return_logits:
            res.append(logits[:n.value])
        if timing:
            res.append(ms.value)
        return res[0] if len(res) == 1 else tuple(res)


def positional_encoding(ctx, max_len, hidden, fused=True):
    out = np.empty((max_len, hidden), np.float32)
    _check(load().dl4s_host_positional_encoding(ctx.handle, int(fused), _i64(max_len), _i64(hidden), _p(out)))
    return out


def tensor_encode_json(ctx, values):
    """Tensor -> the JSON text the reference's Codable conformance produces (through a device tensor)."""
    v = np.require(values, np.float32, "C")        # keeps a 0-d array 0-d (a scalar tensor has shape [])
    shp = (_i64 * max(1, v.ndim))(*v.shape)
    need = C.c_size_t()
    _check(load().dl4s_host_tensor_encode_json(ctx.handle, _p(v), shp, v.ndim, None, C.c_size_t(0), C.byref(need)))
    buf = C.create_string_buffer(need.value)
    _check(load().dl4s_host_tensor_encode_json(ctx.handle, _p(v), shp, v.ndim, buf, C.c_size_t(need.value), None))
    return buf.value.decode()


def tensor_decode_json(ctx, text):
    """JSON text of an encoded Tensor -> numpy array (through a device tensor)."""
    js = text.encode()
    n, dim = _i64(), C.c_int()
    shp = (_i64 * 8)()
    _check(load().dl4s_host_tensor_decode_json(ctx.handle, js, None, C.byref(n), shp, C.byref(dim)))
    out = np.empty(tuple(shp[i] for i in range(dim.value)), np.float32)
    _check(load().dl4s_host_tensor_decode_json(ctx.handle, js, _p(out) if out.size else None, None, None, None))
    return out

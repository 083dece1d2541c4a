"""ctypes binding of libdl4s_hip.so (the C ABI declared in include/dl4s_hip.h).

The binding never computes anything itself and has no CPU fallback: if the shared library is missing,
cannot be loaded or a call fails, it raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdl4s_hip.so")

MASK_NONE, MASK_DENSE, MASK_CAUSAL, MASK_KEY_LENGTHS, MASK_CAUSAL_OR_KEY_LENGTHS = range(5)
SDPA_STRICT = 1
SDPA_TOKEN_MAJOR = 2
SDPA_NO_KEY_SPLIT = 4
ACT_NONE, ACT_GELU = 0, 1
OP_ADD, OP_SUB, OP_MUL, OP_DIV = range(4)

_vp = C.c_void_p
_i64 = C.c_int64


class MaskDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("dense", _vp), ("shape", _i64 * 4), ("lengths", _vp), ("classes", _vp)]


class Dl4sHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("dl4s_hip status %d: %s" % (code, msg))
        self.code = code


_lib = None


def load():
    """Loads the shared library (built in-tree by `python -m dl4s_amd.build`)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m dl4s_amd.build`" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        _lib.dl4s_hip_last_error.restype = C.c_char_p
    return _lib


def _check(rc):
    if rc != 0:
        raise Dl4sHipError(rc, load().dl4s_hip_last_error().decode())


class DeviceBuffer:
    """A device allocation owned by a Context (freed back to its pool on release())."""

    def __init__(self, ctx, nbytes, shape=None, dtype=np.float32):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        self.shape = tuple(shape) if shape is not None else None
        self.dtype = np.dtype(dtype)
        p = _vp()
        _check(ctx.lib.dl4s_hip_alloc(ctx.handle, C.c_size_t(self.nbytes), C.byref(p)))
        self.ptr = p.value

    def release(self):
        if self.ptr is not None:
            _check(self.ctx.lib.dl4s_hip_free(self.ctx.handle, _vp(self.ptr)))
            self.ptr = None

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        _check(self.ctx.lib.dl4s_hip_assign_d2h(self.ctx.handle, out.ctypes.data_as(_vp), _vp(self.ptr),
                                                C.c_size_t(out.nbytes)))
        return out

    def offset(self, nbytes):
        return self.ptr + int(nbytes)


def _shape_arr(shape):
    return (_i64 * max(1, len(shape)))(*shape)


def graph_supported():
    """False when the process runs under rocprofv3 (graph launches abort its intercepted queue)."""
    return bool(load().dl4s_hip_graph_supported())


class Graph:
    """A recorded sequence of calls (dl4s_hip_graph_*); replay() enqueues it on the context's stream."""

    def __init__(self, ctx, handle):
        self.ctx, self.handle = ctx, handle

    def replay(self):
        _check(self.ctx.lib.dl4s_hip_graph_launch(self.ctx.handle, self.handle))

    @property
    def nodes(self):
        n = C.c_size_t()
        _check(self.ctx.lib.dl4s_hip_graph_node_count(self.ctx.handle, self.handle, C.byref(n)))
        return n.value

    def destroy(self):
        if self.handle is not None and self.ctx.handle is not None:
            _check(self.ctx.lib.dl4s_hip_graph_destroy(self.ctx.handle, self.handle))
        self.handle = None


class Context:
    """One GPU, one stream, one pooled allocator (dl4s_hip_ctx)."""

    def __init__(self, device=0):
        self.lib = load()
        h = _vp()
        _check(self.lib.dl4s_hip_create(int(device), C.byref(h)))
        self.handle = h

    def close(self):
        if self.handle is not None:
            _check(self.lib.dl4s_hip_destroy(self.handle))
            self.handle = None

    # ---- memory
    def empty(self, shape, dtype=np.float32):
        n = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        return DeviceBuffer(self, n, shape, dtype)

    def to_device(self, arr, dtype=np.float32):
        a = np.ascontiguousarray(arr, dtype=dtype)
        buf = DeviceBuffer(self, a.nbytes, a.shape, dtype)
        _check(self.lib.dl4s_hip_assign_h2d(self.handle, _vp(buf.ptr), a.ctypes.data_as(_vp), C.c_size_t(a.nbytes)))
        return buf

    def assign_h2d(self, buf, arr):
        """Overwrites a DeviceBuffer with a host array of the same byte size."""
        a = np.ascontiguousarray(arr, dtype=buf.dtype)
        assert a.nbytes == buf.nbytes
        _check(self.lib.dl4s_hip_assign_h2d(self.handle, _vp(buf.ptr), a.ctypes.data_as(_vp), C.c_size_t(a.nbytes)))

    def sync(self):
        _check(self.lib.dl4s_hip_sync(self.handle))

    def timer_begin(self):
        _check(self.lib.dl4s_hip_timer_begin(self.handle))

    def timer_end(self):
        ms = C.c_float()
        _check(self.lib.dl4s_hip_timer_end(self.handle, C.byref(ms)))
        return ms.value

    # ---- recorded call sequences
    def graph_begin(self):
        _check(self.lib.dl4s_hip_graph_begin(self.handle))

    def graph_end(self, keep=True):
        """Ends the recording; returns a Graph, or None when keep is False (the recording is given up)."""
        if not keep:
            _check(self.lib.dl4s_hip_graph_end(self.handle, None))
            return None
        g = _vp()
        _check(self.lib.dl4s_hip_graph_end(self.handle, C.byref(g)))
        return Graph(self, g)

    def device_info(self):
        cu, khz = C.c_int(), C.c_int()
        name = C.create_string_buffer(256)
        _check(self.lib.dl4s_hip_device_info(self.handle, C.byref(cu), C.byref(khz), name, C.c_size_t(256)))
        return {"cu_count": cu.value, "clock_khz": khz.value, "name": name.value.decode()}

    def mem_stats(self):
        a, b = C.c_size_t(), C.c_size_t()
        _check(self.lib.dl4s_hip_mem_stats(self.handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    def pool_trim(self, keep_bytes=0):
        _check(self.lib.dl4s_hip_pool_trim(self.handle, C.c_size_t(keep_bytes)))

    # ---- fused attention
    def mask_desc(self, kind=MASK_NONE, dense=None, lengths=None):
        """dense: DeviceBuffer with .shape of rank <= 4; lengths: DeviceBuffer of int32 [B]."""
        m = MaskDesc()
        m.kind = kind
        if kind == MASK_DENSE:
            sh = (1,) * (4 - len(dense.shape)) + tuple(dense.shape)
            m.dense = dense.ptr
            m.shape = (_i64 * 4)(*sh)
        if kind in (MASK_KEY_LENGTHS, MASK_CAUSAL_OR_KEY_LENGTHS):
            m.lengths = lengths.ptr
        return m

    def mask_describe(self, mask, B, H, Lq, Lk):
        """dl4s_hip_mask_describe_f32: returns (descriptor, lengths DeviceBuffer); the descriptor is structured when the
        dense mask's values are exactly a structured kind's (keep the lengths buffer alive while it is used)."""
        lengths = DeviceBuffer(self, 4 * max(int(B), 1), shape=(int(B),), dtype=np.int32)
        out = MaskDesc()
        _check(self.lib.dl4s_hip_mask_describe_f32(self.handle, C.byref(mask), _i64(B), _i64(H), _i64(Lq), _i64(Lk), _vp(lengths.ptr),
                                                   C.byref(out)))
        return out, lengths

    def mask_classify(self, mask, B, H, Lq, Lk):
        """Prepares the tile classes of a dense mask descriptor once; returns the DeviceBuffer that holds them and sets
        mask.classes (keep the buffer alive as long as the descriptor is used)."""
        n = C.c_size_t()
        _check(self.lib.dl4s_hip_mask_classes_size(C.byref(mask), _i64(B), _i64(H), _i64(Lq), _i64(Lk), C.byref(n)))
        buf = DeviceBuffer(self, max(int(n.value), 1), shape=(int(n.value),), dtype=np.uint8)
        _check(self.lib.dl4s_hip_mask_classify_f32(self.handle, C.byref(mask), _i64(B), _i64(H), _i64(Lq), _i64(Lk), _vp(buf.ptr)))
        mask.classes = buf.ptr
        return buf

    def sdpa_fwd(self, q, k, v, out, B, H, Lq, Lk, dk, dv, inv_temperature, mask=None, flags=0):
        _check(self.lib.dl4s_hip_sdpa_fwd_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(k)), _vp(_ptr(v)), _vp(_ptr(out)), _i64(B), _i64(H),
                                              _i64(Lq), _i64(Lk), _i64(dk), _i64(dv), C.c_float(inv_temperature),
                                              C.byref(mask) if mask is not None else None, C.c_uint32(flags)))

    def sdpa_fwd_stats(self, q, k, v, out, stats, B, H, Lq, Lk, d, inv_temperature, mask=None, flags=0):
        _check(self.lib.dl4s_hip_sdpa_fwd_stats_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(k)), _vp(_ptr(v)), _vp(_ptr(out)),
                                                    _vp(_ptr(stats)), _i64(B), _i64(H), _i64(Lq), _i64(Lk), _i64(d),
                                                    C.c_float(inv_temperature), C.byref(mask) if mask is not None else None,
                                                    C.c_uint32(flags)))

    def sdpa_bwd(self, q, k, v, out, stats, dout, dq, dk, dv, B, H, Lq, Lk, d, inv_temperature, mask=None, flags=0):
        _check(self.lib.dl4s_hip_sdpa_bwd_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(k)), _vp(_ptr(v)), _vp(_ptr(out)), _vp(_ptr(stats)),
                                              _vp(_ptr(dout)), _vp(_ptr(dq)), _vp(_ptr(dk)), _vp(_ptr(dv)), _i64(B), _i64(H), _i64(Lq),
                                              _i64(Lk), _i64(d), C.c_float(inv_temperature),
                                              C.byref(mask) if mask is not None else None, C.c_uint32(flags)))

    def sdpa_decode(self, q, kcache, vcache, out, B, H, T, Tcap, d, inv_temperature):
        _check(self.lib.dl4s_hip_sdpa_decode_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(kcache)), _vp(_ptr(vcache)), _vp(_ptr(out)),
                                                 _i64(B), _i64(H), _i64(T), _i64(Tcap), _i64(d), C.c_float(inv_temperature)))

    def sdpa_decode_lengths(self, q, kcache, vcache, out, B, H, T, Tcap, d, inv_temperature, lengths):
        """sdpa_decode with a valid key count per batch element (device int32 [B], or None)."""
        _check(self.lib.dl4s_hip_sdpa_decode_lengths_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(kcache)), _vp(_ptr(vcache)),
                                                         _vp(_ptr(out)), _i64(B), _i64(H), _i64(T), _i64(Tcap), _i64(d),
                                                         C.c_float(inv_temperature),
                                                         _vp(_ptr(lengths)) if lengths is not None else None))

    def sdpa_decode_noalloc(self, q, kcache, vcache, out, B, H, T, Tcap, d, inv_temperature):
        """sdpa_decode with its partial records in the library's fixed device block (no allocation)."""
        _check(self.lib.dl4s_hip_sdpa_decode_noalloc_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(kcache)), _vp(_ptr(vcache)),
                                                         _vp(_ptr(out)), _i64(B), _i64(H), _i64(T), _i64(Tcap), _i64(d),
                                                         C.c_float(inv_temperature)))

    def kv_append(self, kcache, vcache, k_new, v_new, B, H, pos, Tcap, d):
        _check(self.lib.dl4s_hip_kv_append_f32(self.handle, _vp(_ptr(kcache)), _vp(_ptr(vcache)), _vp(_ptr(k_new)), _vp(_ptr(v_new)),
                                               _i64(B), _i64(H), _i64(pos), _i64(Tcap), _i64(d)))

    def sdpa_decode_step(self, q, kcache, vcache, k_new, v_new, out, B, H, pos, Tcap, d, inv_temperature):
        _check(self.lib.dl4s_hip_sdpa_decode_step_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(kcache)), _vp(_ptr(vcache)),
                                                      _vp(_ptr(k_new)), _vp(_ptr(v_new)), _vp(_ptr(out)), _i64(B), _i64(H),
                                                      _i64(pos), _i64(Tcap), _i64(d), C.c_float(inv_temperature)))

    def sdpa_decode_step_at(self, q, kcache, vcache, k_new, v_new, out, B, H, pos_dev, Tcap, d, inv_temperature):
        """pos_dev: device address of the int32 row index."""
        _check(self.lib.dl4s_hip_sdpa_decode_step_at_f32(self.handle, _vp(_ptr(q)), _vp(_ptr(kcache)), _vp(_ptr(vcache)),
                                                         _vp(_ptr(k_new)), _vp(_ptr(v_new)), _vp(_ptr(out)), _i64(B), _i64(H),
                                                         _vp(_ptr(pos_dev)), _i64(Tcap), _i64(d), C.c_float(inv_temperature)))

    # ---- engine primitives
    def fill(self, value, result, count):
        _check(self.lib.dl4s_hip_fill_f32(self.handle, C.c_float(value), _vp(_ptr(result)), _i64(count)))

    def _bin(self, name, a, b, y, n):
        _check(getattr(self.lib, name)(self.handle, _vp(_ptr(a)), _vp(_ptr(b)), _vp(_ptr(y)), _i64(n)))

    def vadd(self, a, b, y, n): self._bin("dl4s_hip_vadd_f32", a, b, y, n)
    def vsub(self, a, b, y, n): self._bin("dl4s_hip_vsub_f32", a, b, y, n)
    def vmul(self, a, b, y, n): self._bin("dl4s_hip_vmul_f32", a, b, y, n)
    def vdiv(self, a, b, y, n): self._bin("dl4s_hip_vdiv_f32", a, b, y, n)

    def _un(self, name, x, y, n):
        _check(getattr(self.lib, name)(self.handle, _vp(_ptr(x)), _vp(_ptr(y)), _i64(n)))

    def vneg(self, x, y, n): self._un("dl4s_hip_vneg_f32", x, y, n)
    def exp(self, x, y, n): self._un("dl4s_hip_exp_f32", x, y, n)
    def sqrt(self, x, y, n): self._un("dl4s_hip_sqrt_f32", x, y, n)
    def relu(self, x, y, n): self._un("dl4s_hip_relu_f32", x, y, n)
    def tanh(self, x, y, n): self._un("dl4s_hip_tanh_f32", x, y, n)
    def log(self, x, y, n): self._un("dl4s_hip_log_f32", x, y, n)
    def sin(self, x, y, n): self._un("dl4s_hip_sin_f32", x, y, n)
    def cos(self, x, y, n): self._un("dl4s_hip_cos_f32", x, y, n)

    def argmax(self, x, count):
        idx, val = C.c_int64(), C.c_float()
        _check(self.lib.dl4s_hip_argmax_f32(self.handle, _vp(_ptr(x)), _i64(count), C.byref(idx), C.byref(val)))
        return idx.value, val.value

    def argmax_to(self, x, count, out_index_dev, counter_dev=None):
        """Index of the first maximum to device int32 *out_index_dev; *counter_dev += 1 when given."""
        _check(self.lib.dl4s_hip_argmax_to_f32(self.handle, _vp(_ptr(x)), _i64(count), _vp(_ptr(out_index_dev)),
                                               _vp(_ptr(counter_dev)) if counter_dev is not None else None))

    def embed_at(self, table, vocab, D, token_dev, scale, positions, position_rows, position_dev, y):
        sc = C.byref(C.c_float(scale)) if scale is not None else None
        _check(self.lib.dl4s_hip_embed_at_f32(self.handle, _vp(_ptr(table)), _i64(vocab), _i64(D), _vp(_ptr(token_dev)), sc,
                                              _vp(_ptr(positions)) if positions is not None else None, _i64(position_rows),
                                              _vp(_ptr(position_dev)) if position_dev is not None else None, _vp(_ptr(y))))

    def stack_axis(self, buffers, chunks, outer, y):
        arr = (_vp * max(1, len(buffers)))(*[_ptr(b) for b in buffers])
        ch = (C.c_int64 * max(1, len(chunks)))(*chunks)
        _check(self.lib.dl4s_hip_stack_axis_f32(self.handle, arr, ch, _i64(len(buffers)), _i64(outer), _vp(_ptr(y))))

    def embed_positions(self, table, vocab, D, tokens, batch, L, ignore_index, scale, positions, y):
        sc = C.byref(C.c_float(scale)) if scale is not None else None
        _check(self.lib.dl4s_hip_embed_positions_f32(self.handle, _vp(_ptr(table)), _i64(vocab), _i64(D), _vp(_ptr(tokens)),
                                                     _i64(batch), _i64(L), C.c_int32(ignore_index), sc,
                                                     _vp(_ptr(positions)) if positions is not None else None, _vp(_ptr(y))))

    def log_softmax(self, x, rows, n, y):
        _check(self.lib.dl4s_hip_log_softmax_f32(self.handle, _vp(_ptr(x)), _i64(rows), _i64(n), _vp(_ptr(y))))

    def gemm(self, lhs, lshape, rhs, rshape, result, alpha=1.0, beta=0.0, ta=False, tb=False):
        _check(self.lib.dl4s_hip_gemm_f32(self.handle, _vp(_ptr(lhs)), _i64(lshape[0]), _i64(lshape[1]), _vp(_ptr(rhs)),
                                          _i64(rshape[0]), _i64(rshape[1]), _vp(_ptr(result)), C.c_float(alpha),
                                          C.c_float(beta), int(ta), int(tb)))

    def gemm_batched(self, lhs, lshape, lstride, rhs, rshape, rstride, result, cstride, batch, alpha=1.0, beta=0.0,
                     ta=False, tb=False):
        _check(self.lib.dl4s_hip_gemm_batched_f32(self.handle, _vp(_ptr(lhs)), _i64(lshape[0]), _i64(lshape[1]), _i64(lstride),
                                                  _vp(_ptr(rhs)), _i64(rshape[0]), _i64(rshape[1]), _i64(rstride),
                                                  _vp(_ptr(result)), _i64(cstride), _i64(batch), C.c_float(alpha),
                                                  C.c_float(beta), int(ta), int(tb)))

    def gemm_grouped(self, lhs, lshape, rhs, rshape, results, alpha=1.0, beta=0.0, ta=False, tb=False):
        """len(lhs) (at most 4) products of one shape, operands anywhere, in one launch."""
        n = len(lhs)
        arr = lambda xs: (C.c_void_p * max(1, n))(*[_ptr(x) for x in xs])
        _check(self.lib.dl4s_hip_gemm_grouped_f32(self.handle, n, arr(lhs), _i64(lshape[0]), _i64(lshape[1]), arr(rhs),
                                                  _i64(rshape[0]), _i64(rshape[1]), arr(results), C.c_float(alpha),
                                                  C.c_float(beta), int(ta), int(tb)))

    def band(self, x, y, rows, cols, below, above):
        _check(self.lib.dl4s_hip_band_f32(self.handle, _vp(_ptr(x)), _vp(_ptr(y)), _i64(rows), _i64(cols),
                                          int(below is not None), _i64(below or 0), int(above is not None), _i64(above or 0)))

    def broadcast(self, op, a, ashape, b, bshape, y):
        _check(self.lib.dl4s_hip_broadcast_f32(self.handle, int(op), _vp(_ptr(a)), _shape_arr(ashape), len(ashape),
                                               _vp(_ptr(b)), _shape_arr(bshape), len(bshape), _vp(_ptr(y))))

    def reduce_sum(self, x, shape, axes, y):
        ax = (C.c_int32 * max(1, len(axes)))(*axes)
        _check(self.lib.dl4s_hip_reduce_sum_f32(self.handle, _vp(_ptr(x)), _shape_arr(shape), len(shape), ax, len(axes),
                                                _vp(_ptr(y))))

    def reduce_max(self, x, shape, axis, y):
        _check(self.lib.dl4s_hip_reduce_max_f32(self.handle, _vp(_ptr(x)), _shape_arr(shape), len(shape), int(axis),
                                                _vp(_ptr(y))))

    def permute_axes(self, x, shape, arrangement, y):
        arr = (C.c_int32 * max(1, len(arrangement)))(*arrangement)
        _check(self.lib.dl4s_hip_permute_axes_f32(self.handle, _vp(_ptr(x)), _shape_arr(shape), len(shape), arr, _vp(_ptr(y))))

    def subscript_read(self, x, shape, start, extent, y):
        """y (contiguous, shape `extent`) = x[start : start + extent] along every axis."""
        _check(self.lib.dl4s_hip_subscript_read_f32(self.handle, _vp(_ptr(x)), _shape_arr(shape), len(shape), _shape_arr(start),
                                                    _shape_arr(extent), _vp(_ptr(y))))

    def subscript_write(self, x, y, shape, start, extent):
        """y[start : start + extent] = x (contiguous, shape `extent`); y has shape `shape`."""
        _check(self.lib.dl4s_hip_subscript_write_f32(self.handle, _vp(_ptr(x)), _vp(_ptr(y)), _shape_arr(shape), len(shape),
                                                     _shape_arr(start), _shape_arr(extent)))

    def stack(self, buffers, count, y):
        arr = (_vp * max(1, len(buffers)))(*[_ptr(b) for b in buffers])
        _check(self.lib.dl4s_hip_stack_f32(self.handle, arr, _i64(len(buffers)), _i64(count), _vp(_ptr(y))))

    def layernorm(self, x, residual, scale, shift, y, B, rows, D):
        _check(self.lib.dl4s_hip_layernorm_f32(self.handle, _vp(_ptr(x)), _vp(_ptr(residual)) if residual is not None else None,
                                               _vp(_ptr(scale)), _vp(_ptr(shift)), _vp(_ptr(y)), _i64(B), _i64(rows), _i64(D)))

    def layernorm_reference_order(self, x, residual, scale, shift, y, B, rows, D):
        _check(self.lib.dl4s_hip_layernorm_reference_order_f32(
            self.handle, _vp(_ptr(x)), _vp(_ptr(residual)) if residual is not None else None, _vp(_ptr(scale)), _vp(_ptr(shift)),
            _vp(_ptr(y)), _i64(B), _i64(rows), _i64(D)))

    def dense_fused(self, x, rows, in_features, weights, out_features, bias, activation, residual, y):
        _check(self.lib.dl4s_hip_dense_fused_f32(self.handle, _vp(_ptr(x)), _i64(rows), _i64(in_features), _vp(_ptr(weights)),
                                                 _i64(out_features), _vp(_ptr(bias)) if bias is not None else None, int(activation),
                                                 _vp(_ptr(residual)) if residual is not None else None, _vp(_ptr(y))))

    def dense_layernorm(self, x, rows, in_features, weights, out_features, bias, activation, residual, item_rows, scale, shift, y):
        _check(self.lib.dl4s_hip_dense_layernorm_f32(self.handle, _vp(_ptr(x)), _i64(rows), _i64(in_features), _vp(_ptr(weights)),
                                                     _i64(out_features), _vp(_ptr(bias)) if bias is not None else None, int(activation),
                                                     _vp(_ptr(residual)) if residual is not None else None, _i64(item_rows),
                                                     _vp(_ptr(scale)), _vp(_ptr(shift)), _vp(_ptr(y))))

    def bias_gelu(self, x, bias, y, rows, D):
        _check(self.lib.dl4s_hip_bias_gelu_f32(self.handle, _vp(_ptr(x)), _vp(_ptr(bias)) if bias is not None else None,
                                               _vp(_ptr(y)), _i64(rows), _i64(D)))


def _ptr(x):
    """DeviceBuffer or raw integer device address."""
    return x.ptr if isinstance(x, DeviceBuffer) else int(x)

// Host-side mirror of the DL4S interfaces on the attention forward path, written against the C ABI of
// libdl4s_hip.so.  The reference is Swift; this is the C++ rendering of the same surface with the same
// names, argument meaning and error behaviour:
//
//   DeviceType / MemoryOperatorsType / EngineType   Engine/Engine.swift:30-35, :39-139, :143-581
//   Buffer / ShapedBuffer                           Engine/Buffer.swift:30-107
//   Tensor / TensorHandle                           Tensor/Tensor.swift:29-176
//   tensor operators                                Tensor/Operators/{Binary,Unary,Reduce,Matrix,Shape,Stack,Subscript,UtilOps}.swift
//   LayerNorm, Dense, Dropout                       NN/Layer/{LayerNorm,Dense,Dropout}.swift
//   ScaledDotProductAttention, MultiHeadAttention, PointwiseFeedForward, TransformerEncoderBlock,
//   TransformerDecoderBlock, makeEncoderMasks, makeDecoderMasks   NN/Models/Transformer/*.swift
//
// Contract violations that the reference traps on (precondition / fatalError) throw dl4s::Trap here.
//
// Two execution modes, selected by HIP::fused():
//   false  every tensor operator issues exactly the engine calls the reference issues (per-slice gemm loop +
//          stack, materialised score tensors, softmax and LayerNorm as primitive sequences);
//   true   the layers take the backend's fused entry points where it has them: one fused attention launch in
//          ScaledDotProductAttention, one strided-batched gemm per broadcastMatrixMultiplied, fused
//          residual + LayerNorm, fused bias + GELU.
// HIP::attentionHook() with fused() == false is the reference with nothing but the fused-attention hook patched into
// ScaledDotProductAttention.callAsFunction: that layer makes its one fused call on the [B,H,L,d] tensors it is handed,
// every other operator issues the reference's engine calls.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <memory>
#include <numeric>
#include <optional>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/dl4s_hip.h"

namespace dl4s {

struct Trap : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline void precondition(bool ok, const char *msg) {
    if (!ok) throw Trap(msg);
}

using Shape = std::vector<int64_t>;

inline int64_t count_of(const Shape &s) {
    int64_t n = 1;
    for (int64_t v : s) n *= v;
    return n;
}

// Util.swift:40-45
inline Shape shapeForBroadcastedOperands(const Shape &lhs, const Shape &rhs) {
    const size_t dim = std::max(lhs.size(), rhs.size());
    Shape out(dim);
    for (size_t i = 0; i < dim; ++i) {
        const int64_t l = i < dim - lhs.size() ? 1 : lhs[i - (dim - lhs.size())];
        const int64_t r = i < dim - rhs.size() ? 1 : rhs[i - (dim - rhs.size())];
        out[i] = std::max(l, r);
    }
    return out;
}

// ------------------------------------------------------------------------- Buffer.swift
struct Buffer {
    float *memory = nullptr;  // RawBuffer of the HIP device: a device pointer (offset views are pointer arithmetic)
};

struct ShapedBuffer {
    Buffer values;
    Shape shape;
    int dim() const { return (int)shape.size(); }
    int64_t count() const { return count_of(shape); }
    ShapedBuffer reshaped(Shape s) const { return ShapedBuffer{values, std::move(s)}; }
};

// ------------------------------------------------------------------------- the HIP device
struct HIP {
    static dl4s_hip_ctx *&context() {
        static dl4s_hip_ctx *ctx = nullptr;
        return ctx;
    }
    static bool &fused() {
        static bool f = true;
        return f;
    }
    static bool &attentionHook() {
        static bool f = false;
        return f;
    }
    // Fused layers only.  false: key tiles that the mask blocks entirely are skipped (their weights are exactly zero;
    // the reference's 0 * v at such keys only differs when k or v hold NaN / Inf there) and the LayerNorm sums are
    // added in a tree.  true: every tile is visited and the LayerNorm sums are added in the reference's sequential
    // order, so that NaN / Inf come out where the reference has them whatever the values.
    static bool &strictMasks() {
        static bool f = false;
        return f;
    }
    static void check(int rc) {
        if (rc != DL4S_HIP_OK) throw Trap(std::string("dl4s_hip: ") + dl4s_hip_last_error());
    }

    // MemoryOperatorsType (Engine/Engine.swift:39-139), the subset the path uses
    struct Memory {
        static Buffer allocateBuffer(int64_t capacity) {
            void *p = nullptr;
            check(dl4s_hip_alloc(context(), (size_t)capacity * sizeof(float), &p));
            return Buffer{static_cast<float *>(p)};
        }
        static ShapedBuffer allocateBuffer(const Shape &shape) { return ShapedBuffer{allocateBuffer(count_of(shape)), shape}; }
        static void free(Buffer b) { check(dl4s_hip_free(context(), b.memory)); }
        static void assign(const float *host, Buffer dst, int64_t count) {
            check(dl4s_hip_assign_h2d(context(), dst.memory, host, (size_t)count * sizeof(float)));
        }
        static void assign(Buffer src, Buffer dst, int64_t count) {
            check(dl4s_hip_assign_d2d(context(), dst.memory, src.memory, (size_t)count * sizeof(float)));
        }
        static void assign(Buffer src, float *host, int64_t count) {
            check(dl4s_hip_assign_d2h(context(), host, src.memory, (size_t)count * sizeof(float)));
        }
        static float getValue(Buffer src) {
            float v;
            check(dl4s_hip_get_value_f32(context(), src.memory, &v));
            return v;
        }
        static int64_t getSize(Buffer b) {
            size_t bytes;
            check(dl4s_hip_get_size(context(), b.memory, &bytes));
            return (int64_t)(bytes / sizeof(float));
        }
        static Buffer advance(Buffer b, int64_t by) { return Buffer{b.memory + by}; }
    };

    // EngineType (Engine/Engine.swift:143-581), the subset the path uses
    struct Engine {
        static void fill(float value, Buffer result, int64_t count) { check(dl4s_hip_fill_f32(context(), value, result.memory, count)); }
        static void vAdd(Buffer l, Buffer r, Buffer res, int64_t n) { check(dl4s_hip_vadd_f32(context(), l.memory, r.memory, res.memory, n)); }
        static void vNeg(Buffer v, Buffer res, int64_t n) { check(dl4s_hip_vneg_f32(context(), v.memory, res.memory, n)); }
        static void vSub(Buffer l, Buffer r, Buffer res, int64_t n) { check(dl4s_hip_vsub_f32(context(), l.memory, r.memory, res.memory, n)); }
        static void vMul(Buffer l, Buffer r, Buffer res, int64_t n) { check(dl4s_hip_vmul_f32(context(), l.memory, r.memory, res.memory, n)); }
        static void vDiv(Buffer l, Buffer r, Buffer res, int64_t n) { check(dl4s_hip_vdiv_f32(context(), l.memory, r.memory, res.memory, n)); }
        static void gemm(const ShapedBuffer &lhs, const ShapedBuffer &rhs, const ShapedBuffer &result, float alpha, float beta,
                         bool transposeFirst, bool transposeSecond) {
            check(dl4s_hip_gemm_f32(context(), lhs.values.memory, lhs.shape[0], lhs.shape[1], rhs.values.memory, rhs.shape[0],
                                    rhs.shape[1], result.values.memory, alpha, beta, transposeFirst, transposeSecond));
        }
        static void band(const ShapedBuffer &buffer, const ShapedBuffer &result, std::optional<int64_t> below,
                         std::optional<int64_t> above) {
            precondition(buffer.shape == result.shape, "Shape of result must be equal to shape of buffer.");
            precondition(buffer.dim() == 2, "Band can only be computed on tensor of dimensionality 2.");
            check(dl4s_hip_band_f32(context(), buffer.values.memory, result.values.memory, buffer.shape[0], buffer.shape[1],
                                    below.has_value(), below.value_or(0), above.has_value(), above.value_or(0)));
        }
        static void broadcast(int op, const ShapedBuffer &l, const ShapedBuffer &r, const ShapedBuffer &res) {
            check(dl4s_hip_broadcast_f32(context(), op, l.values.memory, l.shape.data(), l.dim(), r.values.memory, r.shape.data(),
                                         r.dim(), res.values.memory));
        }
        static void broadcastAdd(const ShapedBuffer &l, const ShapedBuffer &r, const ShapedBuffer &res) { broadcast(DL4S_OP_ADD, l, r, res); }
        static void broadcastSub(const ShapedBuffer &l, const ShapedBuffer &r, const ShapedBuffer &res) { broadcast(DL4S_OP_SUB, l, r, res); }
        static void broadcastMul(const ShapedBuffer &l, const ShapedBuffer &r, const ShapedBuffer &res) { broadcast(DL4S_OP_MUL, l, r, res); }
        static void broadcastDiv(const ShapedBuffer &l, const ShapedBuffer &r, const ShapedBuffer &res) { broadcast(DL4S_OP_DIV, l, r, res); }
        static void reduceSum(const ShapedBuffer &values, const ShapedBuffer &result, const std::vector<int> &axes) {
            std::vector<int32_t> ax(axes.begin(), axes.end());
            check(dl4s_hip_reduce_sum_f32(context(), values.values.memory, values.shape.data(), values.dim(), ax.data(), (int)ax.size(),
                                          result.values.memory));
        }
        static void reduceMax(const ShapedBuffer &values, const ShapedBuffer &result, int axis) {
            check(dl4s_hip_reduce_max_f32(context(), values.values.memory, values.shape.data(), values.dim(), axis, result.values.memory));
        }
        static void exp(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_exp_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void tanh(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_tanh_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void sqrt(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_sqrt_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void relu(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_relu_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void permuteAxes(const ShapedBuffer &values, const ShapedBuffer &result, const std::vector<int> &arangement) {
            std::vector<int32_t> ar(arangement.begin(), arangement.end());
            check(dl4s_hip_permute_axes_f32(context(), values.values.memory, values.shape.data(), values.dim(), ar.data(),
                                            result.values.memory));
        }
        static void stack(const std::vector<ShapedBuffer> &buffers, const ShapedBuffer &result, int axis) {
            std::vector<const float *> ptrs;
            for (auto &b : buffers) ptrs.push_back(b.values.memory);
            bool equal = true;
            for (auto &b : buffers) equal = equal && b.shape == buffers[0].shape;
            if (axis == 0 && equal) {
                check(dl4s_hip_stack_f32(context(), ptrs.data(), (int64_t)ptrs.size(), buffers.empty() ? 0 : buffers[0].count(),
                                         result.values.memory));
                return;
            }
            int64_t outer = 1;
            for (int i = 0; i < axis; ++i) outer *= result.shape[i];
            std::vector<int64_t> chunks;
            for (auto &b : buffers) chunks.push_back(outer == 0 ? 0 : b.count() / outer);
            check(dl4s_hip_stack_axis_f32(context(), ptrs.data(), chunks.data(), (int64_t)ptrs.size(), outer, result.values.memory));
        }
        static void log(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_log_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void sin(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_sin_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static void cos(const ShapedBuffer &v, const ShapedBuffer &r) { check(dl4s_hip_cos_f32(context(), v.values.memory, r.values.memory, v.count())); }
        static std::pair<int64_t, float> argmax(Buffer values, int64_t count) {
            int64_t i;
            float v;
            check(dl4s_hip_argmax_f32(context(), values.memory, count, &i, &v));
            return {i, v};
        }
        // Fused entry points of this backend (no counterpart in EngineType).
        // tokenMajor: q, result are [B,Lq,H,d] and k, v [B,Lk,H,d] (the projections before their permutes)
        // the dense mask tensor of a layer as the library's descriptor (right-aligned to [B,H,Lq,Lk])
        static dl4s_mask_desc denseMaskDescriptor(const ShapedBuffer &mask) {
            precondition(mask.dim() <= 4, "mask must be broadcastable to [batchSize, heads, queryCount, keyCount]");
            dl4s_mask_desc md{};
            md.kind = DL4S_MASK_DENSE_F32;
            md.dense = mask.values.memory;
            for (int i = 0; i < 4; ++i) md.shape[i] = 1;
            for (int i = 0; i < mask.dim(); ++i) md.shape[4 - mask.dim() + i] = mask.shape[i];
            return md;
        }
        // prepared: the mask as Tensor::attentionMask left it (structured, or dense with its tile classes), or nullptr to
        // hand the mask tensor over as it is
        static void fusedAttention(const ShapedBuffer &q, const ShapedBuffer &k, const ShapedBuffer &v, const ShapedBuffer *mask,
                                   const ShapedBuffer &result, float temperature, bool tokenMajor = false,
                                   const dl4s_mask_desc *prepared = nullptr) {
            dl4s_mask_desc md{};
            if (mask) md = prepared ? *prepared : denseMaskDescriptor(*mask);
            const int h = tokenMajor ? 2 : 1, l = tokenMajor ? 1 : 2;
            check(dl4s_hip_sdpa_fwd_f32(context(), q.values.memory, k.values.memory, v.values.memory, result.values.memory,
                                        q.shape[0], q.shape[h], q.shape[l], k.shape[l], q.shape[3], v.shape[3],
                                        1.0f / temperature, mask && md.kind != DL4S_MASK_NONE ? &md : nullptr,
                                        (strictMasks() ? DL4S_SDPA_STRICT : 0u) | (tokenMajor ? DL4S_SDPA_TOKEN_MAJOR : 0u)));
        }
        // the same with a structured mask descriptor (kind + device int32 lengths) instead of a dense mask tensor
        static void fusedAttentionStructured(const ShapedBuffer &q, const ShapedBuffer &k, const ShapedBuffer &v, int kind,
                                             const int32_t *lengths, const ShapedBuffer &result, float temperature, bool tokenMajor) {
            dl4s_mask_desc md{};
            md.kind = kind;
            md.lengths = lengths;
            const int h = tokenMajor ? 2 : 1, l = tokenMajor ? 1 : 2;
            check(dl4s_hip_sdpa_fwd_f32(context(), q.values.memory, k.values.memory, v.values.memory, result.values.memory,
                                        q.shape[0], q.shape[h], q.shape[l], k.shape[l], q.shape[3], v.shape[3], 1.0f / temperature,
                                        kind == DL4S_MASK_NONE ? nullptr : &md,
                                        (strictMasks() ? DL4S_SDPA_STRICT : 0u) | (tokenMajor ? DL4S_SDPA_TOKEN_MAJOR : 0u)));
        }
        // one query row per (batch, head) over a key / value cache [B,H,Tcap,d]: q, result [B,H,1,d] (equally [B,1,H,d])
        static void decodeAttention(const ShapedBuffer &q, const ShapedBuffer &keyCache, const ShapedBuffer &valueCache, int64_t rows,
                                    const ShapedBuffer &result, float temperature) {
            check(dl4s_hip_sdpa_decode_f32(context(), q.values.memory, keyCache.values.memory, valueCache.values.memory,
                                           result.values.memory, keyCache.shape[0], keyCache.shape[1], rows, keyCache.shape[2],
                                           keyCache.shape[3], 1.0f / temperature));
        }
        // the same after writing newKey, newValue [B,H,1,d] into row `position` of the caches (rows 0 ... position attended)
        static void decodeAttentionAppending(const ShapedBuffer &q, const ShapedBuffer &keyCache, const ShapedBuffer &valueCache,
                                             const ShapedBuffer &newKey, const ShapedBuffer &newValue, int64_t position,
                                             const ShapedBuffer &result, float temperature) {
            check(dl4s_hip_sdpa_decode_step_f32(context(), q.values.memory, keyCache.values.memory, valueCache.values.memory,
                                                newKey.values.memory, newValue.values.memory, result.values.memory, keyCache.shape[0],
                                                keyCache.shape[1], position, keyCache.shape[2], keyCache.shape[3], 1.0f / temperature));
        }
        // the same with the row position read from device memory (a step that is recorded once and replayed)
        static void decodeAttentionAppendingAt(const ShapedBuffer &q, const ShapedBuffer &keyCache, const ShapedBuffer &valueCache,
                                               const ShapedBuffer &newKey, const ShapedBuffer &newValue, const int32_t *positionOnDevice,
                                               const ShapedBuffer &result, float temperature) {
            check(dl4s_hip_sdpa_decode_step_at_f32(context(), q.values.memory, keyCache.values.memory, valueCache.values.memory,
                                                   newKey.values.memory, newValue.values.memory, result.values.memory, keyCache.shape[0],
                                                   keyCache.shape[1], positionOnDevice, keyCache.shape[2], keyCache.shape[3],
                                                   1.0f / temperature));
        }
        // result[D] = table[*token] * scale + positions[*position], token and position in device memory
        static void embedAt(const ShapedBuffer &table, const int32_t *tokenOnDevice, const float *scale, const ShapedBuffer &positions,
                            const int32_t *positionOnDevice, const ShapedBuffer &result) {
            check(dl4s_hip_embed_at_f32(context(), table.values.memory, table.shape[0], table.shape[1], tokenOnDevice, scale,
                                        positions.values.memory, positions.shape[0], positionOnDevice, result.values.memory));
        }
        // *tokenOnDevice = argmax(values); *counterOnDevice += 1
        static void argmaxTo(const ShapedBuffer &values, int32_t *tokenOnDevice, int32_t *counterOnDevice) {
            check(dl4s_hip_argmax_to_f32(context(), values.values.memory, values.count(), tokenOnDevice, counterOnDevice));
        }
        // result = act(x . weights + bias) + residual  (bias, residual optional)
        static void denseFused(const ShapedBuffer &x, const ShapedBuffer &weights, const ShapedBuffer *bias, int activation,
                               const ShapedBuffer *residual, const ShapedBuffer &result) {
            precondition(x.count() % weights.shape[0] == 0, "Matmul operands must have matching shapes");
            check(dl4s_hip_dense_fused_f32(context(), x.values.memory, x.count() / weights.shape[0], weights.shape[0],
                                           weights.values.memory, weights.shape[1], bias ? bias->values.memory : nullptr, activation,
                                           residual ? residual->values.memory : nullptr, result.values.memory));
        }
        // result = LayerNorm(act(x . weights + bias) + residual), statistics over items of itemRows rows
        static void denseFusedLayerNorm(const ShapedBuffer &x, const ShapedBuffer &weights, const ShapedBuffer *bias, int activation,
                                        const ShapedBuffer *residual, int64_t itemRows, const ShapedBuffer &scale, const ShapedBuffer &shift,
                                        const ShapedBuffer &result) {
            precondition(x.count() % weights.shape[0] == 0, "Matmul operands must have matching shapes");
            if (strictMasks()) {      // the product with its epilogue, then the statistics in the reference's order
                denseFused(x, weights, bias, activation, residual, result);
                const int64_t rows = x.count() / weights.shape[0], D = weights.shape[1];
                check(dl4s_hip_layernorm_reference_order_f32(context(), result.values.memory, nullptr, scale.values.memory,
                                                             shift.values.memory, result.values.memory, rows / itemRows, itemRows, D));
                return;
            }
            check(dl4s_hip_dense_layernorm_f32(context(), x.values.memory, x.count() / weights.shape[0], weights.shape[0],
                                               weights.values.memory, weights.shape[1], bias ? bias->values.memory : nullptr, activation,
                                               residual ? residual->values.memory : nullptr, itemRows, scale.values.memory,
                                               shift.values.memory, result.values.memory));
        }
        static void gemmBatched(const ShapedBuffer &lhs, int64_t lstride, const ShapedBuffer &rhs, int64_t rstride,
                                const ShapedBuffer &result, int64_t batch, bool tA, bool tB) {
            const int ld = lhs.dim(), rd = rhs.dim(), od = result.dim();
            check(dl4s_hip_gemm_batched_f32(context(), lhs.values.memory, lhs.shape[ld - 2], lhs.shape[ld - 1], lstride,
                                            rhs.values.memory, rhs.shape[rd - 2], rhs.shape[rd - 1], rstride, result.values.memory,
                                            result.shape[od - 2] * result.shape[od - 1], batch, 1.0f, 0.0f, tA, tB));
        }
        // up to 4 products [rows, in] . [in, out] of one shape in one launch (operands anywhere)
        static void gemmGrouped(const std::vector<ShapedBuffer> &lhs, int64_t rows, const std::vector<ShapedBuffer> &rhs,
                                const std::vector<ShapedBuffer> &results) {
            const float *a[4], *b[4];
            float *c[4];
            precondition(lhs.size() == rhs.size() && lhs.size() == results.size() && lhs.size() <= 4, "bad group");
            for (size_t i = 0; i < lhs.size(); ++i) {
                precondition(lhs[i].count() == rows * rhs[i].shape[0] && rhs[i].shape == rhs[0].shape, "Matmul operands must have matching shapes");
                a[i] = lhs[i].values.memory;
                b[i] = rhs[i].values.memory;
                c[i] = results[i].values.memory;
            }
            check(dl4s_hip_gemm_grouped_f32(context(), (int)lhs.size(), a, rows, rhs[0].shape[0], b, rhs[0].shape[0], rhs[0].shape[1], c,
                                            1.0f, 0.0f, 0, 0));
        }
        static void layerNorm(const ShapedBuffer &x, const ShapedBuffer *residual, const ShapedBuffer &scale,
                              const ShapedBuffer &shift, const ShapedBuffer &result) {
            const int64_t B = x.shape[0], D = scale.count();
            check((strictMasks() ? dl4s_hip_layernorm_reference_order_f32 : dl4s_hip_layernorm_f32)(context(), x.values.memory, residual ? residual->values.memory : nullptr, scale.values.memory,
                                         shift.values.memory, result.values.memory, B, x.count() / (B * D), D));
        }
        // rows of `table` for device int32 tokens [batch, L], optionally * scale + positions[l]
        static void embedPositions(const ShapedBuffer &table, const int32_t *tokens, int64_t batch, int64_t L, int32_t ignoreIndex,
                                   const float *scale, const ShapedBuffer *positions, const ShapedBuffer &result) {
            check(dl4s_hip_embed_positions_f32(context(), table.values.memory, table.shape[0], table.shape[1], tokens, batch, L, ignoreIndex,
                                               scale, positions ? positions->values.memory : nullptr, result.values.memory));
        }
        static void logSoftmax(const ShapedBuffer &x, const ShapedBuffer &result) {
            const int64_t n = x.shape.back();
            check(dl4s_hip_log_softmax_f32(context(), x.values.memory, n == 0 ? 0 : x.count() / n, n, result.values.memory));
        }
        static void biasGelu(const ShapedBuffer &x, const ShapedBuffer &bias, const ShapedBuffer &result) {
            const int64_t D = bias.count();
            check(dl4s_hip_bias_gelu_f32(context(), x.values.memory, bias.values.memory, result.values.memory, x.count() / D, D));
        }
    };
};

using Device = HIP;

// A sequence of engine calls recorded into a HIP graph (dl4s_hip_graph_*; no counterpart in the reference).  Tensors
// created and released inside the recorded function stay reserved for the graph until it is destroyed.
class RecordedCalls {
    dl4s_hip_graph *graph_ = nullptr;
    dl4s_hip_ctx *ctx_ = nullptr;

   public:
    RecordedCalls() = default;
    RecordedCalls(const RecordedCalls &) = delete;
    RecordedCalls &operator=(const RecordedCalls &) = delete;
    ~RecordedCalls() { reset(); }
    explicit operator bool() const { return graph_ != nullptr; }
    void reset() {
        if (graph_) (void)dl4s_hip_graph_destroy(ctx_, graph_);
        graph_ = nullptr;
    }
    template <class F>
    void record(F &&calls) {
        reset();
        ctx_ = Device::context();
        Device::check(dl4s_hip_graph_begin(ctx_));
        try {
            calls();
        } catch (...) {
            (void)dl4s_hip_graph_end(ctx_, nullptr);
            throw;
        }
        Device::check(dl4s_hip_graph_end(ctx_, &graph_));
    }
    void replay() const {
        precondition(graph_ != nullptr, "nothing recorded");
        Device::check(dl4s_hip_graph_launch(ctx_, graph_));
    }
};

// ------------------------------------------------------------------------- Tensor.swift
// Owns a buffer; a handle with a parent is a view into the parent's allocation and frees nothing
// (Tensor/Tensor.swift:29-43).
struct TensorHandle {
    ShapedBuffer values;
    std::shared_ptr<TensorHandle> parent;
    // Not in the reference.  This buffer read as the attention mask of a [B,H,Lq,Lk] problem, prepared by the first fused
    // attention call that receives the tensor as its mask: the structured descriptor when the values are exactly those of
    // a causal and / or key-length mask (dl4s_hip_mask_describe_f32), else the dense descriptor with its tile classes
    // (dl4s_hip_mask_classify_f32).  The layers of a model all receive the one mask tensor their model built
    // (TransformerEncoder.swift:63, TransformerDecoder.swift:53-54), and tensors of this layer are never written after
    // they are made.
    struct PreparedMask {
        dl4s_mask_desc descriptor{};
        unsigned char *classes = nullptr;
        int32_t *lengths = nullptr;
        Shape shape;
        int64_t extents[4] = {0, 0, 0, 0};
        ~PreparedMask() {
            if (classes) dl4s_hip_free(Device::context(), classes);
            if (lengths) dl4s_hip_free(Device::context(), lengths);
        }
    };
    std::unique_ptr<PreparedMask> preparedMask;
    TensorHandle(ShapedBuffer v, std::shared_ptr<TensorHandle> p) : values(std::move(v)), parent(std::move(p)) {}
    TensorHandle(const TensorHandle &) = delete;
    ~TensorHandle() {
        preparedMask.reset();
        if (!parent) dl4s_hip_free(Device::context(), values.values.memory);
    }
};

class Tensor {
   public:
    std::shared_ptr<TensorHandle> handle;
    Shape shape;

    Tensor() = default;
    // Tensor(using:context:) -- takes ownership of a freshly allocated buffer
    explicit Tensor(ShapedBuffer buffer) : handle(std::make_shared<TensorHandle>(buffer, nullptr)), shape(buffer.shape) {}
    Tensor(std::shared_ptr<TensorHandle> h, Shape s) : handle(std::move(h)), shape(std::move(s)) {}
    // Tensor([Float], shape:)  (Tensor/Tensor.swift:143-153)
    Tensor(const float *host, const Shape &s) : Tensor(Device::Memory::allocateBuffer(s)) {
        Device::Memory::assign(host, handle->values.values, count());
    }
    Tensor(const std::vector<float> &host, const Shape &s) : Tensor(host.data(), s) {
        precondition((int64_t)host.size() == count_of(s), "element count does not match shape");
    }
    // Tensor(scalar): shape []  (Tensor/TensorExt.swift:88-90)
    explicit Tensor(float scalar) : Tensor(&scalar, Shape{}) {}
    // Tensor(repeating:shape:)
    static Tensor repeating(float value, const Shape &s) {
        Tensor t(Device::Memory::allocateBuffer(s));
        Device::Engine::fill(value, t.buffer(), t.count());
        return t;
    }

    int dim() const { return (int)shape.size(); }
    int64_t count() const { return count_of(shape); }
    Buffer buffer() const { return handle->values.values; }
    ShapedBuffer values() const { return ShapedBuffer{handle->values.values, shape}; }
    // elements (Tensor/TensorExt.swift:275-281)
    std::vector<float> elements() const {
        std::vector<float> out((size_t)count());
        Device::Memory::assign(buffer(), out.data(), count());
        return out;
    }
    float item() const { return Device::Memory::getValue(buffer()); }
    // Not in the reference.  This tensor as the attention mask of a [B,H,Lq,Lk] problem, prepared by the first call and
    // kept with the handle (see TensorHandle::PreparedMask), so that the attention calls of every layer that receives the
    // tensor neither classify its tiles nor, where it is a structured mask, read its values.  nullptr when the shape does
    // not fit the problem (the attention call then reports it).
    const dl4s_mask_desc *attentionMask(int64_t B, int64_t H, int64_t Lq, int64_t Lk) const {
        auto &slot = handle->preparedMask;
        if (slot && slot->shape == shape && slot->extents[0] == B && slot->extents[1] == H && slot->extents[2] == Lq && slot->extents[3] == Lk)
            return &slot->descriptor;
        if (dim() > 4 || B < 1) return nullptr;
        const dl4s_mask_desc dense = Device::Engine::denseMaskDescriptor(values());
        size_t bytes = 0;
        if (dl4s_hip_mask_classes_size(&dense, B, H, Lq, Lk, &bytes) != DL4S_HIP_OK) return nullptr;
        slot.reset(new TensorHandle::PreparedMask());
        slot->shape = shape;
        slot->extents[0] = B; slot->extents[1] = H; slot->extents[2] = Lq; slot->extents[3] = Lk;
        void *p = nullptr;
        Device::check(dl4s_hip_alloc(Device::context(), (size_t)B * sizeof(int32_t), &p));
        slot->lengths = static_cast<int32_t *>(p);
        // (refused while a call sequence is being recorded - it waits for the stream: the dense descriptor then)
        if (dl4s_hip_mask_describe_f32(Device::context(), &dense, B, H, Lq, Lk, slot->lengths, &slot->descriptor) != DL4S_HIP_OK)
            slot->descriptor = dense;
        if (slot->descriptor.kind == DL4S_MASK_DENSE_F32) {
            Device::check(dl4s_hip_alloc(Device::context(), bytes ? bytes : 1, &p));
            slot->classes = static_cast<unsigned char *>(p);
            Device::check(dl4s_hip_mask_classify_f32(Device::context(), &dense, B, H, Lq, Lk, slot->classes));
            slot->descriptor.classes = slot->classes;
        }
        return &slot->descriptor;
    }

    // view(as:) -- shares the handle; one extent may be -1 (Tensor/Operators/Shape.swift:40-67)
    Tensor view(Shape s) const {
        int64_t known = 1;
        int unknown = -1;
        for (size_t i = 0; i < s.size(); ++i) {
            if (s[i] == -1) {
                precondition(unknown < 0, "The size of at most one dimension can be unknown (-1).");
                unknown = (int)i;
            } else known *= s[i];
        }
        if (unknown >= 0) s[unknown] = known == 0 ? 0 : count() / known;
        precondition(count_of(s) == count(), "Number of elements in result must be equal to number of elements in source");
        return Tensor(handle, s);
    }
    Tensor unsqueezed(int at) const {
        Shape s = shape;
        s.insert(s.begin() + at, 1);
        return view(s);
    }
    // subscript with a prefix index: a zero-copy view kept alive through `parent`
    // (Tensor/Operators/Subscript.swift:42-67, Engine/CPU/CPU.swift:137-158)
    Tensor operator[](const std::vector<int64_t> &index) const {
        precondition((int)index.size() <= dim(), "index has more entries than the tensor has axes");
        int64_t offset = 0, stride = count();
        for (size_t i = 0; i < index.size(); ++i) {
            precondition(index[i] >= 0 && index[i] < shape[i], "index out of bounds");
            stride /= shape[i];
            offset += index[i] * stride;
        }
        Shape rest(shape.begin() + index.size(), shape.end());
        auto h = std::make_shared<TensorHandle>(ShapedBuffer{Device::Memory::advance(buffer(), offset), rest}, handle);
        return Tensor(h, rest);
    }

    // ---- binary operators (Tensor/Operators/Binary.swift:44-52, :104-112, :161-169, :235-243)
   private:
    template <class Same, class Bc>
    static Tensor binary(const Tensor &l, const Tensor &r, Same same, Bc bc) {
        Tensor res(Device::Memory::allocateBuffer(shapeForBroadcastedOperands(l.shape, r.shape)));
        if (l.shape == r.shape) same(l.buffer(), r.buffer(), res.buffer(), l.count());
        else bc(l.values(), r.values(), res.values());
        return res;
    }

   public:
    friend Tensor operator+(const Tensor &l, const Tensor &r) { return binary(l, r, Device::Engine::vAdd, Device::Engine::broadcastAdd); }
    friend Tensor operator-(const Tensor &l, const Tensor &r) { return binary(l, r, Device::Engine::vSub, Device::Engine::broadcastSub); }
    friend Tensor operator*(const Tensor &l, const Tensor &r) { return binary(l, r, Device::Engine::vMul, Device::Engine::broadcastMul); }
    friend Tensor operator/(const Tensor &l, const Tensor &r) { return binary(l, r, Device::Engine::vDiv, Device::Engine::broadcastDiv); }
    Tensor operator-() const {
        Tensor res(Device::Memory::allocateBuffer(shape));
        Device::Engine::vNeg(buffer(), res.buffer(), count());
        return res;
    }

    // ---- unary (Tensor/Operators/Unary.swift)
   private:
    template <class F>
    Tensor unary(F f) const {
        Tensor res(Device::Memory::allocateBuffer(shape));
        f(values(), res.values());
        return res;
    }

   public:
    Tensor exp() const { return unary(Device::Engine::exp); }          // :33-36
    Tensor tanh() const { return unary(Device::Engine::tanh); }        // :79-82
    Tensor sqrt() const { return unary(Device::Engine::sqrt); }
    Tensor rectifiedLinear() const { return unary(Device::Engine::relu); }
    Tensor log() const { return unary(Device::Engine::log); }          // :60-77
    Tensor sine() const { return unary(Device::Engine::sin); }         // :207-223
    Tensor cosine() const { return unary(Device::Engine::cos); }       // :225-241
    Tensor raised(const Tensor &power) const { return (log() * power).exp(); }                             // Binary.swift:408-410
    Tensor logSoftmax(int axis = 1) const {                                                                // :198-204
        if (Device::fused() && axis == dim() - 1) {
            Tensor res(Device::Memory::allocateBuffer(shape));
            Device::Engine::logSoftmax(values(), res.values());
            return res;
        }
        Tensor norm = *this - reduceMax({axis}).unsqueezed(axis);
        Tensor logSumExp = norm.exp().reduceSum({axis}).log().unsqueezed(axis);
        return norm - logSumExp;
    }
    int64_t argmax() const { return Device::Engine::argmax(buffer(), count()).first; }                     // Reduce.swift:128-130
    Tensor sigmoid() const { return Tensor(0.5f) * (*this * Tensor(0.5f)).tanh() + Tensor(0.5f); }        // :184-186
    Tensor gaussianErrorLinear() const { return *this * (*this * Tensor(1.702f)).sigmoid(); }             // :245-247
    Tensor softmax(int axis = 1) const {                                                                   // :190-194
        Tensor normalizer = reduceMax({axis}).unsqueezed(axis);
        Tensor exponentiated = (*this - normalizer).exp();
        return exponentiated / exponentiated.reduceSum({axis}).unsqueezed(axis);
    }

    // ---- reductions (Tensor/Operators/Reduce.swift:35-46, :87-110, :216-256)
    Shape reducedShape(const std::vector<int> &axes) const {
        Shape s;
        for (int i = 0; i < dim(); ++i)
            if (std::find(axes.begin(), axes.end(), i) == axes.end()) s.push_back(shape[i]);
        return s;
    }
    Tensor reduceSum(const std::vector<int> &axes) const {
        if (axes.empty()) return *this;
        Tensor res(Device::Memory::allocateBuffer(reducedShape(axes)));
        Device::Engine::reduceSum(values(), res.values(), axes);
        return res;
    }
    Tensor reduceMean(const std::vector<int> &axes) const {
        int64_t n = 1;
        for (int a : axes) n *= shape[a];
        return reduceSum(axes) / Tensor((float)n);
    }
    Tensor variance(const std::vector<int> &axes) const {
        Tensor m = reduceMean(axes);
        return (*this * *this).reduceMean(axes) - m * m;
    }
    Tensor reduceMax(const std::vector<int> &axes) const {
        precondition(axes.size() == 1, "reduceMax along several axes is not available for HIP");
        Tensor res(Device::Memory::allocateBuffer(reducedShape(axes)));
        Device::Engine::reduceMax(values(), res.values(), axes[0]);
        return res;
    }

    // ---- shape (Tensor/Operators/Shape.swift:121-155): source axis i goes to destination axis axes[i]
    Tensor permuted(const std::vector<int> &axes) const {
        precondition((int)axes.size() == dim(), "Axis arangement must have dimensionality of source tensor");
        Shape dst(dim());
        for (int i = 0; i < dim(); ++i) {
            precondition(axes[i] >= 0 && axes[i] < dim(), "Axis arangement must be a permutation");
            dst[axes[i]] = shape[i];
        }
        Tensor res(Device::Memory::allocateBuffer(dst));
        Device::Engine::permuteAxes(values(), res.values(), axes);
        return res;
    }
    // Tensor(stacking:along:) (Tensor/Operators/Stack.swift:79-122)
    static Tensor stacking(const std::vector<Tensor> &tensors, int axis) {
        if (axis == 0) return stacking(tensors);
        precondition(!tensors.empty(), "cannot stack zero tensors");
        precondition(axis >= 0 && axis < tensors[0].dim(), "Dimensionality of tensors must be in dimensionality range of source tensors");
        Shape s = tensors[0].shape;
        std::vector<ShapedBuffer> bufs;
        int64_t extent = 0;
        for (auto &t : tensors) {
            precondition(t.dim() == tensors[0].dim(), "All vector shapes must match except on concatenation axis.");
            for (int i = 0; i < t.dim(); ++i)
                precondition(i == axis || t.shape[i] == s[i], "All vector shapes must match except on concatenation axis.");
            extent += t.shape[axis];
            bufs.push_back(t.values());
        }
        s[axis] = extent;
        Tensor res(Device::Memory::allocateBuffer(s));
        Device::Engine::stack(bufs, res.values(), axis);
        return res;
    }
    static Tensor stacking(const std::vector<Tensor> &tensors) {
        precondition(!tensors.empty(), "cannot stack zero tensors");
        Shape s = tensors[0].shape;
        precondition(!s.empty(), "cannot stack scalars");
        std::vector<ShapedBuffer> bufs;
        int64_t rows = 0;
        for (auto &t : tensors) {
            precondition(Shape(t.shape.begin() + 1, t.shape.end()) == Shape(s.begin() + 1, s.end()),
                         "All vectors must have same shape except along the stacking axis");
            rows += t.shape[0];
            bufs.push_back(t.values());
        }
        s[0] = rows;
        Tensor res(Device::Memory::allocateBuffer(s));
        bool equal = true;
        for (auto &t : tensors) equal = equal && t.shape == tensors[0].shape;
        if (equal) Device::Engine::stack(bufs, res.values(), 0);
        else {
            int64_t off = 0;
            for (auto &t : tensors) {
                Device::Memory::assign(t.buffer(), Device::Memory::advance(res.buffer(), off), t.count());
                off += t.count();
            }
        }
        return res;
    }
    // bandMatrix (Tensor/Operators/UtilOps.swift:117-132)
    Tensor bandMatrix(std::optional<int64_t> belowDiagonal, std::optional<int64_t> aboveDiagonal) const {
        Tensor res(Device::Memory::allocateBuffer(shape));
        Device::Engine::fill(0.f, res.buffer(), res.count());
        Device::Engine::band(values(), res.values(), belowDiagonal, aboveDiagonal);
        return res;
    }

    // ---- matrix products (Tensor/Operators/Matrix.swift:35-68, :79-135)
   private:
    Tensor _matMul(const Tensor &other, bool transposeSelf, bool transposeOther) const {
        precondition(dim() == 2 && other.dim() == 2, "_matMul operands must be two dimensional");
        precondition(shape[transposeSelf ? 0 : 1] == other.shape[transposeOther ? 1 : 0], "Matrix multiplication operands must have matching shapes.");
        Tensor res(Device::Memory::allocateBuffer(Shape{shape[transposeSelf ? 1 : 0], other.shape[transposeOther ? 0 : 1]}));
        Device::Engine::gemm(values(), other.values(), res.values(), 1.f, 0.f, transposeSelf, transposeOther);
        return res;
    }

   public:
    Tensor matrixMultiplied(const Tensor &other, bool transposeSelf = false, bool transposeOther = false) const {
        precondition(dim() >= 1 && dim() <= 2 && other.dim() >= 1 && other.dim() <= 2,
                     "Matrix multiplication operands must both be one or two dimensional.");
        precondition(!(dim() == 2 && other.dim() == 2) || shape[transposeSelf ? 0 : 1] == other.shape[transposeOther ? 1 : 0],
                     "Matrix multiplication operands must have matching shapes.");
        Tensor l = dim() == 1 ? view({1, -1}) : *this;
        Tensor r = other.dim() == 1 ? other.view({-1, 1}) : other;
        Shape resultViewShape;
        if (dim() == 1 && other.dim() == 1) resultViewShape = {};
        else if (dim() == 1) resultViewShape = {other.shape[transposeOther ? 0 : 1]};
        else if (other.dim() == 1) resultViewShape = {shape[transposeSelf ? 1 : 0]};
        else resultViewShape = {shape[transposeSelf ? 1 : 0], other.shape[transposeOther ? 0 : 1]};
        return l._matMul(r, transposeSelf && dim() == 2, transposeOther && other.dim() == 2).view(resultViewShape);
    }
    Tensor broadcastMatrixMultiplied(const Tensor &other, bool transposeSelf = false, bool transposeOther = false) const {
        precondition(dim() >= 2 && other.dim() >= 2, "Operands must both be at least 2-dimensional.");
        precondition(shape[dim() - 2 + (transposeSelf ? 0 : 1)] == other.shape[other.dim() - 2 + (transposeOther ? 1 : 0)],
                     "Matmul operands must have matching shapes");
        const int d = std::max(dim(), other.dim());
        Shape ls(d - dim(), 1), rs(d - other.dim(), 1);
        ls.insert(ls.end(), shape.begin(), shape.end());
        rs.insert(rs.end(), other.shape.begin(), other.shape.end());
        Tensor lhs = view(ls), rhs = other.view(rs);
        const Shape lb(ls.begin(), ls.end() - 2), rb(rs.begin(), rs.end() - 2);
        const Shape bshape = shapeForBroadcastedOperands(lb, rb);
        Shape mm = {ls[d - 2 + (transposeSelf ? 1 : 0)], rs[d - 2 + (transposeOther ? 0 : 1)]};
        Shape full = bshape;
        full.insert(full.end(), mm.begin(), mm.end());
        const int64_t nb = count_of(bshape);

        if (Device::fused()) {
            // one strided-batched launch when each operand is either fully batched or fully shared
            const bool lfull = lb == bshape, rfull = rb == bshape;
            const bool lone = count_of(lb) == 1, rone = count_of(rb) == 1;
            if ((lfull || lone) && (rfull || rone)) {
                Tensor res(Device::Memory::allocateBuffer(full));
                Device::Engine::gemmBatched(lhs.values(), lfull ? ls[d - 2] * ls[d - 1] : 0, rhs.values(), rfull ? rs[d - 2] * rs[d - 1] : 0,
                                            res.values(), nb, transposeSelf, transposeOther);
                return res;
            }
        }
        // the reference's loop: one gemm per broadcast index into its own buffer, then stack, then view
        std::vector<Tensor> results;
        std::vector<int64_t> idx(bshape.size()), li(bshape.size()), ri(bshape.size());
        for (int64_t n = 0; n < nb; ++n) {
            int64_t rem = n;
            for (int i = (int)bshape.size() - 1; i >= 0; --i) {
                idx[i] = rem % bshape[i];
                rem /= bshape[i];
                li[i] = std::min(idx[i], ls[i] - 1);
                ri[i] = std::min(idx[i], rs[i] - 1);
            }
            results.push_back(lhs[li]._matMul(rhs[ri], transposeSelf, transposeOther));
        }
        return stacking(results).view(full);
    }
};

// ---- Tensor: Codable (Tensor/TensorExt.swift:241-271) in the form Foundation's JSONEncoder gives it: an object with
// "requiresGradient" (Bool), "shape" ([Int]) and "data" (the elements' bytes, little-endian fp32, base64 - the encoder's
// default Data strategy).  Both directions go through Device.Memory.assign, like the reference.
namespace codable {
inline std::string base64(const unsigned char *p, size_t n) {
    static const char *tbl = "ABCDEFGHIJKLMNOPQRSTUVWXYZabcdefghijklmnopqrstuvwxyz0123456789+/";
    std::string out;
    out.reserve((n + 2) / 3 * 4);
    for (size_t i = 0; i < n; i += 3) {
        const unsigned v = (p[i] << 16) | ((i + 1 < n ? p[i + 1] : 0) << 8) | (i + 2 < n ? p[i + 2] : 0);
        out += tbl[(v >> 18) & 63];
        out += tbl[(v >> 12) & 63];
        out += i + 1 < n ? tbl[(v >> 6) & 63] : '=';
        out += i + 2 < n ? tbl[v & 63] : '=';
    }
    return out;
}
inline std::vector<unsigned char> unbase64(const std::string &s) {
    auto val = [](char c) -> int {
        if (c >= 'A' && c <= 'Z') return c - 'A';
        if (c >= 'a' && c <= 'z') return c - 'a' + 26;
        if (c >= '0' && c <= '9') return c - '0' + 52;
        if (c == '+') return 62;
        if (c == '/') return 63;
        return -1;
    };
    std::vector<unsigned char> out;
    unsigned acc = 0;
    int bits = 0;
    for (char c : s) {
        if (c == '=' || c == '\\') continue;       // padding; JSON may escape '/' as "\/"
        const int v = val(c);
        precondition(v >= 0, "The data couldn't be read because it isn't in the correct format.");
        acc = (acc << 6) | (unsigned)v;
        bits += 6;
        if (bits >= 8) {
            bits -= 8;
            out.push_back((unsigned char)((acc >> bits) & 0xff));
        }
    }
    return out;
}
// position just after `"key"` and the following colon, or npos
inline size_t find_key(const std::string &json, const char *key) {
    const std::string k = std::string("\"") + key + "\"";
    size_t at = json.find(k);
    if (at == std::string::npos) return at;
    at = json.find(':', at + k.size());
    return at == std::string::npos ? at : at + 1;
}
}  // namespace codable

inline std::string encodeJSON(const Tensor &t, bool requiresGradient = false) {
    const std::vector<float> e = t.elements();
    std::string out = std::string("{\"requiresGradient\":") + (requiresGradient ? "true" : "false") + ",\"data\":\"" +
                      codable::base64(reinterpret_cast<const unsigned char *>(e.data()), e.size() * sizeof(float)) + "\",\"shape\":[";
    for (size_t i = 0; i < t.shape.size(); ++i) out += (i ? "," : "") + std::to_string(t.shape[i]);
    return out + "]}";
}

inline Tensor decodeJSON(const std::string &json, bool *requiresGradient = nullptr) {
    const char *bad = "The data couldn't be read because it is missing.";
    size_t at = codable::find_key(json, "shape");
    precondition(at != std::string::npos, bad);
    at = json.find('[', at);
    const size_t close = json.find(']', at);
    precondition(at != std::string::npos && close != std::string::npos, bad);
    Shape shape;
    for (size_t i = at + 1; i < close;) {
        while (i < close && (json[i] == ' ' || json[i] == ',' || json[i] == '\n')) ++i;
        if (i >= close) break;
        size_t used = 0;
        shape.push_back(std::stoll(json.substr(i, close - i), &used));
        precondition(shape.back() >= 0, "negative extent");
        i += used;
    }
    at = codable::find_key(json, "data");
    precondition(at != std::string::npos, bad);
    const size_t q0 = json.find('"', at), q1 = json.find('"', q0 + 1);
    precondition(q0 != std::string::npos && q1 != std::string::npos, bad);
    const std::vector<unsigned char> bytes = codable::unbase64(json.substr(q0 + 1, q1 - q0 - 1));
    precondition((int64_t)bytes.size() == count_of(shape) * (int64_t)sizeof(float), "element count does not match shape");
    if (requiresGradient) {
        at = codable::find_key(json, "requiresGradient");
        precondition(at != std::string::npos, bad);
        *requiresGradient = json.compare(json.find_first_not_of(" \n", at), 4, "true") == 0;
    }
    return Tensor(reinterpret_cast<const float *>(bytes.data()), shape);
}

inline Tensor operator*(const Tensor &l, float r) { return l * Tensor(r); }
inline Tensor operator*(float l, const Tensor &r) { return Tensor(l) * r; }
inline Tensor operator+(const Tensor &l, float r) { return l + Tensor(r); }
inline Tensor operator-(float l, const Tensor &r) { return Tensor(l) - r; }
inline Tensor operator/(const Tensor &l, float r) { return l / Tensor(r); }
inline Tensor sqrt(const Tensor &t) { return t.sqrt(); }
inline Tensor relu(const Tensor &t) { return t.rectifiedLinear(); }
inline Tensor softmax(const Tensor &t, int axis) { return t.softmax(axis); }
inline Tensor logSoftmax(const Tensor &t, int axis) { return t.logSoftmax(axis); }
inline Tensor sin(const Tensor &t) { return t.sine(); }
inline Tensor cos(const Tensor &t) { return t.cosine(); }

// ------------------------------------------------------------------------- layers
// NN/Layer/LayerNorm.swift:29-78
struct LayerNorm {
    Tensor shift, scale;
    explicit LayerNorm(const Shape &inputSize) : shift(Tensor::repeating(0.f, inputSize)), scale(Tensor::repeating(1.f, inputSize)) {}
    Tensor operator()(const Tensor &x) const { return normalize(x, nullptr); }
    // residual != nullptr: LayerNorm(x + residual) in one pass (fused mode only)
    Tensor normalize(const Tensor &x, const Tensor *residual) const {
        if (Device::fused() && scale.dim() == 1 && x.dim() >= 2 && x.shape.back() == scale.shape[0]) {
            Tensor res(Device::Memory::allocateBuffer(x.shape));
            ShapedBuffer rb;
            if (residual) rb = residual->values();
            Device::Engine::layerNorm(x.values(), residual ? &rb : nullptr, scale.values(), shift.values(), res.values());
            return res;
        }
        const Tensor in = residual ? x + *residual : x;
        std::vector<int> axes;
        for (int i = 1; i < in.dim(); ++i) axes.push_back(i);
        Shape ms(in.dim(), 1);
        ms[0] = in.shape[0];
        Tensor mean = in.reduceMean(axes).view(ms);
        Tensor variance = in.variance(axes).view(ms);
        Tensor normalized = (in - mean) / (sqrt(variance) + 1e-5f);
        return normalized * scale + shift;
    }
};

// NN/Layer/Dropout.swift:29-56: multiplies by a Bernoulli(1 - rate) mask drawn on the host; identity when inactive
struct Dropout {
    float rate;
    bool isActive = true;
    explicit Dropout(float r) : rate(r) {}
    Tensor operator()(const Tensor &x) const {
        if (!isActive) return x;
        static std::mt19937_64 rng(0);
        std::bernoulli_distribution keep(1.0 - rate);
        std::vector<float> m((size_t)x.count());
        for (auto &v : m) v = keep(rng) ? 1.f : 0.f;
        return x * Tensor(m, x.shape);
    }
};

// NN/Layer/Dense.swift:29-69
struct Dense {
    Tensor weights, bias;
    Dense(int64_t inputSize, int64_t outputSize)
        : weights(Tensor::repeating(0.f, {inputSize, outputSize})), bias(Tensor::repeating(0.f, {outputSize})) {}
    Tensor operator()(const Tensor &inputs) const { return inputs.matrixMultiplied(weights) + bias; }
    // fused mode: act(inputs . weights + bias) + residual as one product with an epilogue; inputs [..., inputSize]
    Tensor fused(const Tensor &inputs, int activation, const Tensor *residual) const {
        Shape os(inputs.shape.begin(), inputs.shape.end() - 1);
        os.push_back(weights.shape[1]);
        Tensor out(Device::Memory::allocateBuffer(os));
        const ShapedBuffer bb = bias.values();
        ShapedBuffer rb;
        if (residual) rb = residual->values();
        Device::Engine::denseFused(inputs.values(), weights.values(), &bb, activation, residual ? &rb : nullptr, out.values());
        return out;
    }
};

// A mask whose structure the caller knows - the two families TransformerUtil.swift:29-50 builds: keys at or beyond each
// sequence's length blocked, optionally together with the causal triangle.  In fused mode the model-level layers hand it
// to the attention kernel as a descriptor instead of materialising the dense tensor: the same bits as the dense mask
// it stands for, and key tiles it blocks entirely are not visited (exact because activations are finite and every row
// keeps at least its first key; a sequence of length 0 - all keys blocked, uniform weights - is computed in full).
struct AttentionMask {
    int kind = DL4S_MASK_NONE;
    Tensor lengths;   // device int32 [batchSize], viewed through a float buffer of the same byte size
    // keyCount: the padded length of the keys.  When no sequence is shorter the mask blocks nothing by length and the
    // descriptor needs no lengths on the device (the kernels give the same bits for either description of a mask).
    static AttentionMask forLengths(const std::vector<int64_t> &sequenceLengths, bool causal, int64_t keyCount) {
        AttentionMask m;
        bool allFull = true;
        for (int64_t v : sequenceLengths) allFull = allFull && v >= keyCount;
        if (allFull) {
            m.kind = causal ? DL4S_MASK_CAUSAL : DL4S_MASK_NONE;
            return m;
        }
        m.kind = causal ? DL4S_MASK_CAUSAL_OR_KEY_LENGTHS : DL4S_MASK_KEY_LENGTHS;
        std::vector<int32_t> l32(sequenceLengths.begin(), sequenceLengths.end());
        for (int32_t v : l32) precondition(v >= 0, "sequence lengths must not be negative");
        m.lengths = Tensor(Device::Memory::allocateBuffer(Shape{(int64_t)l32.size()}));
        Device::check(dl4s_hip_assign_h2d(Device::context(), m.lengths.buffer().memory, l32.data(), l32.size() * sizeof(int32_t)));
        return m;
    }
    const int32_t *lengthsPointer() const {
        const bool needed = kind == DL4S_MASK_KEY_LENGTHS || kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS;
        return needed ? reinterpret_cast<const int32_t *>(lengths.buffer().memory) : nullptr;
    }
};

// NN/Models/Transformer/ScaledDotProductAttention.swift:29-65
struct ScaledDotProductAttention {
    float temperature;
    explicit ScaledDotProductAttention(float t) : temperature(t) {}
    Tensor operator()(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *mask) const {
        precondition(k.dim() == 4, "k must have 4 dimensions");
        if (Device::fused() || Device::attentionHook()) {
            precondition(q.dim() == 4 && v.dim() == 4 && q.shape[0] == k.shape[0] && q.shape[1] == k.shape[1] &&
                             v.shape[0] == k.shape[0] && v.shape[1] == k.shape[1] && q.shape[3] == k.shape[3] && k.shape[2] == v.shape[2],
                         "Matmul operands must have matching shapes");
            Tensor out(Device::Memory::allocateBuffer(Shape{q.shape[0], q.shape[1], q.shape[2], v.shape[3]}));
            ShapedBuffer mb;
            if (mask) mb = mask->values();
            // the mask is looked at once per mask tensor (as the Swift hook does through its table of mask buffers)
            const dl4s_mask_desc *prepared = mask ? mask->attentionMask(q.shape[0], q.shape[1], q.shape[2], k.shape[2]) : nullptr;
            Device::Engine::fusedAttention(q.values(), k.values(), v.values(), mask ? &mb : nullptr, out.values(), temperature, false, prepared);
            return out;
        }
        Tensor attn = (q / Tensor(temperature)).broadcastMatrixMultiplied(k, false, true);
        if (mask) attn = attn - *mask * 1e9f;
        attn = softmax(attn, 3);
        return attn.broadcastMatrixMultiplied(v);
    }
};

// NN/Models/Transformer/MultiHeadAttention.swift:29-128
struct MultiHeadAttention {
    int64_t heads, keyDim, valueDim, hiddenDim;
    ScaledDotProductAttention attn;
    Tensor qDense, kDense, vDense, fc;
    LayerNorm norm;
    Dropout dropout;
    // Not in the reference.  false: the reference's normalisation, over (length, hidden) jointly, because the layer hands
    // LayerNorm a 3-D tensor (MultiHeadAttention.swift:123-124, LayerNorm.swift:62-77).  true: every token normalised by
    // itself (the input viewed as [batch * length, hidden], as PointwiseFeedForward.swift:68 does) - the conventional
    // Transformer, whose output at a position does not depend on later positions, which cached decoding needs.
    bool normalizesPerToken = false;
    Tensor normalized(const Tensor &x, const Tensor *residual) const {
        if (!normalizesPerToken || x.dim() != 3) return norm.normalize(x, residual);
        const Shape flat{x.shape[0] * x.shape[1], x.shape[2]};
        if (!residual) return norm.normalize(x.view(flat), nullptr).view(x.shape);
        const Tensor r = residual->view(flat);
        return norm.normalize(x.view(flat), &r).view(x.shape);
    }
    MultiHeadAttention(int64_t heads_, int64_t hiddenDim_, int64_t keyDim_, int64_t valueDim_, float dropoutRate = 0.1f)
        : heads(heads_), keyDim(keyDim_), valueDim(valueDim_), hiddenDim(hiddenDim_), attn(std::sqrt((float)keyDim_)),
          qDense(Tensor::repeating(0.f, {hiddenDim_, keyDim_ * heads_})), kDense(Tensor::repeating(0.f, {hiddenDim_, keyDim_ * heads_})),
          vDense(Tensor::repeating(0.f, {hiddenDim_, valueDim_ * heads_})), fc(Tensor::repeating(0.f, {valueDim_ * heads_, hiddenDim_})),
          norm(Shape{hiddenDim_}), dropout(dropoutRate) {}
    // fused mode, equal head dims that are a multiple of 4 up to 256 (what the token-major attention kernels take): the
    // key / value projections alone, [B,L,H,d], for callers that attend to the same keys and values repeatedly (the
    // encoder states during greedy decoding)
    bool canCacheProjections() const { return Device::fused() && keyDim == valueDim && keyDim <= 256 && keyDim % 4 == 0; }
    // The projections are separate products in the reference (MultiHeadAttention.swift:105-107); the key and value ones
    // (and the query one, when all three inputs have one length) go out as one grouped launch.
    std::pair<Tensor, Tensor> projectKeysValues(const Tensor &k, const Tensor &v, const Tensor *q = nullptr, Tensor *qp = nullptr) const {
        precondition(canCacheProjections() && k.dim() == 3 && v.dim() == 3 && k.shape[1] == v.shape[1], "Matmul operands must have matching shapes");
        const int64_t B = k.shape[0], L = k.shape[1];
        precondition(k.shape[2] == hiddenDim && v.shape[2] == hiddenDim && k.shape[0] == v.shape[0], "Matmul operands must have matching shapes");
        Tensor kp(Device::Memory::allocateBuffer(Shape{B, L, heads, keyDim})), vp(Device::Memory::allocateBuffer(Shape{B, L, heads, valueDim}));
        std::vector<ShapedBuffer> lhs{k.values(), v.values()}, rhs{kDense.values(), vDense.values()}, res{kp.values(), vp.values()};
        if (q && qp && q->shape == k.shape) {
            *qp = Tensor(Device::Memory::allocateBuffer(Shape{B, L, heads, keyDim}));
            lhs.push_back(q->values());
            rhs.push_back(qDense.values());
            res.push_back(qp->values());
        }
        Device::Engine::gemmGrouped(lhs, B * L, rhs, res);
        return {kp, vp};
    }
    Tensor attendProjected(const Tensor &q, const Tensor &kp, const Tensor &vp, const Tensor *mask,
                           const AttentionMask *structured = nullptr, const Tensor *qProjected = nullptr) const {
        precondition(canCacheProjections() && q.dim() == 3 && kp.dim() == 4 && vp.dim() == 4, "Matmul operands must have matching shapes");
        const int64_t batchSize = q.shape[0], queryCount = q.shape[1];
        Tensor qp = qProjected ? *qProjected
                               : q.view({batchSize * queryCount, hiddenDim}).matrixMultiplied(qDense).view({batchSize, queryCount, heads, keyDim});
        Tensor a(Device::Memory::allocateBuffer(Shape{batchSize, queryCount, heads, valueDim}));
        ShapedBuffer mb;
        if (mask) mb = mask->values();
        if (structured)
            Device::Engine::fusedAttentionStructured(qp.values(), kp.values(), vp.values(), structured->kind, structured->lengthsPointer(),
                                                     a.values(), attn.temperature, true);
        else
            Device::Engine::fusedAttention(qp.values(), kp.values(), vp.values(), mask ? &mb : nullptr, a.values(), attn.temperature, true,
                                           mask ? mask->attentionMask(batchSize, heads, queryCount, kp.shape[1]) : nullptr);
        Tensor a2 = a.view({batchSize * queryCount, heads * valueDim});
        if (!dropout.isActive) {
            // the fc product, `+ res` and the normalisation (MultiHeadAttention.swift:119-124) as one call: the product's
            // epilogue leaves the sums the LayerNorm needs
            Tensor sum(Device::Memory::allocateBuffer(Shape{batchSize, queryCount, hiddenDim}));
            const ShapedBuffer rb = q.values();
            Device::Engine::denseFusedLayerNorm(a2.values(), fc.values(), nullptr, DL4S_ACT_NONE, &rb, normalizesPerToken ? 1 : queryCount,
                                                norm.scale.values(), norm.shift.values(), sum.values());
            return sum;
        }
        Tensor out_drop = dropout(a2.matrixMultiplied(fc).view({batchSize, queryCount, hiddenDim}));
        return normalized(out_drop, &q);
    }
    // ---- one new position against cached keys and values (no counterpart in the reference; fused mode, head dims
    // that are multiples of 4 up to 256, dropout inactive).  x [B,1,hidden].  With a single position the joint normalisation and the per-token one coincide.
    bool canDecodeIncrementally() const { return canCacheProjections() && !dropout.isActive; }
    Tensor finishStep(const Tensor &x, const Tensor &attended) const {
        const int64_t B = x.shape[0];
        Tensor sum(Device::Memory::allocateBuffer(Shape{B, 1, hiddenDim}));
        const ShapedBuffer rb = x.values();
        Device::Engine::denseFused(attended.view({B, heads * valueDim}).values(), fc.values(), nullptr, DL4S_ACT_NONE, &rb, sum.values());
        return norm.normalize(sum, nullptr);
    }
    // self-attention: projects x, writes its key / value row into row `position` of the caches [B,H,capacity,d], attends
    // to rows 0 ... position
    // (positionOnDevice != nullptr: the row index is read from device memory instead, see Transformer::greedyCached)
    Tensor stepAppending(const Tensor &x, const Tensor &keyCache, const Tensor &valueCache, int64_t position,
                         const int32_t *positionOnDevice = nullptr) const {
        precondition(canDecodeIncrementally() && x.dim() == 3 && x.shape[1] == 1 && x.shape[2] == hiddenDim && keyCache.dim() == 4 &&
                         keyCache.shape == valueCache.shape && keyCache.shape[0] == x.shape[0] && keyCache.shape[1] == heads &&
                         (positionOnDevice || (position >= 0 && position < keyCache.shape[2])),
                     "cached attention step: bad shapes");
        const int64_t B = x.shape[0];
        const Shape ps{B, heads, 1, keyDim};
        Tensor qp(Device::Memory::allocateBuffer(ps)), kp(Device::Memory::allocateBuffer(ps)), vp(Device::Memory::allocateBuffer(ps));
        Device::Engine::gemmGrouped({x.values(), x.values(), x.values()}, B, {qDense.values(), kDense.values(), vDense.values()},
                                    {qp.values(), kp.values(), vp.values()});
        Tensor a(Device::Memory::allocateBuffer(ps));
        if (positionOnDevice)
            Device::Engine::decodeAttentionAppendingAt(qp.values(), keyCache.values(), valueCache.values(), kp.values(), vp.values(),
                                                       positionOnDevice, a.values(), attn.temperature);
        else
            Device::Engine::decodeAttentionAppending(qp.values(), keyCache.values(), valueCache.values(), kp.values(), vp.values(), position,
                                                     a.values(), attn.temperature);
        return finishStep(x, a);
    }
    // attention to `rows` cached rows that do not change (the projected encoder states, head-major [B,H,rows,d])
    Tensor stepAttending(const Tensor &x, const Tensor &keys, const Tensor &values) const {
        precondition(canDecodeIncrementally() && x.dim() == 3 && x.shape[1] == 1 && x.shape[2] == hiddenDim && keys.dim() == 4 &&
                         keys.shape == values.shape && keys.shape[0] == x.shape[0] && keys.shape[1] == heads && keys.shape[2] >= 1,
                     "cached attention step: bad shapes");
        const int64_t B = x.shape[0];
        Tensor qp = x.view({B, hiddenDim}).matrixMultiplied(qDense);
        Tensor a(Device::Memory::allocateBuffer(Shape{B, heads, 1, keyDim}));
        Device::Engine::decodeAttention(qp.values(), keys.values(), values.values(), keys.shape[2], a.values(), attn.temperature);
        return finishStep(x, a);
    }
    // self- or cross-attention with a structured mask (fused mode, head dims as for canCacheProjections)
    Tensor structured(const Tensor &q, const Tensor &k, const Tensor &v, const AttentionMask &mask) const {
        Tensor qp;
        auto kv = projectKeysValues(k, v, &q, &qp);
        return attendProjected(q, kv.first, kv.second, nullptr, &mask, qp.dim() ? &qp : nullptr);
    }
    Tensor operator()(const Tensor &q, const Tensor &k, const Tensor &v, const Tensor *mask) const {
        const int64_t batchSize = q.shape[0], queryCount = q.shape[1], keyCount = k.shape[1], valueCount = v.shape[1];
        const Tensor &res = q;
        if (canCacheProjections()) {
            precondition(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && keyCount == valueCount, "Matmul operands must have matching shapes");
            Tensor qp;
            auto kv = projectKeysValues(k, v, &q, &qp);
            return attendProjected(q, kv.first, kv.second, mask, nullptr, qp.dim() ? &qp : nullptr);
        }
        Tensor q_prep = q.broadcastMatrixMultiplied(qDense).view({batchSize, queryCount, heads, keyDim});
        Tensor k_prep = k.broadcastMatrixMultiplied(kDense).view({batchSize, keyCount, heads, keyDim});
        Tensor v_prep = v.broadcastMatrixMultiplied(vDense).view({batchSize, valueCount, heads, valueDim});
        Tensor q_trans = q_prep.permuted({0, 2, 1, 3});
        Tensor k_trans = k_prep.permuted({0, 2, 1, 3});
        Tensor v_trans = v_prep.permuted({0, 2, 1, 3});
        Tensor q_attn = attn(q_trans, k_trans, v_trans, mask);
        Tensor out = q_attn.permuted({0, 2, 1, 3}).view({batchSize, queryCount, -1}).broadcastMatrixMultiplied(fc);
        Tensor out_drop = dropout(out);
        if (Device::fused()) return normalized(out_drop, &res);
        Tensor q_res = out_drop + res;
        return normalized(q_res, nullptr);
    }
};

// NN/Models/Transformer/PointwiseFeedForward.swift:32-83
struct PointwiseFeedForward {
    Dense dense1, dense2;
    LayerNorm norm;
    Dropout dropout;
    PointwiseFeedForward(int64_t size, int64_t hiddenSize, float dropoutRate)
        : dense1(size, hiddenSize), dense2(hiddenSize, size), norm(Shape{size}), dropout(dropoutRate) {}
    Tensor operator()(const Tensor &inputs) const {
        const int64_t batchSize = inputs.shape[0], seqlen = inputs.shape[1], size = inputs.shape[2];
        Tensor denseInputs = inputs.view({batchSize * seqlen, size});
        if (Device::fused()) {
            Tensor h = dense1.fused(denseInputs, DL4S_ACT_GELU, nullptr);
            if (!dropout.isActive) return norm.normalize(dense2.fused(h, DL4S_ACT_NONE, &denseInputs), nullptr).view({batchSize, seqlen, size});
            Tensor tmp4 = dropout(dense2.fused(h, DL4S_ACT_NONE, nullptr));
            return norm.normalize(tmp4, &denseInputs).view({batchSize, seqlen, size});
        }
        Tensor tmp1 = dense1(denseInputs);
        Tensor tmp2 = tmp1.gaussianErrorLinear();
        Tensor tmp3 = dense2(tmp2);
        Tensor tmp4 = dropout(tmp3);
        Tensor n = norm(tmp4 + denseInputs);
        return n.view({batchSize, seqlen, size});
    }
};

// NN/Models/Transformer/TransformerEncoderBlock.swift:29-66
struct TransformerEncoderBlock {
    MultiHeadAttention selfAttention;
    PointwiseFeedForward pointwiseFeedForward;
    TransformerEncoderBlock(int64_t hiddenDim, int64_t forwardDim, int64_t heads, int64_t keyDim, int64_t valueDim, float dropoutRate)
        : selfAttention(heads, hiddenDim, keyDim, valueDim, dropoutRate), pointwiseFeedForward(hiddenDim, forwardDim, dropoutRate) {}
    Tensor operator()(const Tensor &inputs, const Tensor &mask) const {
        Tensor attn = selfAttention(inputs, inputs, inputs, &mask);
        return pointwiseFeedForward(attn);
    }
    Tensor operator()(const Tensor &inputs, const AttentionMask &mask) const {
        return pointwiseFeedForward(selfAttention.structured(inputs, inputs, inputs, mask));
    }
};

// NN/Models/Transformer/TransformerDecoderBlock.swift:29-69
struct TransformerDecoderBlock {
    MultiHeadAttention selfAttention, encoderAttention;
    PointwiseFeedForward pointwiseFeedForward;
    TransformerDecoderBlock(int64_t hiddenDim, int64_t forwardDim, int64_t heads, int64_t keyDim, int64_t valueDim, float dropoutRate)
        : selfAttention(heads, hiddenDim, keyDim, valueDim, dropoutRate), encoderAttention(heads, hiddenDim, keyDim, valueDim, dropoutRate),
          pointwiseFeedForward(hiddenDim, forwardDim, dropoutRate) {}
    Tensor operator()(const Tensor &decoderInput, const Tensor &encoderOutput, const Tensor &encoderMask, const Tensor &decoderMask) const {
        Tensor decAttn = selfAttention(decoderInput, decoderInput, decoderInput, &decoderMask);
        Tensor encAttn = encoderAttention(decAttn, encoderOutput, encoderOutput, &encoderMask);
        return pointwiseFeedForward(encAttn);
    }    // the same block with the encoder-side key / value projections computed once by the caller
    // (encoderAttention.projectKeysValues(encoderOutput, encoderOutput)): they do not depend on the decoder input
    Tensor withProjectedEncoder(const Tensor &decoderInput, const Tensor &encKeys, const Tensor &encValues, const Tensor &encoderMask,
                                const Tensor &decoderMask) const {
        Tensor decAttn = selfAttention(decoderInput, decoderInput, decoderInput, &decoderMask);
        Tensor encAttn = encoderAttention.attendProjected(decAttn, encKeys, encValues, &encoderMask);
        return pointwiseFeedForward(encAttn);
    }
    // one new position: decoderInput [B,1,hidden], self-attention caches [B,H,capacity,d], encoder keys / values [B,H,n,d]
    Tensor step(const Tensor &decoderInput, const Tensor &keyCache, const Tensor &valueCache, int64_t position, const Tensor &encKeys,
                const Tensor &encValues, const int32_t *positionOnDevice = nullptr) const {
        Tensor decAttn = selfAttention.stepAppending(decoderInput, keyCache, valueCache, position, positionOnDevice);
        Tensor encAttn = encoderAttention.stepAttending(decAttn, encKeys, encValues);
        return pointwiseFeedForward(encAttn);
    }
    Tensor withProjectedEncoder(const Tensor &decoderInput, const Tensor &encKeys, const Tensor &encValues, const AttentionMask &encoderMask,
                                const AttentionMask &decoderMask) const {
        Tensor decAttn = selfAttention.structured(decoderInput, decoderInput, decoderInput, decoderMask);
        Tensor encAttn = encoderAttention.attendProjected(decAttn, encKeys, encValues, nullptr, &encoderMask);
        return pointwiseFeedForward(encAttn);
    }
};

// NN/Models/Transformer/TransformerUtil.swift:29-36
inline Tensor makeEncoderMasks(const std::vector<int64_t> &sequenceLengths) {
    const int64_t maxInLen = sequenceLengths.empty() ? 0 : *std::max_element(sequenceLengths.begin(), sequenceLengths.end());
    const int64_t batchSize = (int64_t)sequenceLengths.size();
    std::vector<float> m((size_t)(batchSize * maxInLen));
    for (int64_t b = 0; b < batchSize; ++b)
        for (int64_t j = 0; j < maxInLen; ++j) m[b * maxInLen + j] = j < sequenceLengths[b] ? 0.f : 1.f;
    return Tensor(m, {batchSize, maxInLen}).view({batchSize, 1, 1, maxInLen});
}

// NN/Models/Transformer/TransformerUtil.swift:38-50
inline Tensor makeDecoderMasks(const std::vector<int64_t> &sequenceLengths) {
    const int64_t batchSize = (int64_t)sequenceLengths.size();
    const int64_t maxLen = sequenceLengths.empty() ? 0 : *std::max_element(sequenceLengths.begin(), sequenceLengths.end());
    std::vector<float> m((size_t)(batchSize * maxLen));
    for (int64_t b = 0; b < batchSize; ++b)
        for (int64_t j = 0; j < maxLen; ++j) m[b * maxLen + j] = j < sequenceLengths[b] ? 0.f : 1.f;
    Tensor decoderSeqMask(m, {batchSize, maxLen});
    Tensor decoderCausalMask = Tensor::repeating(1.f, {maxLen, maxLen}).bandMatrix(-1, std::nullopt);
    return 1.f - relu(1.f - decoderSeqMask.view({batchSize, 1, 1, maxLen}) - decoderCausalMask);
}

// ------------------------------------------------------------------------- the model wrapper
// NN/Layer/Embedding.swift:29-166 (forward only): row `token` of the embedding matrix, a row of zeros for ignoreIndex
struct Embedding {
    Tensor embeddingMatrix;   // [inputFeatures, outputSize]
    int32_t ignoreIndex;
    Embedding(int64_t inputFeatures, int64_t outputSize, int32_t ignoreIndex_ = -1)
        : embeddingMatrix(Tensor::repeating(0.f, {inputFeatures, outputSize})), ignoreIndex(ignoreIndex_) {}
    int64_t outputSize() const { return embeddingMatrix.shape[1]; }
    // device copy of host tokens (Tensor<Int32, Device> in the reference)
    static Tensor uploadTokens(const std::vector<int32_t> &tokens) {
        Tensor t(Device::Memory::allocateBuffer(Shape{(int64_t)tokens.size()}));
        Device::check(dl4s_hip_assign_h2d(Device::context(), t.buffer().memory, tokens.data(), tokens.size() * sizeof(int32_t)));
        return t;
    }
    Tensor operator()(const std::vector<int32_t> &inputs) const {
        for (int32_t idx : inputs)
            precondition(idx == ignoreIndex || (idx >= 0 && idx < embeddingMatrix.shape[0]), "index out of bounds");
        if (Device::fused()) {
            Tensor tok = uploadTokens(inputs);
            Tensor res(Device::Memory::allocateBuffer(Shape{(int64_t)inputs.size(), outputSize()}));
            Device::Engine::embedPositions(embeddingMatrix.values(), reinterpret_cast<const int32_t *>(tok.buffer().memory), 1,
                                           (int64_t)inputs.size(), ignoreIndex, nullptr, nullptr, res.values());
            return res;
        }
        std::vector<Tensor> embedded;
        for (int32_t idx : inputs) {
            if (idx == ignoreIndex) embedded.push_back(Tensor::repeating(0.f, {1, outputSize()}));
            else embedded.push_back(embeddingMatrix[{(int64_t)idx}].unsqueezed(0));
        }
        return Tensor::stacking(embedded, 0);
    }
};

// NN/Models/Transformer/PositionalEncoding.swift:33-71
struct PositionalEncoding {
    int64_t hiddenSize;
    explicit PositionalEncoding(int64_t hiddenSize_) : hiddenSize(hiddenSize_) {
        precondition(hiddenSize % 2 == 0, "Hidden size must be multiple of 2");
    }
    Tensor operator()(int64_t maxLen) const {
        std::vector<float> ir((size_t)maxLen), hr((size_t)(hiddenSize / 2));
        std::iota(ir.begin(), ir.end(), 0.f);
        std::iota(hr.begin(), hr.end(), 0.f);
        Tensor inputRange(ir, {maxLen}), hiddenRange(hr, {hiddenSize / 2});
        Tensor frequencies = Tensor(10000.f).raised(hiddenRange / Tensor((float)(hiddenSize / 2)));
        Tensor samplePoints = inputRange.unsqueezed(1) / frequencies.unsqueezed(0);   // [seqlen, hiddenSize / 2]
        return Tensor::stacking({sin(samplePoints).unsqueezed(2), cos(samplePoints).unsqueezed(2)}, 2).view({-1, hiddenSize});
    }
};

// NN/Models/Transformer/TransformerEncoder.swift:29-72
struct TransformerEncoder {
    std::vector<TransformerEncoderBlock> encoderLayers;
    TransformerEncoder(int64_t layerCount, int64_t heads, int64_t keyDim, int64_t valueDim, int64_t modelDim, int64_t forwardDim, float dropout) {
        for (int64_t i = 0; i < layerCount; ++i) encoderLayers.emplace_back(modelDim, forwardDim, heads, keyDim, valueDim, dropout);
    }
    bool canUseStructuredMasks() const {
        for (auto &l : encoderLayers)
            if (!l.selfAttention.canCacheProjections()) return false;
        return !encoderLayers.empty();
    }
    Tensor operator()(const Tensor &input, const std::vector<int64_t> &sequenceLengths) const {
        Tensor acc = input;
        if (canUseStructuredMasks()) {      // fused mode: the mask as a descriptor, never materialised
            const AttentionMask mask = AttentionMask::forLengths(sequenceLengths, false, input.shape[1]);
            for (auto &layer : encoderLayers) acc = layer(acc, mask);
            return acc;
        }
        const Tensor mask = makeEncoderMasks(sequenceLengths);
        for (auto &layer : encoderLayers) acc = layer(acc, mask);
        return acc;
    }
};

// NN/Models/Transformer/TransformerDecoder.swift:29-63
struct TransformerDecoder {
    std::vector<TransformerDecoderBlock> decoderLayers;
    TransformerDecoder(int64_t layerCount, int64_t heads, int64_t keyDim, int64_t valueDim, int64_t modelDim, int64_t forwardDim, float dropout) {
        for (int64_t i = 0; i < layerCount; ++i) decoderLayers.emplace_back(modelDim, forwardDim, heads, keyDim, valueDim, dropout);
    }
    Tensor operator()(const Tensor &decoderInput, const Tensor &encoderStates, const std::vector<int64_t> &encoderInputLengths,
                      const std::vector<int64_t> &decoderInputLengths) const {
        if (canCacheEncoderProjections())   // fused mode, head dims the MFMA kernels take: structured masks, encoder projections per call
            return withProjectedEncoder(decoderInput, projectEncoderStates(encoderStates), encoderInputLengths, decoderInputLengths);
        const Tensor encoderMask = makeEncoderMasks(encoderInputLengths);
        const Tensor decoderMask = makeDecoderMasks(decoderInputLengths);
        Tensor acc = decoderInput;
        for (auto &layer : decoderLayers) acc = layer(acc, encoderStates, encoderMask, decoderMask);
        return acc;
    }
    // Encoder-side key / value projections of every layer, computed once per encoded sequence (fused mode, head dims the MFMA kernels take)
    bool canCacheEncoderProjections() const {
        for (auto &l : decoderLayers)
            if (!l.encoderAttention.canCacheProjections() || !l.selfAttention.canCacheProjections()) return false;
        return !decoderLayers.empty();
    }
    std::vector<std::pair<Tensor, Tensor>> projectEncoderStates(const Tensor &encoderStates) const {
        std::vector<std::pair<Tensor, Tensor>> kv;
        for (auto &l : decoderLayers) kv.push_back(l.encoderAttention.projectKeysValues(encoderStates, encoderStates));
        return kv;
    }
    Tensor withProjectedEncoder(const Tensor &decoderInput, const std::vector<std::pair<Tensor, Tensor>> &kv,
                                const std::vector<int64_t> &encoderInputLengths, const std::vector<int64_t> &decoderInputLengths) const {
        precondition(!kv.empty() && kv.size() == decoderLayers.size(), "one projected key / value pair per decoder layer");
        const AttentionMask encoderMask = AttentionMask::forLengths(encoderInputLengths, false, kv[0].first.shape[1]);
        const AttentionMask decoderMask = AttentionMask::forLengths(decoderInputLengths, true, decoderInput.shape[1]);
        Tensor acc = decoderInput;
        for (size_t i = 0; i < decoderLayers.size(); ++i)
            acc = decoderLayers[i].withProjectedEncoder(acc, kv[i].first, kv[i].second, encoderMask, decoderMask);
        return acc;
    }
};

// NN/Models/Transformer/Transformer.swift:29-138
struct Transformer {
    Embedding embedding;
    PositionalEncoding positionalEncoding;
    Dropout dropout;
    TransformerEncoder encoder;
    TransformerDecoder decoder;
    Tensor outputBias;
    Transformer(int64_t encoderLayers, int64_t decoderLayers, int64_t vocabSize, int64_t hiddenDim, int64_t heads, int64_t keyDim,
                int64_t valueDim, int64_t forwardDim, float dropoutRate = 0.1f)
        : embedding(vocabSize, hiddenDim, -1), positionalEncoding(hiddenDim), dropout(dropoutRate),
          encoder(encoderLayers, heads, keyDim, valueDim, hiddenDim, forwardDim, dropoutRate),
          decoder(decoderLayers, heads, keyDim, valueDim, hiddenDim, forwardDim, dropoutRate),
          outputBias(Tensor::repeating(0.f, {vocabSize})) {}

    // inputs: [batchSize][maxLen] tokens, -1 = padding                                   (Transformer.swift:86-92)
    // positions: optional precomputed encoding with at least maxLen rows (row l does not depend on the length)
    Tensor prepareInputs(const std::vector<int32_t> &inputs, int64_t batchSize, int64_t maxLen, const Tensor *positions = nullptr) const {
        precondition((int64_t)inputs.size() == batchSize * maxLen, "element count does not match shape");
        const int64_t D = embedding.outputSize();
        precondition(!positions || (Device::fused() && positions->shape[0] >= maxLen), "bad positions");
        const Tensor encoderPositions = positions ? *positions : positionalEncoding(maxLen);          // [maxLen, embedDim]
        const float scale = std::sqrt((float)D);
        if (Device::fused()) {
            for (int32_t idx : inputs)
                precondition(idx == -1 || (idx >= 0 && idx < embedding.embeddingMatrix.shape[0]), "index out of bounds");
            Tensor tok = Embedding::uploadTokens(inputs);
            Tensor res(Device::Memory::allocateBuffer(Shape{batchSize, maxLen, D}));
            const ShapedBuffer pb = encoderPositions.values();
            Device::Engine::embedPositions(embedding.embeddingMatrix.values(), reinterpret_cast<const int32_t *>(tok.buffer().memory),
                                           batchSize, maxLen, embedding.ignoreIndex, &scale, &pb, res.values());
            return dropout(res);
        }
        Tensor embedded = embedding(inputs).view({batchSize, maxLen, -1});
        return dropout(embedded * Tensor(scale) + encoderPositions);
    }

    // log-softmax distributions [batchSize, decLen, vocab]                               (Transformer.swift:101-115)
    Tensor operator()(const std::vector<int32_t> &encoderInput, int64_t encLen, const std::vector<int32_t> &decoderInput, int64_t decLen,
                      const std::vector<int64_t> &encInLens, const std::vector<int64_t> &decInLens) const {
        const int64_t batchSize = (int64_t)encInLens.size();
        Tensor encoderStates = encoder(prepareInputs(encoderInput, batchSize, encLen), encInLens);
        Tensor decoded = decoder(prepareInputs(decoderInput, batchSize, decLen), encoderStates, encInLens, decInLens);
        Tensor deembedded = decoded.broadcastMatrixMultiplied(embedding.embeddingMatrix, false, true) + outputBias;
        return logSoftmax(deembedded, 2);
    }

    // every attention layer normalised per token (see MultiHeadAttention::normalizesPerToken; not in the reference)
    void setNormalizesPerToken(bool perToken) {
        for (auto &l : encoder.encoderLayers) l.selfAttention.normalizesPerToken = perToken;
        for (auto &l : decoder.decoderLayers) l.selfAttention.normalizesPerToken = l.encoderAttention.normalizesPerToken = perToken;
    }
    bool canDecodeIncrementally() const {
        if (!Device::fused() || decoder.decoderLayers.empty() || dropout.isActive) return false;
        for (auto &l : decoder.decoderLayers)
            if (!l.selfAttention.normalizesPerToken || !l.encoderAttention.normalizesPerToken || !l.selfAttention.canDecodeIncrementally() ||
                !l.encoderAttention.canDecodeIncrementally() || l.pointwiseFeedForward.dropout.isActive)
                return false;
        return true;
    }

    // Greedy decoding with key / value caches: no counterpart in the reference, which re-runs the whole prefix at every
    // step (greedy() below).  A step runs the decoder on the one new position: every layer appends the position's
    // self-attention key / value row to its cache [1,H,maxLength,d] and attends to the rows so far, then to the encoder
    // states' keys / values, projected once and stored head-major [1,H,n,d].  Only a model whose attention layers
    // normalise per token computes the same function this way (the prefix re-run of such a model gives the same tokens and
    // the same logits up to summation order): with the reference's joint normalisation every earlier position's output
    // changes as the prefix grows, and the precondition refuses the model.
    std::vector<int32_t> greedyCached(const std::vector<int32_t> &inputSequence, int32_t startToken, int32_t endToken, int64_t maxLength,
                                      std::vector<float> *lastLogits = nullptr, bool recorded = true) const {
        precondition(canDecodeIncrementally(),
                     "cached decoding needs fused mode, inactive dropout, equal key and value dims that are a multiple of 4 up to 256, and attention layers that normalise per token");
        const int64_t n = (int64_t)inputSequence.size(), D = embedding.outputSize(), vocab = embedding.embeddingMatrix.shape[0];
        precondition(startToken >= 0 && startToken < vocab, "index out of bounds");
        std::vector<int32_t> tokens;
        if (maxLength <= 0) return tokens;
        Tensor encoded = encoder(prepareInputs(inputSequence, 1, n), {n});
        struct LayerState { Tensor encKeys, encValues, keyCache, valueCache; };
        std::vector<LayerState> state;
        for (auto &l : decoder.decoderLayers) {
            auto kv = l.encoderAttention.projectKeysValues(encoded, encoded);                       // [1,n,H,d]
            const Shape cache{1, l.selfAttention.heads, maxLength, l.selfAttention.keyDim};
            state.push_back({kv.first.permuted({0, 2, 1, 3}), kv.second.permuted({0, 2, 1, 3}),    // [1,H,n,d]
                             Tensor(Device::Memory::allocateBuffer(cache)), Tensor(Device::Memory::allocateBuffer(cache))});
        }
        const Tensor positions = positionalEncoding(maxLength);
        const float scale = std::sqrt((float)D);
        Tensor logits(Device::Memory::allocateBuffer(Shape{1, vocab}));
        // The step's token and position live in device memory (two int32 in a float buffer of the same size): the calls of a
        // step are then the same at every position, and are recorded once and replayed (about 80 launches per token at
        // about 2 us each instead of 3 us issued one by one).
        Tensor cursor(Device::Memory::allocateBuffer(Shape{2}));
        int32_t *token = reinterpret_cast<int32_t *>(cursor.buffer().memory), *position = token + 1;
        const int32_t first[2] = {startToken, 0};
        Device::check(dl4s_hip_assign_h2d(Device::context(), token, first, sizeof(first)));
        auto step = [&] {
            Tensor acc(Device::Memory::allocateBuffer(Shape{1, 1, D}));
            Device::Engine::embedAt(embedding.embeddingMatrix.values(), token, &scale, positions.values(), position, acc.values());
            for (size_t i = 0; i < state.size(); ++i)
                acc = decoder.decoderLayers[i].step(acc, state[i].keyCache, state[i].valueCache, -1, state[i].encKeys, state[i].encValues,
                                                    position);
            Device::Engine::gemm(acc.view({1, D}).values(), embedding.embeddingMatrix.values(), logits.values(), 1.0f, 0.0f, false, true);
            Device::Engine::argmaxTo(logits.values(), token, position);
        };
        RecordedCalls replayable;
        // recording and instantiating the step costs a few eager steps: not for short decodes
        const bool replay = recorded && maxLength >= 16 && dl4s_hip_graph_supported();
        for (int64_t i = 0; i < maxLength; ++i) {
            if (i == 0 || !replay) {
                step();                       // the first step also sizes the library's scratch block
            } else {
                if (!replayable) replayable.record(step);
                replayable.replay();
            }
            int32_t chosen = 0;
            Device::check(dl4s_hip_assign_d2h(Device::context(), &chosen, token, sizeof(chosen)));
            if (lastLogits) {
                const std::vector<float> row = logits.elements();
                lastLogits->insert(lastLogits->end(), row.begin(), row.end());
            }
            tokens.push_back(chosen);
            if (chosen == endToken) break;
        }
        return tokens;
    }

    // greedy decoding                                                                    (Transformer.swift:118-137)
    // The reference re-runs the decoder on the whole prefix at every step, and so does this: MultiHeadAttention
    // normalises over (length, hidden) jointly, so the output at every earlier position changes as the prefix grows and a
    // self-attention key/value cache would compute something else.  What does not change is the encoder side: in fused
    // mode the cross-attention key / value projections of the encoder states are computed once, not once per step.
    std::vector<int32_t> greedy(const std::vector<int32_t> &inputSequence, int32_t startToken, int32_t endToken, int64_t maxLength,
                                std::vector<float> *lastLogits = nullptr) const {
        const int64_t n = (int64_t)inputSequence.size();
        Tensor encoded = encoder(prepareInputs(inputSequence, 1, n), {n});
        const bool cached = decoder.canCacheEncoderProjections();
        std::vector<std::pair<Tensor, Tensor>> kv;
        if (cached) kv = decoder.projectEncoderStates(encoded);
        Tensor positions;     // fused mode: one encoding for the longest prefix instead of one per step
        if (Device::fused()) positions = positionalEncoding(maxLength);
        std::vector<int32_t> tokens;
        for (int64_t step = 0; step < maxLength; ++step) {
            std::vector<int32_t> tokenInput{startToken};
            tokenInput.insert(tokenInput.end(), tokens.begin(), tokens.end());
            const int64_t len = (int64_t)tokenInput.size();
            Tensor decIn = prepareInputs(tokenInput, 1, len, Device::fused() ? &positions : nullptr);
            Tensor output = cached ? decoder.withProjectedEncoder(decIn, kv, {n}, {len}) : decoder(decIn, encoded, {n}, {len});
            Tensor deembedded = output.broadcastMatrixMultiplied(embedding.embeddingMatrix, false, true);
            Tensor last = deembedded[{0, len - 1}];
            if (lastLogits) {
                const std::vector<float> row = last.elements();
                lastLogits->insert(lastLogits->end(), row.begin(), row.end());
            }
            const int32_t nextToken = (int32_t)last.argmax();
            tokens.push_back(nextToken);
            if (nextToken == endToken) break;
        }
        return tokens;
    }
};

}  // namespace dl4s

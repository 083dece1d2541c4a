/*
 * dl4s_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A single-threaded CPU restatement, in plain C, of the arithmetic that DL4S's
 * generic (no MKL, no Accelerate) CPU engine performs on the attention forward
 * path.  Only tests, the smoke check and the benchmark's cpu_baseline leg may
 * load this file's shared object; the GPU library never links or calls it.
 *
 * Every function cites the reference source it restates (paths relative to
 * the reference checkout, Sources/DL4S/...).  Each fp32 operation is one IEEE
 * rounding: build with -ffp-contract=off and without -ffast-math.
 *
 * What pins each function (see tests/test_oracle_pins.py):
 *   orc_gemm                 reference known answers Tests/DL4STests/VecTests.swift:86-156,
 *                            integer-exact cases for all four transpose flags, fp64 brute force
 *   orc_broadcast            numpy broadcasting on integer-exact and fp32 cases (+ - * /)
 *   orc_reduce_sum_axes,
 *   orc_reduce_max_axis      numpy sum/max in fp64, NaN-skipping scan by hand-written vectors
 *   orc_permute              numpy.transpose with the inverse permutation (scatter convention)
 *   orc_band, mask builders  brute-force closed form (j >= len_b) or (j > i)
 *   orc_softmax_last         scipy.special.softmax in fp64, shift invariance, NaN/Inf table
 *   orc_sdpa                 torch.nn.functional.scaled_dot_product_attention in fp64 (additive
 *                            -1e9 mask), blocked-weight and fully-blocked-row invariants
 *   orc_layernorm            torch.nn.functional.layer_norm in fp64; an fp64 closed form with the quirks,
 *                            each on an input where the plausible mistake fails: eps outside the root on
 *                            a low-variance input (the other placement is off by 3x), the biased variance
 *                            on four elements, the one-pass variance on two-element rows where it is
 *                            negative in fp32 (NaN row; a two-pass variance never is).  Far from a zero
 *                            mean the formula's fp32 value is noise of the summation order: only the
 *                            order this file uses (the generic engine's) is restated, and no GPU kernel
 *                            is held to it there
 *   orc_gelu                 x * scipy.special.expit(1.702 x)
 *   orc_mha, orc_ffn,
 *   orc_encoder_block,
 *   orc_decoder_block        torch.nn.functional.multi_head_attention_forward in fp64 for the
 *                            attention core; an independent fp64 numpy model for the whole layer
 *   orc_sdpa_backward        torch.autograd in fp64 through softmax(q k^T / T - 1e9 mask) v, central
 *                            finite differences of the oracle's own forward in fp64 arithmetic
 *   orc_log, orc_sin, orc_cos  numpy fp64 log/sin/cos; the reference's log accuracy test
 *                            Tests/DL4STests/VecTests.swift:242-258 (1e-4)
 *   orc_argmax               numpy.argmax (first maximum), hand-written NaN / tie / empty vectors
 *   orc_embedding            direct table indexing, zero rows for the ignore index
 *   (oracle/transformer.py composes these with the functions above into PositionalEncoding,
 *   prepareInputs, logSoftmax, the Transformer forward and its greedy decoding; pinned by the
 *   closed form sin/cos(pos / 10000^(2i/d)), scipy.special.log_softmax, an independent fp64
 *   numpy model of the whole network and the forward/greedy consistency check)
 * The reference's own tests hold no numeric vectors for softmax, masked attention, MHA,
 * LayerNorm or the transformer blocks (only a loss-convergence test), so beyond the checks
 * above those functions are pinned by mathematics, not by reference fixtures.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAXDIM 8

static void orc_strides(const int64_t *shape, int dim, int64_t *strides) {
    /* Engine/CPU/CPU.swift:47-59 -- row-major strides */
    int64_t s = 1;
    for (int i = dim - 1; i >= 0; --i) { strides[i] = s; s *= shape[i]; }
}

static int64_t orc_count(const int64_t *shape, int dim) {
    int64_t c = 1;
    for (int i = 0; i < dim; ++i) c *= shape[i];
    return c;
}

/* ------------------------------------------------------------------ GEMM */
/* Engine/CPU/Numeric/CPUGeneric.swift:184-256 (gemm_generic), reached from
 * Engine/CPU/Numeric/CPUFloat.swift:263-292.  Row-major, naive r-c-l loops,
 * tmp accumulated sequentially in fp32 over l ascending, C = alpha * tmp.
 * beta only pre-scales C, which is then overwritten (the reference's generic
 * path ignores beta != 0 in effect; restated as is). a_rows/a_cols etc. are the
 * stored shapes of A and B. */
void orc_gemm(int transA, int transB, int64_t M, int64_t N, int64_t K, float alpha,
              const float *A, const float *B, float beta, float *C) {
    if (M == 0 || N == 0 || ((alpha == 0.0f || K == 0) && beta == 1.0f)) return;
    if (alpha == 0.0f) {
        if (beta == 0.0f) for (int64_t i = 0; i < M * N; ++i) C[i] = 0.0f;
        else for (int64_t i = 0; i < M * N; ++i) C[i] *= beta;
    }
    if (beta == 0.0f) for (int64_t i = 0; i < M * N; ++i) C[i] = 0.0f;
    else for (int64_t i = 0; i < M * N; ++i) C[i] *= beta;
    for (int64_t r = 0; r < M; ++r) {
        for (int64_t c = 0; c < N; ++c) {
            float tmp = 0.0f;
            if (transA && transB)
                for (int64_t l = 0; l < K; ++l) tmp += A[r + l * M] * B[l + c * K];
            else if (transA)
                for (int64_t l = 0; l < K; ++l) tmp += A[r + l * M] * B[l * N + c];
            else if (transB)
                for (int64_t l = 0; l < K; ++l) tmp += A[l + r * K] * B[l + c * K];
            else
                for (int64_t l = 0; l < K; ++l) tmp += A[l + r * K] * B[l * N + c];
            C[r * N + c] = alpha * tmp;
        }
    }
}

/* Tensor/Operators/Matrix.swift:79-117 (broadcastMatrixMultiplied): a loop over the
 * broadcast batch dims, one 2-D gemm(alpha=1, beta=0) per index into its own buffer,
 * then Tensor(stacking:) (Stack.swift:79-122 -> CPUEngine.swift:995-1023) copies them
 * into one buffer.  Batch indices clamp to shape-1 (Matrix.swift:107-110).
 * lshape/rshape are full shapes of equal rank dim >= 2 (caller left-pads with 1s as
 * Matrix.swift:88-97 does).  Returns 0, or -1 on a shape error. */
int orc_bmm(const float *lhs, const int64_t *lshape, const float *rhs, const int64_t *rshape,
            int dim, int transL, int transR, float *out) {
    if (dim < 2 || dim > ORC_MAXDIM) return -1;
    int nb = dim - 2;
    int64_t lr = lshape[nb], lc = lshape[nb + 1], rr = rshape[nb], rc = rshape[nb + 1];
    int64_t M = transL ? lc : lr, K = transL ? lr : lc;
    int64_t K2 = transR ? rc : rr, N = transR ? rr : rc;
    if (K != K2) return -1;
    int64_t bshape[ORC_MAXDIM], bstr[ORC_MAXDIM], lstr[ORC_MAXDIM], rstr[ORC_MAXDIM];
    for (int i = 0; i < nb; ++i) {
        if (lshape[i] != rshape[i] && lshape[i] != 1 && rshape[i] != 1) return -1;
        bshape[i] = lshape[i] > rshape[i] ? lshape[i] : rshape[i];
    }
    orc_strides(bshape, nb, bstr);
    orc_strides(lshape, dim, lstr);
    orc_strides(rshape, dim, rstr);
    int64_t nbatch = orc_count(bshape, nb);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(M * N > 0 ? M * N : 1));
    for (int64_t b = 0; b < nbatch; ++b) {
        int64_t lo = 0, ro = 0;
        for (int i = 0; i < nb; ++i) {
            int64_t idx = (b / bstr[i]) % bshape[i];
            int64_t li = idx < lshape[i] - 1 ? idx : lshape[i] - 1;
            int64_t ri = idx < rshape[i] - 1 ? idx : rshape[i] - 1;
            lo += li * lstr[i];
            ro += ri * rstr[i];
        }
        orc_gemm(transL, transR, M, N, K, 1.0f, lhs + lo, rhs + ro, 0.0f, tmp);
        memcpy(out + b * M * N, tmp, sizeof(float) * (size_t)(M * N)); /* stack copy */
    }
    free(tmp);
    return 0;
}

/* ------------------------------------------------------- broadcast binaries */
/* Engine/CPU/CPUEngine.swift:90-214 (broadcast driver) and :589-637 (the four ops).
 * op: 0 add, 1 sub, 2 mul, 3 div.  Shapes are right-aligned, size-1 dims clamp.
 * Mode selection follows the reference: if the common equal-sized suffix has more
 * than one element the slices are combined element by element (vAdd/vSub/vMul/vDiv,
 * CPUFloat.swift:160-224); otherwise one operand is a scalar per slice and the scalar
 * forms are used, which differ in rounding for sub and div:
 *   vector - scalar = x + (-s)           (CPUEngine.swift:611)
 *   scalar - vector = -(x + (-s))        (CPUEngine.swift:607-610)
 *   vector / scalar = x * (1 / s)        (CPUEngine.swift:635)
 *   scalar / vector = s / x              (svDiv)
 * Returns 0 or -1 on incompatible shapes. */
int orc_broadcast(int op, const float *lhs, const int64_t *lshape_in, int ldim,
                  const float *rhs, const int64_t *rshape_in, int rdim,
                  float *out, int64_t *oshape /* out, rank max(ldim,rdim) */) {
    int dim = ldim > rdim ? ldim : rdim;
    if (dim > ORC_MAXDIM) return -1;
    int64_t ls[ORC_MAXDIM], rs[ORC_MAXDIM], os[ORC_MAXDIM];
    for (int i = 0; i < dim; ++i) {
        ls[i] = i < dim - ldim ? 1 : lshape_in[i - (dim - ldim)];
        rs[i] = i < dim - rdim ? 1 : rshape_in[i - (dim - rdim)];
        if (ls[i] != rs[i] && ls[i] != 1 && rs[i] != 1) return -1;
        os[i] = ls[i] > rs[i] ? ls[i] : rs[i];
        if (oshape) oshape[i] = os[i];
    }
    /* mode */
    int64_t sc = 1;
    for (int i = dim - 1; i >= 0 && ls[i] == rs[i]; --i) sc *= ls[i];
    int mode = 0; /* 0 vectorVector, 1 scalarVector (lhs scalar), 2 vectorScalar (rhs scalar) */
    if (sc <= 1) {
        for (int i = dim - 1; i >= 0; --i) {
            if (ls[i] > rs[i]) { mode = 2; break; }
            if (rs[i] > ls[i]) { mode = 1; break; }
        }
    }
    int64_t lstr[ORC_MAXDIM], rstr[ORC_MAXDIM], ostr[ORC_MAXDIM];
    orc_strides(ls, dim, lstr); orc_strides(rs, dim, rstr); orc_strides(os, dim, ostr);
    int64_t n = orc_count(os, dim);
    for (int64_t e = 0; e < n; ++e) {
        int64_t li = 0, ri = 0;
        for (int i = 0; i < dim; ++i) {
            int64_t idx = (e / ostr[i]) % os[i];
            li += lstr[i] * (idx < ls[i] - 1 ? idx : ls[i] - 1);
            ri += rstr[i] * (idx < rs[i] - 1 ? idx : rs[i] - 1);
        }
        float a = lhs[li], b = rhs[ri], r;
        switch (op) {
        case 0: r = a + b; break;
        case 1:
            if (mode == 2) { float nb = -b; r = a + nb; }
            else if (mode == 1) { float na = -a; float t = b + na; r = -t; }
            else r = a - b;
            break;
        case 2: r = a * b; break;
        default:
            if (mode == 2) { float rb = 1.0f / b; r = a * rb; }
            else r = a / b;
            break;
        }
        out[e] = r;
    }
    return 0;
}

/* ------------------------------------------------------------- reductions */
/* Engine/CPU/CPUEngine.swift:714-729 + :306-378 (reduceMultiAxis) with Float.sum
 * (CPUFloat.swift:239-261, generic arm): for every output element, start at 0, and for
 * every index of the reduced axes but the last (row-major order) add the sequential
 * left-to-right fp32 sum along the last reduced axis.  axes ascending.  The reference
 * takes a column-wise path (reducePrefix, vAdd of whole slices) when the axes are the
 * leading 0..n-1 and the result has more than one element: there each output element is
 * the sequential sum over the leading index, which is what the same loop nest gives when
 * the "row" is a single element; both are covered by this routine. */
int orc_reduce_sum_axes(const float *x, const int64_t *shape, int dim, const int *axes, int naxes,
                        float *out) {
    if (dim > ORC_MAXDIM || naxes > dim) return -1;
    int64_t str[ORC_MAXDIM];
    orc_strides(shape, dim, str);
    int reduced[ORC_MAXDIM] = {0};
    for (int i = 0; i < naxes; ++i) { if (axes[i] < 0 || axes[i] >= dim) return -1; reduced[axes[i]] = 1; }
    int64_t kshape[ORC_MAXDIM], kstr_src[ORC_MAXDIM]; int kd = 0;
    for (int i = 0; i < dim; ++i) if (!reduced[i]) { kshape[kd] = shape[i]; kstr_src[kd] = str[i]; ++kd; }
    int64_t kstr[ORC_MAXDIM]; orc_strides(kshape, kd, kstr);
    int64_t nout = orc_count(kshape, kd);
    int prefix = 1;
    for (int i = 0; i < naxes; ++i) if (axes[i] != i) prefix = 0;
    int64_t rshape[ORC_MAXDIM], rstr[ORC_MAXDIM];
    for (int i = 0; i < naxes; ++i) { rshape[i] = shape[axes[i]]; rstr[i] = str[axes[i]]; }
    int64_t inner_n, inner_s, nouter; int nouter_dims;
    if (naxes == 0) { memcpy(out, x, sizeof(float) * (size_t)nout); return 0; }
    if (prefix && nout > 1) { inner_n = 1; inner_s = 1; nouter_dims = naxes; }
    else { inner_n = rshape[naxes - 1]; inner_s = rstr[naxes - 1]; nouter_dims = naxes - 1; }
    int64_t ostr[ORC_MAXDIM]; orc_strides(rshape, nouter_dims, ostr);
    nouter = orc_count(rshape, nouter_dims);
    for (int64_t o = 0; o < nout; ++o) {
        int64_t base = 0;
        for (int i = 0; i < kd; ++i) base += ((o / kstr[i]) % kshape[i]) * kstr_src[i];
        float red = 0.0f;
        for (int64_t q = 0; q < nouter; ++q) {
            int64_t off = base;
            for (int i = 0; i < nouter_dims; ++i) off += ((q / ostr[i]) % rshape[i]) * rstr[i];
            float row = 0.0f;
            for (int64_t j = 0; j < inner_n; ++j) row += x[off + j * inner_s];
            red = red + row;
        }
        out[o] = red;
    }
    return 0;
}

/* Engine/CPU/CPUEngine.swift:655-677 (context == nil, axis != 0 arm) -> reduce :218-262 ->
 * Float.argmax with stride (CPUFloat.swift:294-318 and its strided twin): scan from -inf
 * with "v > max", so NaN is never selected.  For axis 0 with a multi-element result the
 * reference folds slices with an element-wise max; on NaN-free data it is the same value. */
int orc_reduce_max_axis(const float *x, const int64_t *shape, int dim, int axis, float *out) {
    if (dim > ORC_MAXDIM || axis < 0 || axis >= dim) return -1;
    int64_t str[ORC_MAXDIM]; orc_strides(shape, dim, str);
    int64_t outer = 1, inner = str[axis], n = shape[axis];
    for (int i = 0; i < axis; ++i) outer *= shape[i];
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t in = 0; in < inner; ++in) {
            const float *p = x + o * n * inner + in;
            float mx = -INFINITY;
            for (int64_t j = 0; j < n; ++j) { float v = p[j * inner]; if (v > mx) mx = v; }
            out[o * inner + in] = mx;
        }
    return 0;
}

/* ------------------------------------------------------------ elementwise */
/* Engine/CPU/Numeric/CPUFloat.swift:457-511, generic arms: libm expf / tanhf / sqrtf. */
void orc_exp(const float *x, float *out, int64_t n)  { for (int64_t i = 0; i < n; ++i) out[i] = expf(x[i]); }
void orc_tanh(const float *x, float *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = tanhf(x[i]); }
void orc_sqrt(const float *x, float *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = sqrtf(x[i]); }
/* CPUFloat.swift relu arm: max(x, 0) */
/* Engine/CPU/Numeric/CPUFloat.swift:471-483 (logf), :521-533 (sinf), :535-547 (cosf), generic branches */
void orc_log(const float *x, float *out, int64_t n)  { for (int64_t i = 0; i < n; ++i) out[i] = logf(x[i]); }
void orc_sin(const float *x, float *out, int64_t n)  { for (int64_t i = 0; i < n; ++i) out[i] = sinf(x[i]); }
void orc_cos(const float *x, float *out, int64_t n)  { for (int64_t i = 0; i < n; ++i) out[i] = cosf(x[i]); }

/* Engine/CPU/Numeric/CPUFloat.swift:294-318, generic branch: scan from (-inf, 0) with `v > maxV` */
int64_t orc_argmax(const float *x, int64_t n, float *out_value) {
    int64_t mi = 0;
    float mv = -INFINITY;
    for (int64_t i = 0; i < n; ++i) {
        if (x[i] > mv) { mv = x[i]; mi = i; }
    }
    if (out_value) *out_value = mv;
    return mi;
}

/* NN/Layer/Embedding.swift:152-165: row tokens[t] of the [vocab, D] table, zeros for ignore_index */
int orc_embedding(const float *table, int64_t vocab, int64_t D, const int32_t *tokens, int64_t n,
                  int32_t ignore_index, float *out) {
    for (int64_t t = 0; t < n; ++t) {
        if (tokens[t] == ignore_index) {
            for (int64_t c = 0; c < D; ++c) out[t * D + c] = 0.0f;
        } else {
            if (tokens[t] < 0 || tokens[t] >= vocab) return -1;   /* the reference traps on the subscript */
            memcpy(out + t * D, table + (int64_t)tokens[t] * D, (size_t)D * sizeof(float));
        }
    }
    return 0;
}

void orc_relu(const float *x, float *out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = x[i] > 0.0f ? x[i] : 0.0f; }

/* Tensor/Operators/Unary.swift:245-247 (gaussianErrorLinear) with sigmoid :184-186:
 * x * (0.5 * tanh((x * 1.702) * 0.5) + 0.5); each product and sum rounded once. */
void orc_gelu(const float *x, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        float a = x[i] * 1.702f;
        float h = a * 0.5f;
        float t = tanhf(h);
        float s = 0.5f * t;
        s = s + 0.5f;
        out[i] = x[i] * s;
    }
}

/* ----------------------------------------------------------- permute, band */
/* Engine/CPU/CPUEngine.swift:897-935: source axis i lands on destination axis
 * arrangement[i] (a scatter), dstShape[arrangement[i]] = shape[i]
 * (Tensor/Operators/Shape.swift:121-132). */
int orc_permute(const float *x, const int64_t *shape, int dim, const int *arrangement, float *out,
                int64_t *oshape) {
    if (dim > ORC_MAXDIM) return -1;
    int64_t dshape[ORC_MAXDIM], sstr[ORC_MAXDIM], dstr[ORC_MAXDIM];
    int seen[ORC_MAXDIM] = {0};
    for (int i = 0; i < dim; ++i) {
        if (arrangement[i] < 0 || arrangement[i] >= dim || seen[arrangement[i]]) return -1;
        seen[arrangement[i]] = 1;
        dshape[arrangement[i]] = shape[i];
    }
    orc_strides(shape, dim, sstr); orc_strides(dshape, dim, dstr);
    if (oshape) for (int i = 0; i < dim; ++i) oshape[i] = dshape[i];
    int64_t n = orc_count(shape, dim);
    for (int64_t e = 0; e < n; ++e) {
        int64_t d = 0;
        for (int i = 0; i < dim; ++i) d += ((e / sstr[i]) % shape[i]) * dstr[arrangement[i]];
        out[d] = x[e];
    }
    return 0;
}

/* Tensor/Operators/UtilOps.swift:117-121 (zero fill) + Engine/CPU/CPUEngine.swift:1135-1158:
 * keep columns start..end-1 of row i, start = min(max(0, i - below), cols),
 * end = max(min(cols, i + above + 1), start); a negative has_* means "nil" = max(rows, cols). */
void orc_band(const float *x, int64_t rows, int64_t cols, int has_below, int64_t below,
              int has_above, int64_t above, float *out) {
    int64_t mx = rows > cols ? rows : cols;
    if (!has_below) below = mx;
    if (!has_above) above = mx;
    for (int64_t i = 0; i < rows * cols; ++i) out[i] = 0.0f;
    for (int64_t i = 0; i < rows; ++i) {
        int64_t start = i - below; if (start < 0) start = 0; if (start > cols) start = cols;
        int64_t end = i + above + 1; if (end > cols) end = cols; if (end < start) end = start;
        for (int64_t j = start; j < end; ++j) out[i * cols + j] = x[i * cols + j];
    }
}

/* ------------------------------------------------------------ mask builders */
/* NN/Models/Transformer/TransformerUtil.swift:29-36: [B,1,1,maxLen], 1 where j >= len_b. */
int64_t orc_make_encoder_masks(const int32_t *lens, int64_t B, float *out /* B*maxLen or NULL */) {
    int64_t maxLen = 0;
    for (int64_t b = 0; b < B; ++b) if (lens[b] > maxLen) maxLen = lens[b];
    if (out)
        for (int64_t b = 0; b < B; ++b)
            for (int64_t j = 0; j < maxLen; ++j) out[b * maxLen + j] = j < lens[b] ? 0.0f : 1.0f;
    return maxLen;
}

/* NN/Models/Transformer/TransformerUtil.swift:38-50: 1 - relu(1 - pad[B,1,1,L] - causal[L,L]),
 * causal = band(ones, below: -1, above: nil).  Evaluated with the same fp32 steps. Shape [B,1,L,L]. */
int64_t orc_make_decoder_masks(const int32_t *lens, int64_t B, float *out /* B*L*L or NULL */) {
    int64_t L = 0;
    for (int64_t b = 0; b < B; ++b) if (lens[b] > L) L = lens[b];
    if (!out) return L;
    float *ones = (float *)calloc((size_t)(L * L > 0 ? L * L : 1), sizeof(float));
    float *causal = (float *)malloc(sizeof(float) * (size_t)(L * L > 0 ? L * L : 1));
    for (int64_t i = 0; i < L * L; ++i) ones[i] = 1.0f;
    orc_band(ones, L, L, 1, -1, 0, 0, causal);
    for (int64_t b = 0; b < B; ++b)
        for (int64_t i = 0; i < L; ++i)
            for (int64_t j = 0; j < L; ++j) {
                float pad = j < lens[b] ? 0.0f : 1.0f;
                float t = pad + (-1.0f); t = -t;   /* 1 - pad: scalar - vector = -(x + (-s)) */
                t = t - causal[i * L + j];         /* slices of length L: plain vSub */
                t = t > 0.0f ? t : 0.0f;           /* relu */
                t = t + (-1.0f);                   /* 1 - relu(...) */
                out[(b * L + i) * L + j] = -t;
            }
    free(ones); free(causal);
    return L;
}

/* ------------------------------------------------------------------ softmax */
/* Tensor/Operators/Unary.swift:190-194 on the last axis of a [rows, n] matrix:
 * max scan (NaN skipped) -> x + (-max) -> expf -> sequential sum -> e * (1/sum). */
void orc_softmax_last(const float *x, int64_t rows, int64_t n, float *out) {
    for (int64_t r = 0; r < rows; ++r) {
        const float *p = x + r * n; float *o = out + r * n;
        float mx = -INFINITY;
        for (int64_t c = 0; c < n; ++c) if (p[c] > mx) mx = p[c];
        float nmx = -mx;
        for (int64_t c = 0; c < n; ++c) o[c] = expf(p[c] + nmx);
        float s = 0.0f;
        for (int64_t c = 0; c < n; ++c) s += o[c];
        float rs = 1.0f / s;
        for (int64_t c = 0; c < n; ++c) o[c] = o[c] * rs;
    }
}

/* ---------------------------------------------------------------------- SDPA */
/* NN/Models/Transformer/ScaledDotProductAttention.swift:43-64.
 * q [B,H,Lq,dk], k [B,H,Lk,dk], v [B,H,Lk,dv] contiguous; mask may be NULL or a float
 * tensor of rank mdim <= 4, right-aligned broadcastable to [B,H,Lq,Lk], 1 = blocked.
 * Steps: q * (1/T) -> per-(b,h) gemm(tB) + stack -> s - mask * 1e9 -> softmax -> per-(b,h)
 * gemm + stack.  Score-sized temporaries are materialised like the reference does.
 * Returns 0, -1 on bad shapes, -2 when out of memory. */
int orc_sdpa(const float *q, const float *k, const float *v, const float *mask,
             const int64_t *mshape, int mdim, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
             int64_t dk, int64_t dv, float temperature, float *out) {
    int64_t nq = B * H * Lq * dk, ns = B * H * Lq * Lk;
    float *qs = (float *)malloc(sizeof(float) * (size_t)(nq > 0 ? nq : 1));
    float *S = (float *)malloc(sizeof(float) * (size_t)(ns > 0 ? ns : 1));
    float *P = (float *)malloc(sizeof(float) * (size_t)(ns > 0 ? ns : 1));
    if (!qs || !S || !P) { free(qs); free(S); free(P); return -2; }
    float rT = 1.0f / temperature;                       /* CPUEngine.swift:635 */
    for (int64_t i = 0; i < nq; ++i) qs[i] = q[i] * rT;
    int64_t qsh[4] = {B, H, Lq, dk}, ksh[4] = {B, H, Lk, dk}, vsh[4] = {B, H, Lk, dv};
    int64_t ssh[4] = {B, H, Lq, Lk};
    int rc = orc_bmm(qs, qsh, k, ksh, 4, 0, 1, S);
    if (rc == 0 && mask) {
        int64_t mn = orc_count(mshape, mdim);
        float *M = (float *)malloc(sizeof(float) * (size_t)(mn > 0 ? mn : 1));
        if (!M) rc = -2;
        else {
            for (int64_t i = 0; i < mn; ++i) M[i] = mask[i] * 1e9f;   /* mask * 1e9 */
            rc = orc_broadcast(1, S, ssh, 4, M, mshape, mdim, P, NULL); /* attn - that */
            if (rc == 0) memcpy(S, P, sizeof(float) * (size_t)ns);
            free(M);
        }
    }
    if (rc == 0) {
        orc_softmax_last(S, B * H * Lq, Lk, P);
        rc = orc_bmm(P, ssh, v, vsh, 4, 0, 0, out);
    }
    free(qs); free(S); free(P);
    return rc;
}

/* ------------------------------------------------------------- SDPA backward */
/* Gradients of ScaledDotProductAttention with respect to q, k and v for an upstream gradient dout of its result, as
 * the reference's reverse-mode closures produce them for the forward graph of ScaledDotProductAttention.swift:43-64:
 *   o = p.bmm(v)            per slice dp = dout . v^T, dv = p^T . dout          Matrix.swift:139-174 (through the
 *                           subscript views and the stack of broadcastMatrixMultiplied, Matrix.swift:79-117)
 *   p = e / z               de = dp * (1/z);  dz = -sum_j((dp * e) * (1/(z*z)))   Binary.swift:235-300
 *   z = reduceSum(e, 3)     de += dz (broadcast along the row)                    Reduce.swift:35-62
 *   e = exp(d)              dd = de * e                                            Unary.swift:33-55
 *   d = s2 - max (detached), s2 = s - mask*1e9: gradient passes unchanged          Unary.swift:190-194, Binary.swift:161-224
 *   s = a.bmm(k^T)          da = ds . k, dk = (a^T . ds)^T                         Matrix.swift:139-174
 *   a = q / T               dq = da * (1/T)                                        Binary.swift:259-277
 * The mask takes no gradient.  Every product is the generic triple loop, every element-wise step one rounding. */
int orc_sdpa_backward(const float *q, const float *k, const float *v, const float *mask,
                      const int64_t *mshape, int mdim, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                      int64_t dk, int64_t dv, float temperature, const float *dout,
                      float *dq, float *dkey, float *dval) {
    int64_t nq = B * H * Lq * dk, ns = B * H * Lq * Lk;
    float *qs = (float *)malloc(sizeof(float) * (size_t)(nq > 0 ? nq : 1));
    float *S = (float *)malloc(sizeof(float) * (size_t)(ns > 0 ? ns : 1));
    float *E = (float *)malloc(sizeof(float) * (size_t)(ns > 0 ? ns : 1));
    float *Z = (float *)malloc(sizeof(float) * (size_t)(B * H * Lq > 0 ? B * H * Lq : 1));
    float *G = (float *)malloc(sizeof(float) * (size_t)(Lq * Lk > 0 ? Lq * Lk : 1));
    float *Pm = (float *)malloc(sizeof(float) * (size_t)(Lq * Lk > 0 ? Lq * Lk : 1));
    float *da = (float *)malloc(sizeof(float) * (size_t)(Lq * dk > 0 ? Lq * dk : 1));
    float *dkt = (float *)malloc(sizeof(float) * (size_t)(Lk * dk > 0 ? Lk * dk : 1));
    int rc = (!qs || !S || !E || !Z || !G || !Pm || !da || !dkt) ? -2 : 0;
    if (rc == 0) {
        float rT = 1.0f / temperature;
        for (int64_t i = 0; i < nq; ++i) qs[i] = q[i] * rT;
        int64_t qsh[4] = {B, H, Lq, dk}, ksh[4] = {B, H, Lk, dk}, ssh[4] = {B, H, Lq, Lk};
        rc = orc_bmm(qs, qsh, k, ksh, 4, 0, 1, S);
        if (rc == 0 && mask) {
            int64_t mn = orc_count(mshape, mdim);
            float *M = (float *)malloc(sizeof(float) * (size_t)(mn > 0 ? mn : 1));
            if (!M) rc = -2;
            else {
                for (int64_t i = 0; i < mn; ++i) M[i] = mask[i] * 1e9f;
                rc = orc_broadcast(1, S, ssh, 4, M, mshape, mdim, E, NULL);
                if (rc == 0) memcpy(S, E, sizeof(float) * (size_t)ns);
                free(M);
            }
        }
    }
    if (rc == 0) {
        /* forward intermediates of the softmax: e = exp(s - max), z = sum(e) */
        for (int64_t r = 0; r < B * H * Lq; ++r) {
            const float *p = S + r * Lk; float *e = E + r * Lk;
            float mx = -INFINITY;
            for (int64_t c = 0; c < Lk; ++c) if (p[c] > mx) mx = p[c];
            float nmx = -mx, z = 0.0f;
            for (int64_t c = 0; c < Lk; ++c) e[c] = expf(p[c] + nmx);
            for (int64_t c = 0; c < Lk; ++c) z += e[c];
            Z[r] = z;
        }
        float rT = 1.0f / temperature;
        for (int64_t bh = 0; bh < B * H; ++bh) {
            const float *e = E + bh * Lq * Lk, *z = Z + bh * Lq;
            const float *go = dout + bh * Lq * dv, *vv = v + bh * Lk * dv, *kk = k + bh * Lk * dk;
            /* p = e * (1/z) */
            for (int64_t r = 0; r < Lq; ++r) {
                float rz = 1.0f / z[r];
                for (int64_t c = 0; c < Lk; ++c) Pm[r * Lk + c] = e[r * Lk + c] * rz;
            }
            orc_gemm(1, 0, Lk, dv, Lq, 1.0f, Pm, go, 0.0f, dval + bh * Lk * dv);   /* dv = p^T . dout */
            orc_gemm(0, 1, Lq, Lk, dv, 1.0f, go, vv, 0.0f, G);                      /* dp = dout . v^T */
            for (int64_t r = 0; r < Lq; ++r) {
                float zr = z[r], rz = 1.0f / zr, rzz = 1.0f / (zr * zr), acc = 0.0f;
                for (int64_t c = 0; c < Lk; ++c) acc += (G[r * Lk + c] * e[r * Lk + c]) * rzz;
                float dz = -acc;
                for (int64_t c = 0; c < Lk; ++c) {
                    float de = G[r * Lk + c] * rz + dz;
                    G[r * Lk + c] = de * e[r * Lk + c];                                        /* ds */
                }
            }
            orc_gemm(0, 0, Lq, dk, Lk, 1.0f, G, kk, 0.0f, da);                      /* da = ds . k */
            for (int64_t i = 0; i < Lq * dk; ++i) dq[bh * Lq * dk + i] = da[i] * rT;
            orc_gemm(1, 0, dk, Lk, Lq, 1.0f, qs + bh * Lq * dk, G, 0.0f, dkt);      /* a^T . ds : [dk, Lk] */
            for (int64_t c = 0; c < Lk; ++c)
                for (int64_t l = 0; l < dk; ++l) dkey[bh * Lk * dk + c * dk + l] = dkt[l * Lk + c];
        }
    }
    free(qs); free(S); free(E); free(Z); free(G); free(Pm); free(da); free(dkt);
    return rc;
}

/* ----------------------------------------------------------------- LayerNorm */
/* NN/Layer/LayerNorm.swift:62-77 with reduceMean / variance of
 * Tensor/Operators/Reduce.swift:87-110.  x is [B, inner...] flattened to [B, rows, D]
 * where D is the size of scale/shift (last axis) and rows*D = all non-batch elements:
 *   sum  = reduceSum(axes 1..)         (rows summed one by one, then added in order)
 *   mean = sum * (1/N)
 *   var  = reduceSum(x*x) * (1/N) - mean*mean
 *   y    = ((x + (-mean)) * (1 / (sqrt(var) + 1e-5))) * scale + shift
 * N = rows*D as a Float.  eps sits outside the square root. */
void orc_layernorm(const float *x, int64_t B, int64_t rows, int64_t D, const float *scale,
                   const float *shift, float *out) {
    int64_t n = rows * D;
    float rN = 1.0f / (float)n;
    for (int64_t b = 0; b < B; ++b) {
        const float *p = x + b * n; float *o = out + b * n;
        float sum = 0.0f, sumsq = 0.0f;
        for (int64_t r = 0; r < rows; ++r) {
            float row = 0.0f, rowsq = 0.0f;
            for (int64_t d = 0; d < D; ++d) { float e = p[r * D + d]; row += e; float sq = e * e; rowsq += sq; }
            sum = sum + row; sumsq = sumsq + rowsq;
        }
        float mean = sum * rN;
        float msq = sumsq * rN;
        float mm = mean * mean;
        float var = msq - mm;
        float denom = sqrtf(var) + 1e-5f;
        float rden = 1.0f / denom;
        float nmean = -mean;
        for (int64_t i = 0; i < n; ++i) {
            float c = p[i] + nmean;
            float nrm = c * rden;
            float sc = nrm * scale[i % D];
            o[i] = sc + shift[i % D];
        }
    }
}

/* ----------------------------------------------------------------------- MHA */
/* NN/Models/Transformer/MultiHeadAttention.swift:97-127 with dropout inactive
 * (NN/Layer/Dropout.swift:47-55 returns its input).  q [B,Lq,D], k,v [B,Lk,D];
 * Wq,Wk [D,H*dk], Wv [D,H*dv], Wo [H*dv,D] (no biases); mask as for orc_sdpa;
 * temperature = sqrtf(dk) (:74).  attn_out, if non-NULL, receives the SDPA output
 * [B,H,Lq,dv] for tests. */
int orc_mha(const float *q, const float *k, const float *v, const float *mask,
            const int64_t *mshape, int mdim, int64_t B, int64_t Lq, int64_t Lk, int64_t D,
            int64_t H, int64_t dk, int64_t dv, const float *Wq, const float *Wk, const float *Wv,
            const float *Wo, const float *ln_scale, const float *ln_shift, float *out,
            float *attn_out) {
    int rc = 0;
    int64_t nqp = B * Lq * H * dk, nkp = B * Lk * H * dk, nvp = B * Lk * H * dv, nop = B * Lq * H * dv;
    float *qp = (float *)malloc(sizeof(float) * (size_t)nqp), *qt = (float *)malloc(sizeof(float) * (size_t)nqp);
    float *kp = (float *)malloc(sizeof(float) * (size_t)nkp), *kt = (float *)malloc(sizeof(float) * (size_t)nkp);
    float *vp = (float *)malloc(sizeof(float) * (size_t)nvp), *vt = (float *)malloc(sizeof(float) * (size_t)nvp);
    float *at = (float *)malloc(sizeof(float) * (size_t)nop), *am = (float *)malloc(sizeof(float) * (size_t)nop);
    float *fo = (float *)malloc(sizeof(float) * (size_t)(B * Lq * D));
    if (!qp || !qt || !kp || !kt || !vp || !vt || !at || !am || !fo) { rc = -2; goto done; }
    {
        int64_t xq[3] = {B, Lq, D}, xk[3] = {B, Lk, D};
        int64_t wq[3] = {1, D, H * dk}, wv[3] = {1, D, H * dv}, wo[3] = {1, H * dv, D};
        int perm[4] = {0, 2, 1, 3};
        if ((rc = orc_bmm(q, xq, Wq, wq, 3, 0, 0, qp))) goto done;        /* :109 */
        if ((rc = orc_bmm(k, xk, Wk, wq, 3, 0, 0, kp))) goto done;        /* :110 */
        if ((rc = orc_bmm(v, xk, Wv, wv, 3, 0, 0, vp))) goto done;        /* :111 */
        int64_t s1[4] = {B, Lq, H, dk}, s2[4] = {B, Lk, H, dk}, s3[4] = {B, Lk, H, dv};
        orc_permute(qp, s1, 4, perm, qt, NULL);                           /* :113-115 */
        orc_permute(kp, s2, 4, perm, kt, NULL);
        orc_permute(vp, s3, 4, perm, vt, NULL);
        if ((rc = orc_sdpa(qt, kt, vt, mask, mshape, mdim, B, H, Lq, Lk, dk, dv, sqrtf((float)dk), at))) goto done;
        if (attn_out) memcpy(attn_out, at, sizeof(float) * (size_t)nop);
        int64_t s4[4] = {B, H, Lq, dv};
        orc_permute(at, s4, 4, perm, am, NULL);                           /* :119-120 */
        int64_t xo[3] = {B, Lq, H * dv};
        if ((rc = orc_bmm(am, xo, Wo, wo, 3, 0, 0, fo))) goto done;       /* :121 */
        for (int64_t i = 0; i < B * Lq * D; ++i) fo[i] = fo[i] + q[i];    /* :123 residual = query input */
        orc_layernorm(fo, B, Lq, D, ln_scale, ln_shift, out);             /* :124 over (L, D) jointly */
    }
done:
    free(qp); free(qt); free(kp); free(kt); free(vp); free(vt); free(at); free(am); free(fo);
    return rc;
}

/* ----------------------------------------------------------------------- FFN */
/* NN/Models/Transformer/PointwiseFeedForward.swift:67-82 with Dense
 * (NN/Layer/Dense.swift:64-68: 2-D gemm then + bias) and dropout inactive.
 * x [B, L, D] viewed [B*L, D]; W1 [D,F], b1 [F], W2 [F,D], b2 [D];
 * LayerNorm on the 2-D tensor normalises each token (rows = 1). */
int orc_ffn(const float *x, int64_t BL, int64_t D, int64_t F, const float *W1, const float *b1,
            const float *W2, const float *b2, const float *ln_scale, const float *ln_shift,
            float *out) {
    float *h = (float *)malloc(sizeof(float) * (size_t)(BL * F));
    float *g = (float *)malloc(sizeof(float) * (size_t)(BL * F));
    float *o = (float *)malloc(sizeof(float) * (size_t)(BL * D));
    if (!h || !g || !o) { free(h); free(g); free(o); return -2; }
    orc_gemm(0, 0, BL, F, D, 1.0f, x, W1, 0.0f, h);
    for (int64_t i = 0; i < BL * F; ++i) h[i] = h[i] + b1[i % F];
    orc_gelu(h, g, BL * F);
    orc_gemm(0, 0, BL, D, F, 1.0f, g, W2, 0.0f, o);
    for (int64_t i = 0; i < BL * D; ++i) o[i] = o[i] + b2[i % D];
    for (int64_t i = 0; i < BL * D; ++i) o[i] = o[i] + x[i];               /* tmp4 + denseInputs */
    orc_layernorm(o, BL, 1, D, ln_scale, ln_shift, out);
    free(h); free(g); free(o);
    return 0;
}

/* -------------------------------------------------------------------- blocks */
struct orc_mha_params { const float *Wq, *Wk, *Wv, *Wo, *ln_scale, *ln_shift; };
struct orc_ffn_params { const float *W1, *b1, *W2, *b2, *ln_scale, *ln_shift; };

/* NN/Models/Transformer/TransformerEncoderBlock.swift:58-65. */
int orc_encoder_block(const float *x, const float *mask, const int64_t *mshape, int mdim,
                      int64_t B, int64_t L, int64_t D, int64_t H, int64_t dk, int64_t dv, int64_t F,
                      const struct orc_mha_params *a, const struct orc_ffn_params *f, float *out) {
    float *t = (float *)malloc(sizeof(float) * (size_t)(B * L * D));
    if (!t) return -2;
    int rc = orc_mha(x, x, x, mask, mshape, mdim, B, L, L, D, H, dk, dv, a->Wq, a->Wk, a->Wv, a->Wo,
                     a->ln_scale, a->ln_shift, t, NULL);
    if (rc == 0) rc = orc_ffn(t, B * L, D, F, f->W1, f->b1, f->W2, f->b2, f->ln_scale, f->ln_shift, out);
    free(t);
    return rc;
}

/* NN/Models/Transformer/TransformerDecoderBlock.swift:61-68: self-attention with the decoder
 * mask, cross-attention over the encoder output with the encoder mask, then the FFN. */
int orc_decoder_block(const float *dec, const float *enc, const float *dec_mask,
                      const int64_t *dmshape, int dmdim, const float *enc_mask,
                      const int64_t *emshape, int emdim, int64_t B, int64_t Ld, int64_t Le, int64_t D,
                      int64_t H, int64_t dk, int64_t dv, int64_t F, const struct orc_mha_params *self_a,
                      const struct orc_mha_params *cross_a, const struct orc_ffn_params *f, float *out) {
    float *t1 = (float *)malloc(sizeof(float) * (size_t)(B * Ld * D));
    float *t2 = (float *)malloc(sizeof(float) * (size_t)(B * Ld * D));
    if (!t1 || !t2) { free(t1); free(t2); return -2; }
    int rc = orc_mha(dec, dec, dec, dec_mask, dmshape, dmdim, B, Ld, Ld, D, H, dk, dv, self_a->Wq,
                     self_a->Wk, self_a->Wv, self_a->Wo, self_a->ln_scale, self_a->ln_shift, t1, NULL);
    if (rc == 0)
        rc = orc_mha(t1, enc, enc, enc_mask, emshape, emdim, B, Ld, Le, D, H, dk, dv, cross_a->Wq,
                     cross_a->Wk, cross_a->Wv, cross_a->Wo, cross_a->ln_scale, cross_a->ln_shift, t2, NULL);
    if (rc == 0) rc = orc_ffn(t2, B * Ld, D, F, f->W1, f->b1, f->W2, f->b2, f->ln_scale, f->ln_shift, out);
    free(t1); free(t2);
    return rc;
}

/* -------------------------------------------------------------------- decode */
/* The reference has no key/value cache (greedy decoding re-runs the prefix,
 * NN/Models/Transformer/Transformer.swift:118-137); one decode step is the same
 * ScaledDotProductAttention call with Lq = 1 over the first T rows of a cache laid out
 * [B,H,Tcap,d].  The cache rows are gathered to contiguous [B,H,T,d] tensors and handed
 * to orc_sdpa unchanged. */
int orc_sdpa_decode(const float *q, const float *kcache, const float *vcache, int64_t B, int64_t H,
                    int64_t T, int64_t Tcap, int64_t d, float temperature, float *out) {
    int64_t n = B * H * T * d;
    float *kc = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    float *vc = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    if (!kc || !vc) { free(kc); free(vc); return -2; }
    for (int64_t bh = 0; bh < B * H; ++bh) {
        memcpy(kc + bh * T * d, kcache + bh * Tcap * d, sizeof(float) * (size_t)(T * d));
        memcpy(vc + bh * T * d, vcache + bh * Tcap * d, sizeof(float) * (size_t)(T * d));
    }
    int rc = orc_sdpa(q, kc, vc, NULL, NULL, 0, B, H, 1, T, d, d, temperature, out);
    free(kc); free(vc);
    return rc;
}

// Gradients of the fused attention for head dims above 128 and up to 256 (multiples of 4, head-major tensors): the row
// fragments and accumulators of a fused kernel of that width do not fit a wavefront's registers, so the five products run
// as batched GEMMs around one elementwise pass, on score tensors held in the context's pool.  Included by
// sdpa_backward.hip only.
//
//   S2 = ((q * rT) * log2(e)) . k^T        the forward kernel's scores (base-2 exponent domain), [pairs, Lq, Lk]
//   dP = dout . v^T                        [pairs, Lq, Lk]
//   P  = 2^(mask(S2) - m) / l              in place of S2; m, l: the row's maximum and sum of 2^(s - m), formed here from
//                                          these very scores (the forward call's statistics come from another summation
//                                          order: against scores of a few hundred that is 1e-4 of a weight)
//   dS = P * (dP - D)                      in place of dP; D_i = sum_j P_ij dP_ij (= dout_i . out_i; summed here so that it
//                                          belongs to these weights to the last bit of their rounding)
//   dv = P^T . dout,  dk = rT * dS^T . q,  dq = rT * dS . k
//
// (Tensor/Operators/Matrix.swift:139-174, Binary.swift:235-300, Unary.swift:33-55, Reduce.swift:35-62 give the same
// gradients closure by closure.)  The (batch, head) pairs are taken in chunks whose two score tensors stay inside the
// gradient scratch bound.  Under the plain causal mask (without DL4S_SDPA_STRICT) the queries go in blocks of 512 rows
// that contract only the keys up to their last row - the weights beyond are exactly zero - and add their dk / dv
// contributions block after block; every other mask kind visits every key.  Deterministic: no atomics, every sum in a fixed
// order.
#pragma once
#include "sdpa_common.h"

namespace {

// qs = (q * rT) * log2(e): the two roundings of the forward kernels' Q fragment
__global__ __launch_bounds__(256) void sdpa_bwd_wide_scale_q(const float *__restrict__ q, float *__restrict__ qs, long long n4, float rT) {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n4; i += (long long)gridDim.x * 256) {
        const f32x4 t = reinterpret_cast<const f32x4 *>(q)[i];
        const f32x4 r = {(t.x * rT) * LOG2E, (t.y * rT) * LOG2E, (t.z * rT) * LOG2E, (t.w * rT) * LOG2E};
        reinterpret_cast<f32x4 *>(qs)[i] = r;
    }
}

// One workgroup per query row of a block of a chunk: S2 -> P and dP -> dS in place.  pair0: the chunk's first (batch, head)
// pair; the block holds the query rows i0 .. i0 + nq - 1 of every pair against the keys 0 .. Lk - 1 (Lk: the block's key
// count, the row length of S and dP; keys beyond it are blocked and weigh exactly zero).  Four passes over the row, which
// stays in cache: the masked scores and their maximum, the sum, D, the weights and dS.  Sums in a fixed order.
__global__ __launch_bounds__(256) void sdpa_bwd_wide_weights(float *__restrict__ S, float *__restrict__ dP, MaskArgs mask, long long pair0,
                                                             int H, int i0, int nq, int Lk) {
    __shared__ float red[4];
    const long long row = blockIdx.x;                 // over the chunk's pairs x nq
    const long long bh = pair0 + row / nq;
    const int qi = i0 + (int)(row % nq);
    const int b = (int)(bh / H), hh = (int)(bh % H);
    const bool causal = mask.kind == DL4S_MASK_CAUSAL || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS;
    const bool lens = mask.kind == DL4S_MASK_KEY_LENGTHS || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS;
    const int len = lens ? mask.lengths[b] : Lk;
    const float *mrow = mask.kind == DL4S_MASK_DENSE_F32 ? mask.dense + b * mask.sb + hh * mask.sh + qi * mask.sq : nullptr;
    float *srow = S + row * Lk, *drow = dP + row * Lk;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < Lk; j += 256) {
        float s = srow[j];
        if (mrow) s = dense_masked2(s, mrow[j * mask.sk]);
        else if ((causal && j > qi) || (lens && j >= len)) s = blocked_score2(s);
        srow[j] = s;
        mx = fmaxf(mx, s);      // a NaN score does not move the maximum; it makes the sum NaN below, as in the reference
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float m = (mx == -INFINITY) ? 0.f : mx;     // a row of -inf: weights 0 / 0
    __syncthreads();
    float sum = 0.f;
    for (int j = threadIdx.x; j < Lk; j += 256) sum += fast_exp2(srow[j] - m);
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    const float inv = 1.0f / (((red[0] + red[1]) + red[2]) + red[3]);
    __syncthreads();
    float dsum = 0.f;
    for (int j = threadIdx.x; j < Lk; j += 256) {
        const float p = fast_exp2(srow[j] - m) * inv;
        srow[j] = p;
        dsum += p * drow[j];
    }
    for (int o = 32; o > 0; o >>= 1) dsum += __shfl_xor(dsum, o, 64);
    if (lane == 0) red[wave] = dsum;
    __syncthreads();
    const float Di = ((red[0] + red[1]) + red[2]) + red[3];
    for (int j = threadIdx.x; j < Lk; j += 256) drow[j] = srow[j] * (drow[j] - Di);
}

int sdpa_backward_wide(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *out, const float *stats,
                       const float *dout, float *dq, float *dk, float *dv, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t d,
                       float rT, const dl4s_mask_desc *mask, int strict, long long scratch_max_bytes) {
    (void)out; (void)stats;     // the weights and D are formed again from the scores of this call (see above)
    MaskArgs m{};
    int rc = build_mask_args(ctx, mask, B, H, Lq, Lk, false, m);
    if (rc != DL4S_HIP_OK) return rc;
    const int64_t pairs = B * H;
    DL4S_REQUIRE(pairs * Lq < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "sdpa backward: too many query rows");
    // (batch, head) pairs per chunk: two [Lq, Lk] tensors per pair inside the bound, at least one pair
    const long long per_pair = 2ll * Lq * Lk * (long long)sizeof(float);
    int64_t chunk = scratch_max_bytes / per_pair;
    if (chunk < 1) chunk = 1;
    if (chunk > pairs) chunk = pairs;
    void *bufs[3] = {nullptr, nullptr, nullptr};     // S2 / P, dP / dS, scaled q
    const size_t sizes[3] = {(size_t)(chunk * Lq * Lk) * sizeof(float), (size_t)(chunk * Lq * Lk) * sizeof(float),
                             (size_t)(chunk * Lq * d) * sizeof(float)};
    for (int i = 0; i < 3; ++i)
        if (dl4s_hip_alloc(ctx, sizes[i], &bufs[i]) != DL4S_HIP_OK) {
            for (int j = 0; j < i; ++j) (void)dl4s_hip_free(ctx, bufs[j]);
            return DL4S_HIP_EOOM;
        }
    float *S = static_cast<float *>(bufs[0]), *dP = static_cast<float *>(bufs[1]), *qs = static_cast<float *>(bufs[2]);
    // A product whose own shape would send it to the skinny kernels (few output blocks) comes here with a batch of pairs: when
    // the batch as a whole has more blocks than that rule's bound, the tiled kernels take it.
    const auto gemm = [&](dl4s_hip_ctx *c, const float *a, int64_t ar, int64_t ac, int64_t as, const float *b, int64_t br, int64_t bc,
                          int64_t bs, float *r, int64_t rs, int64_t n, float alpha, float beta, int ta, int tb) {
        const int64_t M = ta ? ac : ar, N = tb ? br : bc;
        if (n * ((M + 31) / 32) * ((N + 31) / 32) > 2ll * c->cu_count)
            return dl4s::gemm_batched_tiled(c, a, ar, ac, as, b, br, bc, bs, r, rs, n, alpha, beta, ta, tb);
        return dl4s_hip_gemm_batched_f32(c, a, ar, ac, as, b, br, bc, bs, r, rs, n, alpha, beta, ta, tb);
    };
    // the plain causal mask: blocks of query rows against the keys up to the block's last row (with key lengths a sequence
    // of length zero spreads its weights over every key, so that kind visits them all)
    const bool blocks = m.kind == DL4S_MASK_CAUSAL && !strict && Lq > 512;
    const int64_t QB = blocks ? 512 : Lq;
    for (int64_t p0 = 0; p0 < pairs && rc == DL4S_HIP_OK; p0 += chunk) {
        const int64_t n = std::min(chunk, pairs - p0);
        const float *qc = q + p0 * Lq * d, *kc = k + p0 * Lk * d, *vc = v + p0 * Lk * d, *gc = dout + p0 * Lq * d;
        float *dqc = dq + p0 * Lq * d, *dkc = dk + p0 * Lk * d, *dvc = dv + p0 * Lk * d;
        const long long n4 = n * Lq * d / 4;
        hipLaunchKernelGGL(sdpa_bwd_wide_scale_q, dim3((unsigned)std::min<long long>((n4 + 255) / 256, 65536)), dim3(256), 0, ctx->stream, qc,
                           qs, n4, rT);
        rc = dl4s::launch_status("sdpa_bwd_wide_scale_q");
        if (blocks && rc == DL4S_HIP_OK) rc = dl4s_hip_fill_f32(ctx, 0.f, dkc, n * Lk * d);     // the blocks add into dk and dv
        if (blocks && rc == DL4S_HIP_OK) rc = dl4s_hip_fill_f32(ctx, 0.f, dvc, n * Lk * d);
        for (int64_t i0 = 0; i0 < Lq && rc == DL4S_HIP_OK; i0 += QB) {
            const int64_t nq = std::min(QB, Lq - i0);
            const int64_t nk = blocks ? std::min(Lk, i0 + nq) : Lk;      // keys beyond the block's last row are blocked for all of it
            const float beta = blocks ? 1.0f : 0.0f;
            // S2 = qs . k^T
            rc = gemm(ctx, qs + i0 * d, nq, d, Lq * d, kc, nk, d, Lk * d, S, nq * nk, n, 1.0f, 0.0f, 0, 1);
            if (rc == DL4S_HIP_OK)      // dP = dout . v^T
                rc = gemm(ctx, gc + i0 * d, nq, d, Lq * d, vc, nk, d, Lk * d, dP, nq * nk, n, 1.0f, 0.0f, 0, 1);
            if (rc == DL4S_HIP_OK) {
                hipLaunchKernelGGL(sdpa_bwd_wide_weights, dim3((unsigned)(n * nq)), dim3(256), 0, ctx->stream, S, dP, m, (long long)p0, (int)H, (int)i0,
                                   (int)nq, (int)nk);
                rc = dl4s::launch_status("sdpa_bwd_wide_weights");
            }
            if (rc == DL4S_HIP_OK)      // dv (+)= P^T . dout
                rc = gemm(ctx, S, nq, nk, nq * nk, gc + i0 * d, nq, d, Lq * d, dvc, Lk * d, n, 1.0f, beta, 1, 0);
            if (rc == DL4S_HIP_OK)      // dk (+)= rT * dS^T . q
                rc = gemm(ctx, dP, nq, nk, nq * nk, qc + i0 * d, nq, d, Lq * d, dkc, Lk * d, n, rT, beta, 1, 0);
            if (rc == DL4S_HIP_OK)      // dq = rT * dS . k
                rc = gemm(ctx, dP, nq, nk, nq * nk, kc, nk, d, Lk * d, dqc + i0 * d, Lq * d, n, rT, 0.0f, 0, 0);
        }
    }
    // the pool hands a block out again only to work enqueued later on the same stream
    for (int i = 0; i < 3; ++i) (void)dl4s_hip_free(ctx, bufs[i]);
    return rc;
}

}  // namespace

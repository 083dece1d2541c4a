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
// gradient scratch bound.  Under the plain causal mask (without DL4S_SDPA_STRICT, more than 512 queries) the keys beyond a
// query are left out - their weights are exactly zero: the score products compute only the tiles that reach the diagonal and
// the three products that contract the weights start or stop at the diagonal tile (the triangle forms of the tiled GEMM
// kernels); with a key count that is no multiple of 4 or operands off the 16-byte grid, which those kernels do not take,
// the queries go in blocks of 512 rows that contract the keys up to their last row and add their dk / dv contributions
// block after block.  Every other mask kind visits every key.  Deterministic: no atomics, every sum in a fixed order.
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
// tri (plain causal mask only): the keys beyond the row's query were never computed and weigh exactly zero; they are not
// read, and zeros are written up to the end of the row's 128-key tile, which is as far as the products after this read.
__global__ __launch_bounds__(256) void sdpa_bwd_wide_weights(float *__restrict__ S, float *__restrict__ dP, MaskArgs mask, long long pair0,
                                                             int H, int i0, int nq, int Lk, int tri) {
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
    const int Lrow = Lk;
    if (tri) Lk = min(Lk, qi + 1);
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
    if (tri)
        for (int j = Lk + threadIdx.x; j < min(Lrow, (qi / 128 + 1) * 128); j += 256) srow[j] = drow[j] = 0.f;
}

// The same step for rows of at most 256 * NV keys (a multiple of 4): one wavefront per row, which holds its scores and dP
// values in registers from one read to one write - no pass goes back to memory and nothing waits on a workgroup barrier.
// rows: the launch's row count (pairs x nq).  Lane l holds the keys 4 (64 it + l) .. + 3 of step it; sums per lane in that
// order, then across the lanes.
template <int NV>
__global__ __launch_bounds__(256, NV <= 4 ? 8 : NV <= 8 ? 4 : 2) void sdpa_bwd_wide_weights_rows(float *__restrict__ S, float *__restrict__ dP, MaskArgs mask, long long pair0,
                                                                  int H, int i0, int nq, int Lk, long long rows, int tri) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const long long bh = pair0 + row / nq;
    const int qi = i0 + (int)(row % nq);
    const int b = (int)(bh / H), hh = (int)(bh % H);
    const bool causal = mask.kind == DL4S_MASK_CAUSAL || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS;
    const bool lens = mask.kind == DL4S_MASK_KEY_LENGTHS || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS;
    const int len = lens ? mask.lengths[b] : Lk;
    const float *mrow = mask.kind == DL4S_MASK_DENSE_F32 ? mask.dense + b * mask.sb + hh * mask.sh + qi * mask.sq : nullptr;
    f32x4 *srow = reinterpret_cast<f32x4 *>(S + row * Lk), *drow = reinterpret_cast<f32x4 *>(dP + row * Lk);
    // quads read (tri: those that hold a key up to the query) and written (tri: to the end of the query's 128-key tile)
    const int nv = tri ? min(Lk >> 2, (qi >> 2) + 1) : Lk >> 2;
    const int nvw = tri ? min(Lk >> 2, (qi / 128 + 1) * 32) : Lk >> 2;
    f32x4 s[NV], g[NV];
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int c = it * 64 + lane;
        if (c < nv) {
            s[it] = srow[c];
            g[it] = drow[c];
        } else {        // past the row: weight exactly zero
            s[it] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            g[it] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int j0 = 4 * (it * 64 + lane);
        if (j0 < 4 * nv) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = j0 + e;
                float x = s[it][e];
                if (mrow) x = dense_masked2(x, mrow[j * mask.sk]);
                else if (tri && j > qi) x = -INFINITY;
                else if ((causal && j > qi) || (lens && j >= len)) x = blocked_score2(x);
                s[it][e] = x;
                mx = fmaxf(mx, x);      // a NaN score does not move the maximum; it makes the sum NaN below, as in the reference
            }
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float m = (mx == -INFINITY) ? 0.f : mx;     // a row of -inf: weights 0 / 0
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < NV; ++it)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s[it][e] = fast_exp2(s[it][e] - m);
            sum += s[it][e];
        }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    const float inv = 1.0f / sum;
    float dsum = 0.f;
#pragma unroll
    for (int it = 0; it < NV; ++it)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s[it][e] *= inv;
            dsum += s[it][e] * g[it][e];
        }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dsum += __shfl_xor(dsum, o, 64);
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int c = it * 64 + lane;
        if (c < nvw) {
            f32x4 ds;
#pragma unroll
            for (int e = 0; e < 4; ++e) ds[e] = s[it][e] * (g[it][e] - dsum);
            srow[c] = s[it];
            drow[c] = ds;
        }
    }
}

// Launches the weights step for one block of query rows: the register form when the row fits it
int launch_wide_weights(dl4s_hip_ctx *ctx, float *S, float *dP, const MaskArgs &m, long long pair0, int H, int i0, int nq, int nk, long long rows,
                        int tri) {
    const dim3 grid4((unsigned)((rows + 3) / 4)), block(256);
    if (nk % 4 == 0 && nk <= 1024)
        hipLaunchKernelGGL(sdpa_bwd_wide_weights_rows<4>, grid4, block, 0, ctx->stream, S, dP, m, pair0, H, i0, nq, nk, rows, tri);
    else if (nk % 4 == 0 && nk <= 2048)
        hipLaunchKernelGGL(sdpa_bwd_wide_weights_rows<8>, grid4, block, 0, ctx->stream, S, dP, m, pair0, H, i0, nq, nk, rows, tri);
    else if (nk % 4 == 0 && nk <= 4096)
        hipLaunchKernelGGL(sdpa_bwd_wide_weights_rows<16>, grid4, block, 0, ctx->stream, S, dP, m, pair0, H, i0, nq, nk, rows, tri);
    else
        hipLaunchKernelGGL(sdpa_bwd_wide_weights, dim3((unsigned)rows), block, 0, ctx->stream, S, dP, m, pair0, H, i0, nq, nk, tri);
    return dl4s::launch_status("sdpa_bwd_wide_weights");
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
    // the call's pairs as a whole have more blocks than that rule's bound, the tiled kernels take it (all the pairs, not the
    // chunk's: a call gets the same kernels, and with them the same bits, whatever the scratch bound makes of its chunks).
    const auto gemm = [&](dl4s_hip_ctx *c, const float *a, int64_t ar, int64_t ac, int64_t as, const float *b, int64_t br, int64_t bc,
                          int64_t bs, float *r, int64_t rs, int64_t n, float alpha, float beta, int ta, int tb, int triangle) {
        const int64_t M = ta ? ac : ar, N = tb ? br : bc;
        if (triangle || pairs * ((M + 31) / 32) * ((N + 31) / 32) > 2ll * c->cu_count)
            return dl4s::gemm_batched_tiled(c, a, ar, ac, as, b, br, bc, bs, r, rs, n, alpha, beta, ta, tb, triangle);
        return dl4s_hip_gemm_batched_f32(c, a, ar, ac, as, b, br, bc, bs, r, rs, n, alpha, beta, ta, tb);
    };
    // the plain causal mask: blocks of query rows against the keys up to the block's last row (with key lengths a sequence
    // of length zero spreads its weights over every key, so that kind visits them all)
    const bool skip = m.kind == DL4S_MASK_CAUSAL && !strict && Lq > 512;
    // ... in one piece where the tiled GEMM kernels take every operand (extents in multiples of 4 on the 16-byte grid,
    // 32-bit byte offsets): the score products leave out the tiles beyond the diagonal, the three products that contract
    // the weights stop (or start) at the diagonal tile.  Otherwise in blocks of queries.
    const auto on_grid = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool tri = skip && Lk % 4 == 0 && Lk < (1ll << 21) && Lq * Lk < (1ll << 29) && Lq * d < (1ll << 29) && Lk * d < (1ll << 29) &&
                     on_grid(q) && on_grid(k) && on_grid(v) && on_grid(dout) && on_grid(dq) && on_grid(dk) && on_grid(dv);
    const bool blocks = skip && !tri;
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
            rc = gemm(ctx, qs + i0 * d, nq, d, Lq * d, kc, nk, d, Lk * d, S, nq * nk, n, 1.0f, 0.0f, 0, 1, tri ? 1 : 0);
            if (rc == DL4S_HIP_OK)      // dP = dout . v^T
                rc = gemm(ctx, gc + i0 * d, nq, d, Lq * d, vc, nk, d, Lk * d, dP, nq * nk, n, 1.0f, 0.0f, 0, 1, tri ? 1 : 0);
            if (rc == DL4S_HIP_OK)
                rc = launch_wide_weights(ctx, S, dP, m, (long long)p0, (int)H, (int)i0, (int)nq, (int)nk, (long long)(n * nq), tri ? 1 : 0);
            if (rc == DL4S_HIP_OK)      // dv (+)= P^T . dout
                rc = gemm(ctx, S, nq, nk, nq * nk, gc + i0 * d, nq, d, Lq * d, dvc, Lk * d, n, 1.0f, beta, 1, 0, tri ? 2 : 0);
            if (rc == DL4S_HIP_OK)      // dk (+)= rT * dS^T . q
                rc = gemm(ctx, dP, nq, nk, nq * nk, qc + i0 * d, nq, d, Lq * d, dkc, Lk * d, n, rT, beta, 1, 0, tri ? 2 : 0);
            if (rc == DL4S_HIP_OK)      // dq = rT * dS . k
                rc = gemm(ctx, dP, nq, nk, nq * nk, kc, nk, d, Lk * d, dqc + i0 * d, Lq * d, n, rT, 0.0f, 0, 0, tri ? 3 : 0);
        }
    }
    // the pool hands a block out again only to work enqueued later on the same stream
    for (int i = 0; i < 3; ++i) (void)dl4s_hip_free(ctx, bufs[i]);
    return rc;
}

}  // namespace

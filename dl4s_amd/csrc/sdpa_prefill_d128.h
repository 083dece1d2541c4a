// Fused attention forward for head dims above 64 and up to 128 (key dim = value dim, a multiple of 4): the same
// transposed two-contraction scheme as sdpa_prefill_f32_d64 (sdpa_prefill.hip) on tiles that are 128 wide.  Included by
// sdpa_prefill.hip only.
//
//   S^T[key, query] = K[key, :] . Q[query, :]       64 MFMA steps: step j contracts d = 64*half + j
//   O^T[d,   query] = V[key, d]^T . P^T[key, query]  four accumulators: accumulator c row i is d = 4*i + c, so that a lane
//                                                   reads its four V values of a key with one 128-bit LDS read and
//                                                   stores four consecutive outputs with one 128-bit store
//
// One workgroup = 4 wavefronts = 128 queries of one (batch, head), K/V in double-buffered LDS tiles of 32 keys on a
// 132-float row stride (2 x 2 x 32 x 132 floats = 66 KiB: two workgroups per CU).  Head dims below 128 are padded with
// zero columns on the fly like the 64-wide kernels do.  Mask kinds, tile skipping, the token-major layout, the work
// order and the row statistics are those of the 64-wide kernel.  Small launches are split over the keys across
// workgroups (grid.y shares per block, partial results in a scratch buffer, sdpa_prefill_merge_d128 adds them up).
#pragma once
#include "sdpa_common.h"

namespace {

constexpr int PART2_STRIDE = HD2 + 4;   // floats per partial row: 128 weighted sums, reference maximum, row sum, padding

// Adds up the nsplit partial results of every query row (32 lanes per row, four columns each), normalises and stores.
// A partial result whose reference maximum is -inf has seen no finite score: its sums are zeros (or NaN, which must
// survive), so it is added with factor 1.
__global__ __launch_bounds__(256) void sdpa_prefill_merge_d128(const float *__restrict__ part, float *__restrict__ out,
                                                               float *__restrict__ stats, int nsplit, long long rows, int H, int Lq,
                                                               int hd, int token_major) {
    const long long row = (long long)blockIdx.x * 8 + (threadIdx.x >> 5);
    const int c = threadIdx.x & 31;
    if (row >= rows) return;
    float m_all = -INFINITY;
    for (int s = 0; s < nsplit; ++s) m_all = fmaxf(m_all, part[((long long)s * rows + row) * PART2_STRIDE + HD2]);
    const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
    float l_tot = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nsplit; ++s) {
        const float *p = part + ((long long)s * rows + row) * PART2_STRIDE;
        const float ms = p[HD2];
        const float f = (ms == -INFINITY) ? 1.0f : fast_exp2(ms - m_ref);
        l_tot += p[HD2 + 1] * f;
        const f32x4 x = *reinterpret_cast<const f32x4 *>(p + 4 * c);
        acc.x += x.x * f; acc.y += x.y * f; acc.z += x.z * f; acc.w += x.w * f;
    }
    const float inv = 1.0f / l_tot;
    if (stats && c == 0) { stats[2 * row] = m_ref; stats[2 * row + 1] = inv; }
    if (4 * c < hd) {
        const long long bh = row / Lq, qi = row % Lq, b = bh / H, hh = bh % H;
        const long long at = token_major ? (((b * Lq + qi) * H + hh) * hd) : (row * hd);
        acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
        *reinterpret_cast<f32x4 *>(out + at + 4 * c) = acc;
    }
}

template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_prefill_f32_d128(const float *__restrict__ q, const float *__restrict__ k,
                                                                 const float *__restrict__ v, float *__restrict__ out, int H,
                                                                 int Lq, int Lk, float rT, MaskArgs mask, int strict, int nqb,
                                                                 int total_blocks, int lpt, int token_major,
                                                                 float *__restrict__ stats, int hd, int nsplit,
                                                                 float *__restrict__ part, int shares_adjacent) {
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                      // [2][BN][LSTR2]
    float *Vs = lds + 2 * TILE2_FLOATS;   // [2][BN][LSTR2]
    int bh, unit;
    // Key split with blocks of different length.  A launch that is resident at once: the workgroups of an odd share walk the
    // block order backwards, so that the CU that got the longest block's first share gets the shortest block's second (the
    // dispatcher deals both rounds out in the same order).  A larger launch: the shares of a block next to each other in the
    // longest-first order, so that the dispatcher hands the short blocks to whichever CU is free first.
    int blk = ((lpt & 1) && (blockIdx.y & 1) && !shares_adjacent) ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;
    int sp = blockIdx.y;
    if ((lpt & 1) && shares_adjacent) dl4s_work_order::split_item_at(blockIdx.x, blockIdx.y, gridDim.x, nsplit, blk, sp);
    if (!dl4s_work_order::work_item_at(blk, nqb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, half = lane >> 5, ln = lane & 31;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int qb = nqb - 1 - unit;   // longest rows first
    const int q0 = qb * BM + wave * 32;
    const int qi = q0 + ln;
    const int qic = qi < Lq ? qi : Lq - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    // keys this workgroup / wavefront has to visit (see sdpa_prefill_f32_d64)
    int kend = Lk, wkend = Lk;
    bool skip_ones = false;
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { kend = min(kend, qb * BM + BM); wkend = min(wkend, q0 + 32); }
        if (LENS) { kend = min(kend, len); wkend = min(wkend, len); }
        if (DENSE && mask.cls) dense_key_bounds(mask, b, hh, qb * BM, wave, Lq, Lk, kend, wkend, skip_ones);
    }
    const int ntiles = (kend + BN - 1) / BN;

    // Q fragment: Q[qi][64*half + s] * rT (one rounding, like the reference's q / temperature) * log2(e)
    float qr[64];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * 64;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * 64 + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E;
            qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E;
            qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // global -> LDS staging: thread covers rows (i*8 + tid/32), 4 floats at column (tid%32)*4; buffer loads with the
    // whole byte offset in the range-checked vector operand (rows past Lk and columns past hd read zeros)
    const int ld_row = tid >> 5, ld_col = (tid & 31) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off0 = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned row8_bytes = 8u * rs * 4u, tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[4], vst[4];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int o = (int)(ld_off0 + t * tile_bytes + i * row8_bytes);
            kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
            vst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int off = buf * TILE2_FLOATS + (i * 8 + ld_row) * LSTR2 + ld_col;
            *reinterpret_cast<f32x4 *>(Ks + off) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + off) = vst[i];
        }
    };

    f32x16 o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[c][i] = 0.f;
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    // Key split over workgroups (small launches): workgroup blockIdx.y of nsplit takes the key tiles y, y + nsplit, ... -
    // an assignment that does not depend on how many tiles the mask lets the block skip, so skipping keeps the bits.
    if (sp < ntiles) { load_tile(sp); store_tile(0); }
    __syncthreads();

    const int k_lds = ln * LSTR2 + half * 64;        // K fragment base: row ln, columns 64*half ..
    const int v_lds = (4 * half) * LSTR2 + 4 * ln;   // V fragment base: row 4*half (+ const), columns 4*ln .. 4*ln+3
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    for (int t = sp, it = 0; t < ntiles; t += nsplit, ++it) {
        const int buf = it & 1;
        const bool more = (t + nsplit < ntiles);
        if (more) load_tile(t + nsplit);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (k0 < wkend && !(DENSE && skip_ones && cls == 1)) {
            f32x16 s0 = masked_scores<KIND, 16>(Ks + buf * TILE2_FLOATS + k_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
            // online softmax with a lazily moved reference maximum (see attend_tile in sdpa_prefill.hip)
            const float tmax = max_across_halves(max_of_16(s0));
            const bool upd = tmax - m_run > 8.0f;      // also right at m_run = -inf: +inf, or NaN for tmax = -inf
            if (__any(upd)) {
                const float m_new = fmaxf(m_run, tmax);
                const float alpha = (m_run == m_new) ? 1.0f : fast_exp2(m_run - m_new);
                m_run = m_new;
                m_use = (m_new == -INFINITY) ? 0.f : m_new;
                l_run *= alpha;
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[c][i] *= alpha;
            }
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s0[r] = fast_exp2(s0[r] - m_use);
                psum += s0[r];
            }
            l_run += psum;
            const float *Vb = Vs + buf * TILE2_FLOATS + v_lds;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const f32x4 vv = *reinterpret_cast<const f32x4 *>(Vb + (8 * (r >> 2) + (r & 3)) * LSTR2);
                o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, s0[r], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, s0[r], o[1], 0, 0, 0);
                o[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.z, s0[r], o[2], 0, 0, 0);
                o[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.w, s0[r], o[3], 0, 0, 0);
            }
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- normalise and store.  Register r of accumulator c is d = 4*(8(r/4) + 4*half + r%4) + c.
    const float l_tot = sum_across_halves(l_run);
    if (part) {   // this workgroup's share of the keys: the weighted sums as they are, with their reference maximum and row sum
        if (qi < Lq) {
            const long long pairs = total_blocks / nqb;
            float *pp = part + (((long long)sp * pairs + bh) * Lq + qi) * PART2_STRIDE;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int d0 = 4 * (8 * (r >> 2) + 4 * half + (r & 3));
                const f32x4 a = {o[0][r], o[1][r], o[2][r], o[3][r]};
                *reinterpret_cast<f32x4 *>(pp + d0) = a;
            }
            if (half == 0) { pp[HD2] = m_run; pp[HD2 + 1] = l_tot; }
        }
        return;
    }
    const float inv = 1.0f / l_tot;
    if (stats && half == 0 && qi < Lq) {
        stats[2 * ((long long)bh * Lq + qi)] = m_use;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    if (qi < Lq) {
        float *op = out + q_base + (long long)qi * rs;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int d0 = 4 * (8 * (r >> 2) + 4 * half + (r & 3));
            f32x4 a;
            a.x = o[0][r] * inv; a.y = o[1][r] * inv; a.z = o[2][r] * inv; a.w = o[3][r] * inv;
            if (d0 < hd) *reinterpret_cast<f32x4 *>(op + d0) = a;
        }
    }
}

template <int KIND>
int launch_d128(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk,
                float rT, const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit, float *part) {
    const int nqb = (Lq + BM - 1) / BM;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb >= 2) ? 1 : 0;
    if (lpt && total <= 2ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
    const size_t lds_bytes = 4 * TILE2_FLOATS * sizeof(float);
    if (dl4s::lds_limit_pending(ctx, dl4s::LDS_PREFILL_D128, KIND)) {
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_prefill_f32_d128<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        dl4s::lds_limit_done(ctx, dl4s::LDS_PREFILL_D128, KIND);
    }
    if (nsplit <= 1 || !part) { nsplit = 1; part = nullptr; }
    hipLaunchKernelGGL(sdpa_prefill_f32_d128<KIND>, dim3((unsigned)((total + 7) / 8 * 8), (unsigned)nsplit), dim3(256), lds_bytes,
                       ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt, token_major, stats, hd, nsplit, part,
                       // (two workgroups per CU are resident: B1 H24 L2048 d128 causal 348 -> 274 us; B1 H16 L2048, which fits, 166 us
                       // against 205 us with the shares adjacent)
                       ((total + 7) / 8 * 8 * nsplit > 2ll * ctx->cu_count) ? 1 : 0);
    int st = dl4s::launch_status("sdpa_prefill_f32_d128");
    if (st != DL4S_HIP_OK || nsplit == 1) return st;
    const long long rows = (long long)B * H * Lq;
    hipLaunchKernelGGL(sdpa_prefill_merge_d128, dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, ctx->stream, part, out, stats, nsplit, rows,
                       H, Lq, hd, token_major);
    return dl4s::launch_status("sdpa_prefill_merge_d128");
}

}  // namespace

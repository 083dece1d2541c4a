// Fused attention forward for head dims above 128 and up to 256 (key dim = value dim, a multiple of 4): the transposed
// two-contraction scheme of sdpa_prefill_f32_d128 on tiles that are W = 160, 192 or 256 columns wide.  Included by
// sdpa_prefill.hip only.
//
//   S^T[key, query] = K[key, :] . Q[query, :]       W/2 MFMA steps: step j contracts d = (W/2)*half + j
//   O^T[d,   query] = V[key, d]^T . P^T[key, query]  W/32 accumulators in groups of columns: the first 128 columns on four
//                                                   accumulators whose rows interleave (accumulator c row i is d = 4*i + c,
//                                                   one 128-bit LDS read per key); the columns from 128 up the same way on
//                                                   four more (W = 256: d = 128 + 4*i + c), on two (W = 192:
//                                                   d = 128 + 2*i + c, one 64-bit read) or on one (W = 160: d = 128 + i)
//
// The Q fragment (W/2 registers), the accumulators (W/2 registers) and the staged K/V pieces leave room for one wavefront per
// SIMD; K/V in double-buffered LDS tiles of 32 keys on a (W + 4)-float row stride (4 x 32 x (W + 4) floats: 98 or 130 KiB,
// one workgroup per CU).  With 2 x W/2 MFMAs per key tile against the same softmax work as the narrower kernels the matrix
// pipe stays busy nonetheless.  Mask kinds, tile skipping, the token-major layout and the work order are those of the
// 64-wide kernel, the row statistics have the form every MFMA kernel leaves.  Launches that leave CUs without a workgroup
// are split over the keys across workgroups like the 128-wide kernel's: share y of n takes the key tiles y, y + n, ..., leaves
// its weighted sums with their reference maximum and row sum in a scratch record, and sdpa_prefill_merge_wide adds the
// shares up.
#pragma once
#include "sdpa_common.h"

namespace {

template <int W> struct WideFwdTile {
    static_assert(W == 160 || W == 192 || W == 256, "tile widths above 128");
    static constexpr int LS = W + 4;              // LDS row stride (floats): 4 mod 32
    static constexpr int TF = BN * LS;            // floats per tile
    static constexpr int NC = W / 32;             // accumulators
    static constexpr int NC2 = NC - 4;            // accumulators of the columns from 128 up: 1, 2 or 4
    static constexpr int PPR = W / 4;             // 128-bit pieces per tile row
    static constexpr int NP = BN * PPR / 256;     // pieces per thread and tile: thread tid moves the pieces tid, tid + 256, ...
};

constexpr int PARTW_STRIDE = 256 + 4;   // floats per partial row: up to 256 weighted sums, reference maximum, row sum, padding

// Adds up the nsplit partial results of every query row (64 lanes per row, four columns each), normalises and stores; see
// sdpa_prefill_merge_d128.
__global__ __launch_bounds__(256) void sdpa_prefill_merge_wide(const float *__restrict__ part, float *__restrict__ out,
                                                               float *__restrict__ stats, int nsplit, long long rows, int H, int Lq,
                                                               int hd, int token_major) {
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int c = threadIdx.x & 63;
    if (row >= rows) return;
    float m_all = -INFINITY;
    for (int s = 0; s < nsplit; ++s) m_all = fmaxf(m_all, part[((long long)s * rows + row) * PARTW_STRIDE + 256]);
    const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
    float l_tot = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < nsplit; ++s) {
        const float *p = part + ((long long)s * rows + row) * PARTW_STRIDE;
        const float ms = p[256];
        const float f = (ms == -INFINITY) ? 1.0f : fast_exp2(ms - m_ref);
        l_tot += p[257] * f;
        if (4 * c < hd) {
            const f32x4 x = *reinterpret_cast<const f32x4 *>(p + 4 * c);
            acc.x += x.x * f; acc.y += x.y * f; acc.z += x.z * f; acc.w += x.w * f;
        }
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

template <int KIND, int W>
__global__ __launch_bounds__(256, 1) void sdpa_prefill_f32_wide(const float *__restrict__ q, const float *__restrict__ k,
                                                                 const float *__restrict__ v, float *__restrict__ out, int H,
                                                                 int Lq, int Lk, float rT, MaskArgs mask, int strict, int nqb,
                                                                 int total_blocks, int lpt, int token_major,
                                                                 float *__restrict__ stats, int hd, int nsplit,
                                                                 float *__restrict__ part, int shares_adjacent) {
    using WT = WideFwdTile<W>;
    constexpr int LS = WT::LS, TF = WT::TF, NC = WT::NC, NC2 = WT::NC2, NP = WT::NP, PPR = WT::PPR;
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;              // [2][BN][LS]
    float *Vs = lds + 2 * TF;     // [2][BN][LS]
    int bh, unit;
    // key split with blocks of different length: see sdpa_prefill_f32_d128
    int blk = ((lpt & 1) && (blockIdx.y & 1) && !shares_adjacent) ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;
    int sp = blockIdx.y;       // this workgroup's share of the key tiles: sp, sp + nsplit, ...
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

    // Q fragment: Q[qi][(W/2)*half + s] * rT (one rounding, like the reference's q / temperature) * log2(e)
    float qr[W / 2];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * (W / 2);
#pragma unroll
        for (int j = 0; j < W / 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * (W / 2) + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E;
            qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E;
            qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // global -> LDS staging: thread tid moves the 128-bit pieces tid, tid + 256, ... of a tile (piece p = row p / PPR,
    // columns 4 * (p % PPR) ..); buffer loads with the whole byte offset in the range-checked vector operand (rows past Lk
    // and columns past hd read zeros)
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    unsigned ld_off[NP];
    int st_off[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = tid + 256 * i, row = p / PPR, col = (p % PPR) * 4;
        ld_off[i] = col < hd ? (unsigned)(row * rs + col) * 4u : 0x80000000u;
        st_off[i] = row * LS + col;
    }
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    // One set of staging registers serves both tiles: the next K tile is in flight during the score product and goes to LDS
    // after it, then the next V tile is in flight during the weights x values product.
    f32x4 stg[NP];
    auto load_pieces = [&](const __amdgpu_buffer_rsrc_t rsrc, int t) {
#pragma unroll
        for (int i = 0; i < NP; ++i)
            stg[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(ld_off[i] + t * tile_bytes), 0, 0));
    };
    auto store_pieces = [&](float *tile) {
#pragma unroll
        for (int i = 0; i < NP; ++i) *reinterpret_cast<f32x4 *>(tile + st_off[i]) = stg[i];
    };

    f32x16 o[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[c][i] = 0.f;
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    if (sp < ntiles) {
        load_pieces(krsrc, sp);
        store_pieces(Ks);
        load_pieces(vrsrc, sp);
        store_pieces(Vs);
    }
    __syncthreads();

    const int k_lds = ln * LS + half * (W / 2);      // K fragment base: row ln, columns (W/2)*half ..
    const int v_lds = (4 * half) * LS + 4 * ln;      // V fragment base, first 128 columns: row 4*half (+ const), columns 4*ln ..
    const int v_lds2 = (4 * half) * LS + 128 + NC2 * ln;   // columns from 128 up: NC2*ln ..
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    for (int t = sp, buf = 0; t < ntiles; t += nsplit, buf ^= 1) {
        const bool more = (t + nsplit < ntiles);
        if (more) load_pieces(krsrc, t + nsplit);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        const bool visit = k0 < wkend && !(DENSE && skip_ones && cls == 1);
        f32x16 s0;
        if (visit) {
            s0 = masked_scores<KIND, W / 8>(Ks + buf * TF + k_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
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
                for (int c = 0; c < NC; ++c)
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
        }
        if (more) {
            store_pieces(Ks + (buf ^ 1) * TF);
            load_pieces(vrsrc, t + nsplit);
        }
        if (visit) {
            const float *Vb = Vs + buf * TF;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row_off = (8 * (r >> 2) + (r & 3)) * LS;
                const f32x4 va = *reinterpret_cast<const f32x4 *>(Vb + v_lds + row_off);
                o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(va.x, s0[r], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(va.y, s0[r], o[1], 0, 0, 0);
                o[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(va.z, s0[r], o[2], 0, 0, 0);
                o[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(va.w, s0[r], o[3], 0, 0, 0);
                if constexpr (NC2 == 4) {
                    const f32x4 vb = *reinterpret_cast<const f32x4 *>(Vb + v_lds2 + row_off);
                    o[4] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.x, s0[r], o[4], 0, 0, 0);
                    o[5] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.y, s0[r], o[5], 0, 0, 0);
                    o[6] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.z, s0[r], o[6], 0, 0, 0);
                    o[7] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.w, s0[r], o[7], 0, 0, 0);
                } else if constexpr (NC2 == 2) {
                    const f32x2 vb = *reinterpret_cast<const f32x2 *>(Vb + v_lds2 + row_off);
                    o[4] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.x, s0[r], o[4], 0, 0, 0);
                    o[5] = __builtin_amdgcn_mfma_f32_32x32x2f32(vb.y, s0[r], o[5], 0, 0, 0);
                } else {
                    o[4] = __builtin_amdgcn_mfma_f32_32x32x2f32(Vb[v_lds2 + row_off], s0[r], o[4], 0, 0, 0);
                }
            }
        }
        if (more) store_pieces(Vs + (buf ^ 1) * TF);
        __syncthreads();
    }

    // ---- normalise and store.  Register r of accumulator c < 4 is d = 4*(8(r/4) + 4*half + r%4) + c; of accumulator 4 + c,
    // d = 128 + NC2*(8(r/4) + 4*half + r%4) + c.
    const float l_tot = sum_across_halves(l_run);
    if (part) {   // this share's weighted sums as they are, with their reference maximum and row sum
        if (qi < Lq) {
            float *pp = part + (((long long)sp * (total_blocks / nqb) + bh) * Lq + qi) * PARTW_STRIDE;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = 8 * (r >> 2) + 4 * half + (r & 3);
                const f32x4 a = {o[0][r], o[1][r], o[2][r], o[3][r]};
                *reinterpret_cast<f32x4 *>(pp + 4 * i) = a;
                if constexpr (NC2 == 4) {
                    const f32x4 c4 = {o[4][r], o[5][r], o[6][r], o[7][r]};
                    *reinterpret_cast<f32x4 *>(pp + 128 + 4 * i) = c4;
                } else if constexpr (NC2 == 2) {
                    const f32x2 c2 = {o[4][r], o[5][r]};
                    *reinterpret_cast<f32x2 *>(pp + 128 + 2 * i) = c2;
                } else {
                    pp[128 + i] = o[4][r];
                }
            }
            if (half == 0) { pp[256] = m_run; pp[257] = l_tot; }
        }
        return;
    }
    const float inv = 1.0f / l_tot;
    if (stats && half == 0 && qi < Lq) {      // for the gradient call: a weight is 2^(s - m_use) * inv
        stats[2 * ((long long)bh * Lq + qi)] = m_use;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    if (qi < Lq) {
        float *op = out + q_base + (long long)qi * rs;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = 8 * (r >> 2) + 4 * half + (r & 3);
            const f32x4 a = {o[0][r] * inv, o[1][r] * inv, o[2][r] * inv, o[3][r] * inv};
            if (4 * i < hd) *reinterpret_cast<f32x4 *>(op + 4 * i) = a;
            const int d2 = 128 + NC2 * i;
            if constexpr (NC2 == 4) {
                const f32x4 c4 = {o[4][r] * inv, o[5][r] * inv, o[6][r] * inv, o[7][r] * inv};
                if (d2 < hd) *reinterpret_cast<f32x4 *>(op + d2) = c4;
            } else if constexpr (NC2 == 2) {     // head dims are multiples of 4 and d2 is even: a pair is inside or outside as a whole
                const f32x2 c2 = {o[4][r] * inv, o[5][r] * inv};
                if (d2 < hd) *reinterpret_cast<f32x2 *>(op + d2) = c2;
            }
        }
        if constexpr (NC2 == 1) {     // registers 4g .. 4g+3 of the fifth accumulator are four consecutive columns
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d2 = 128 + 8 * g + 4 * half;
                const f32x4 c4 = {o[4][4 * g + 0] * inv, o[4][4 * g + 1] * inv, o[4][4 * g + 2] * inv, o[4][4 * g + 3] * inv};
                if (d2 < hd) *reinterpret_cast<f32x4 *>(op + d2) = c4;
            }
        }
    }
}

template <int KIND, int W>
int launch_wide_kind(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk,
                     float rT, const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit, float *part) {
    const int nqb = (Lq + BM - 1) / BM;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb >= 2) ? 1 : 0;
    if (lpt && total <= 1ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
    const size_t lds_bytes = 4 * WideFwdTile<W>::TF * sizeof(float);
    constexpr int family = W == 160 ? dl4s::LDS_PREFILL_W160 : (W == 192 ? dl4s::LDS_PREFILL_W192 : dl4s::LDS_PREFILL_W256);
    if (dl4s::lds_limit_pending(ctx, family, KIND)) {
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_prefill_f32_wide<KIND, W>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        dl4s::lds_limit_done(ctx, family, KIND);
    }
    if (nsplit <= 1 || !part) { nsplit = 1; part = nullptr; }
    hipLaunchKernelGGL((sdpa_prefill_f32_wide<KIND, W>), dim3((unsigned)((total + 7) / 8 * 8), (unsigned)nsplit), dim3(256), lds_bytes,
                       ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt, token_major, stats, hd, nsplit, part,
                       // (one workgroup per CU is resident: B1 H16 L2048 d256 causal 514 -> 353 us, B1 H8 L4096 967 -> 644 us)
                       ((total + 7) / 8 * 8 * nsplit > (long long)ctx->cu_count) ? 1 : 0);
    const int st = dl4s::launch_status("sdpa_prefill_f32_wide");
    if (st != DL4S_HIP_OK || nsplit == 1) return st;
    const long long rows = (long long)B * H * Lq;
    hipLaunchKernelGGL(sdpa_prefill_merge_wide, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, ctx->stream, part, out, stats, nsplit, rows,
                       H, Lq, hd, token_major);
    return dl4s::launch_status("sdpa_prefill_merge_wide");
}

template <int W>
int launch_wide(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk, float rT,
                const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit = 1, float *part = nullptr) {
    switch (m.kind) {
        case DL4S_MASK_NONE: return launch_wide_kind<DL4S_MASK_NONE, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_DENSE_F32: return launch_wide_kind<DL4S_MASK_DENSE_F32, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_CAUSAL: return launch_wide_kind<DL4S_MASK_CAUSAL, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_KEY_LENGTHS: return launch_wide_kind<DL4S_MASK_KEY_LENGTHS, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        default: return launch_wide_kind<DL4S_MASK_CAUSAL_OR_KEY_LENGTHS, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
    }
}

}  // namespace

// Gradients of the fused attention for head dims above 64 and up to 128 (multiples of 4): the deterministic kernels of
// sdpa_backward.hip on tiles that are W = 128 columns wide, W = 96 for head dims up to 96, or the 80-column form of the
// latter for head dims up to 80.  Included by sdpa_backward.hip only.
//
// The operand layouts follow the forward kernels of the same width.  A score product contracts d = (W/2)*half + j over
// W/2 MFMA steps.  A transposed accumulation (dQ^T, dK^T, dV^T) uses W/32 accumulators.  W = 128: their rows interleave
// (accumulator c row i is d = 4*i + c), fed by one 128-bit LDS read per key (query) and stored 128 bits at a time.
// W = 96: accumulator c row i is d = 32*c + i, the operand read a float at a time (sdpa_prefill_w96.h).  The row
// fragments of two operands (2 x W/2 registers) and up to 2 x W/32 accumulators leave room for one wavefront per SIMD
// only, so these kernels run at a lower MFMA rate than the 64-wide ones; a head dim of 96 issues three quarters of the
// MFMAs it would on 128-wide tiles.
#pragma once
#include "sdpa_common.h"

namespace {

// D[b,h,i] = sum_d dout[i][d] * out[i][d] for head dims up to 128: 32 lanes per row, eight rows per workgroup
__global__ __launch_bounds__(256) void sdpa_bwd_rowdot128(const float *__restrict__ out, const float *__restrict__ dout,
                                                          float *__restrict__ D, int H, int Lq, long long rows, int token_major, int hd) {
    const long long r = (long long)blockIdx.x * 8 + (threadIdx.x >> 5);
    const int c = (threadIdx.x & 31) * 4;
    float acc = 0.f;
    if (r < rows && c < hd) {
        const long long bh = r / Lq, qi = r % Lq;
        const long long off = token_major ? (((bh / H) * Lq + qi) * H + bh % H) * hd : r * hd;
        const f32x4 a = *reinterpret_cast<const f32x4 *>(out + off + c);
        const f32x4 g = *reinterpret_cast<const f32x4 *>(dout + off + c);
        acc = a.x * g.x + a.y * g.y + a.z * g.z + a.w * g.w;
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 8, 64);
    acc += __shfl_xor(acc, 4, 64);
    acc += __shfl_xor(acc, 2, 64);
    acc += __shfl_xor(acc, 1, 64);
    if (r < rows && (threadIdx.x & 31) == 0) D[r] = acc;
}

// 32 x 32 product tile over a contraction of 8 NJ columns: A rows from LDS (row lane % 32, columns (W/2)*half + 4j), B
// from the lane's 4 NJ registers
template <int NJ>
__device__ __forceinline__ f32x16 tile_product_w(const float *Ab, const float (&br)[4 * NJ]) {
    f32x16 acc;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const f32x4 a0 = *reinterpret_cast<const f32x4 *>(Ab + 4 * j);
        if (j == 0) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, br[0], zero, 0, 0, 0);
        } else {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, br[4 * j + 0], acc, 0, 0, 0);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, br[4 * j + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, br[4 * j + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, br[4 * j + 3], acc, 0, 0, 0);
    }
    return acc;
}

// What depends on the tile width W.  W = 80 (head dims up to 80): the LDS tiles of W = 96 (columns from the head dim up are
// zeros either way), score products that contract 40 steps per half, and transposed accumulations whose columns 64 .. 79
// live in two 16 x 16 accumulators on v_mfma_f32_16x16x4_f32 (the wavefront's columns 0-15 and 16-31; lane: column =
// lane % 16, rows d = 64 + 4 * (lane / 16) + i) fed through v_permlane16_swap - see attend_tile_16 in sdpa_prefill_narrow.h.
template <int W> struct WideTile {
    static constexpr int SW = W == 80 ? 96 : W;   // columns of a tile in LDS
    static constexpr int LS = SW + 4;             // LDS row stride (floats): 4 mod 32
    static constexpr int TF = BN * LS;            // floats per tile
    static constexpr int HALF = W / 2;            // columns a half of the wavefront contracts in a score product
    static constexpr int NJ = W / 8;              // 128-bit reads per row fragment
    static constexpr int NC = W == 80 ? 2 : W / 32;   // 32 x 32 accumulators of a transposed product
    static constexpr int PPR = SW / 4;            // 128-bit pieces per tile row
    static constexpr int NP = BN * PPR / 256;     // pieces per thread and tile: thread tid moves the pieces tid, tid + 256, ...
    // the accumulators of one transposed product (column = the lane's query or key); g: W = 80 only
    struct Acc {
        f32x16 a[NC];
        f32x4 g[2];
    };
    static __device__ __forceinline__ void zero(Acc &x) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int i = 0; i < 16; ++i) x.a[c][i] = 0.f;
        x.g[0] = f32x4{0.f, 0.f, 0.f, 0.f};
        x.g[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // acc += A^T . B where A is a [32][LS] LDS tile and B the accumulator-layout tile b
    static __device__ __forceinline__ void accumulate(const float *tile, const int half, const int ln, const int lane, const f32x16 &b,
                                                      Acc &acc) {
        const float *At = tile + (4 * half) * LS + (W == 128 ? 4 * ln : ln);   // the lane's base: row 4*half + const
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float *ar = At + (8 * (r >> 2) + (r & 3)) * LS;
            if constexpr (W == 128) {
                const f32x4 a = *reinterpret_cast<const f32x4 *>(ar);
                acc.a[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b[r], acc.a[0], 0, 0, 0);
                acc.a[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b[r], acc.a[1], 0, 0, 0);
                acc.a[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b[r], acc.a[2], 0, 0, 0);
                acc.a[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b[r], acc.a[3], 0, 0, 0);
            } else {
#pragma unroll
                for (int c = 0; c < NC; ++c) acc.a[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(ar[32 * c], b[r], acc.a[c], 0, 0, 0);
            }
        }
        if constexpr (W == 80) {
            const int slot = lane >> 4;
            const float *At16 = tile + ((slot & 1) + 4 * (slot >> 1)) * LS + 64 + (lane & 15);
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(b[2 * p]), __float_as_uint(b[2 * p + 1]), false, false);
                const float a = At16[(8 * (p >> 1) + 2 * (p & 1)) * LS];
                acc.g[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, __uint_as_float(sw[0]), acc.g[0], 0, 0, 0);
                acc.g[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, __uint_as_float(sw[1]), acc.g[1], 0, 0, 0);
            }
        }
    }
    // Stores the wavefront's 32 rows row0 .. row0 + 31 (those below nrows) of the transposed accumulators, scaled, to
    // base[row * stride + 0 .. ncols - 1]: the lane's own row row0 + ln from the 32 x 32 accumulators, the rows
    // row0 + 16 g + lane % 16 from the 16 x 16 ones.
    static __device__ __forceinline__ void store_rows(float *base, const long long stride, const int row0, const int nrows, const Acc &acc,
                                                      const float scale, const int half, const int ln, const int lane, const int ncols) {
        if (row0 + ln < nrows) {
            float *p = base + (long long)(row0 + ln) * stride;
            if constexpr (W == 128) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int d0 = 4 * (8 * (r >> 2) + 4 * half + (r & 3));
                    f32x4 a;
                    a.x = acc.a[0][r] * scale; a.y = acc.a[1][r] * scale; a.z = acc.a[2][r] * scale; a.w = acc.a[3][r] * scale;
                    if (d0 < ncols) *reinterpret_cast<f32x4 *>(p + d0) = a;
                }
            } else {
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d0 = 32 * c + 8 * g + 4 * half;
                        const f32x4 a = {acc.a[c][4 * g + 0] * scale, acc.a[c][4 * g + 1] * scale, acc.a[c][4 * g + 2] * scale,
                                         acc.a[c][4 * g + 3] * scale};
                        if (d0 < ncols) *reinterpret_cast<f32x4 *>(p + d0) = a;
                    }
            }
        }
        if constexpr (W == 80) {
            const int d0 = 64 + 4 * (lane >> 4);
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const int row = row0 + 16 * g + (lane & 15);
                const f32x4 a = {acc.g[g].x * scale, acc.g[g].y * scale, acc.g[g].z * scale, acc.g[g].w * scale};
                if (row < nrows && d0 < ncols) *reinterpret_cast<f32x4 *>(base + (long long)row * stride + d0) = a;
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------ dQ
template <int KIND, int W = 128>
__global__ __launch_bounds__(256, 1) void sdpa_bwd_dq_f32_d128(const float *__restrict__ q, const float *__restrict__ k,
                                                                const float *__restrict__ v, const float *__restrict__ dout,
                                                                const float *__restrict__ stats, const float *__restrict__ D,
                                                                float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                                MaskArgs mask, int strict, int nqb, int total_blocks, int lpt,
                                                                int token_major, int hd) {
    using WT = WideTile<W>;
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                      // [2][BN][WT::LS]
    float *Vs = lds + 2 * WT::TF;   // [2][BN][WT::LS]
    int bh, unit;
    if (!work_item(nqb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, ln = lane & 31;

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

    int kend = Lk, wkend = Lk;
    bool skip_ones = false;
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { kend = min(kend, qb * BM + BM); wkend = min(wkend, q0 + 32); }
        if (LENS) { kend = min(kend, len); wkend = min(wkend, len); }
        if (DENSE && mask.cls) dense_key_bounds(mask, b, hh, qb * BM, wave, Lq, Lk, kend, wkend, skip_ones);
    }
    const int ntiles = (kend + BN - 1) / BN;

    float qr[WT::HALF], gr[WT::HALF];   // the lane's Q fragment (scaled as in the forward pass) and dout fragment, columns (W/2)*half ..
    {
        const float *qp = q + q_base + (long long)qic * rs + half * WT::HALF;
        const float *gp = dout + q_base + (long long)qic * rs + half * WT::HALF;
#pragma unroll
        for (int j = 0; j < WT::NJ; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
            if (half * WT::HALF + 4 * j < hd) {
                t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
                g = *reinterpret_cast<const f32x4 *>(gp + 4 * j);
            }
            qr[4 * j + 0] = (t.x * rT) * LOG2E; qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E; qr[4 * j + 3] = (t.w * rT) * LOG2E;
            gr[4 * j + 0] = g.x; gr[4 * j + 1] = g.y; gr[4 * j + 2] = g.z; gr[4 * j + 3] = g.w;
        }
    }
    const float m_i = stats[2 * ((long long)bh * Lq + qic)];
    const float rl_i = stats[2 * ((long long)bh * Lq + qic) + 1];
    const float D_i = D[(long long)bh * Lq + qic];

    // staging: thread tid moves the 128-bit pieces tid, tid + 256, ... of a tile (row piece / PPR, column 4 * (piece % PPR))
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    unsigned ld_off[WT::NP];
    int lds_off[WT::NP];
#pragma unroll
    for (int i = 0; i < WT::NP; ++i) {
        const int pc = tid + 256 * i, row = pc / WT::PPR, col = (pc % WT::PPR) * 4;
        ld_off[i] = col < hd ? (unsigned)(row * rs + col) * 4u : 0x80000000u;
        lds_off[i] = row * WT::LS + col;
    }
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[WT::NP], vst[WT::NP];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i) {
            const int o = (int)(ld_off[i] + t * tile_bytes);
            kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
            vst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i) {
            *reinterpret_cast<f32x4 *>(Ks + buf * WT::TF + lds_off[i]) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + buf * WT::TF + lds_off[i]) = vst[i];
        }
    };

    typename WT::Acc acc;   // dQ^T
    WT::zero(acc);

    if (ntiles > 0) { load_tile(0); store_tile(0); }
    __syncthreads();

    const int row_lds = ln * WT::LS + half * WT::HALF;  // row-fragment base (S^T and dP^T products)
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1 < ntiles);
        if (more) load_tile(t + 1);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (k0 < wkend && !(DENSE && skip_ones && cls == 1)) {
            f32x16 p = masked_scores<KIND, WT::NJ>(Ks + buf * WT::TF + row_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = fast_exp2(p[r] - m_i) * rl_i;                    // the forward pass's weights
            const f32x16 dp = tile_product_w<WT::NJ>(Vs + buf * WT::TF + row_lds, gr);            // dP^T = V . dout^T
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = p[r] * (dp[r] - D_i);                            // dS^T
            WT::accumulate(Ks + buf * WT::TF, half, ln, lane, p, acc);               // dQ^T += K^T . dS^T
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    WT::store_rows(dq + q_base, rs, q0, Lq, acc, rT, half, ln, lane, hd);
}

// ------------------------------------------------------------------------------------------------ dK, dV
// WRITE_DS: every visited tile of dS is also stored to ds [batch*head][Lkp][Lqp] for sdpa_bwd_dq_from_ds_f32_d128 (the
// layout and rules of the 64-wide kernels).
// nsplit > 1 (small launches: the kernel runs one workgroup per CU): workgroup blockIdx.y of nsplit takes the query tiles
// y, y + nsplit, ... of its key block - an assignment by tile index, whatever the mask lets the block skip - and leaves its
// unscaled sums in part [share][dk | dv][batch*head*Lk][128]; sdpa_bwd_merge_d128 adds the shares up in order.
template <int KIND, bool WRITE_DS = false, int W = 128>
__global__ __launch_bounds__(256, 1) void sdpa_bwd_dkv_f32_d128(const float *__restrict__ q, const float *__restrict__ k,
                                                                 const float *__restrict__ v, const float *__restrict__ dout,
                                                                 const float *__restrict__ stats, const float *__restrict__ D,
                                                                 float *__restrict__ dk, float *__restrict__ dv, int H, int Lq,
                                                                 int Lk, float rT, MaskArgs mask, int strict, int nkb,
                                                                 int total_blocks, int lpt, int token_major, int hd,
                                                                 float *__restrict__ ds = nullptr, int nsplit = 1,
                                                                 float *__restrict__ part = nullptr, int shares_adjacent = 0) {
    using WT = WideTile<W>;
    extern __shared__ __align__(16) float lds[];
    float *Qs = lds;                        // [2][BN][WT::LS]  q * rT * log2(e)
    float *Gs = lds + 2 * WT::TF;     // [2][BN][WT::LS]  dout
    float *Ss = lds + 4 * WT::TF;     // per query tile: [2][32] reference maxima, [2][32] 1 / row sums, [2][32] D
    int bh, unit;
    // (the shares of a split launch beyond what is resident at once: next to each other in the longest-first order, see
    // sdpa_prefill_f32_d128)
    int blk = blockIdx.x, sp = blockIdx.y;
    if ((lpt & 1) && shares_adjacent) dl4s_work_order::split_item_at(blockIdx.x, blockIdx.y, gridDim.x, nsplit, blk, sp);
    if (!dl4s_work_order::work_item_at(blk, nkb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, ln = lane & 31;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int kb = unit;
    const int kw0 = kb * BM + wave * 32;
    const int key = kw0 + ln;
    const int keyc = key < Lk ? key : Lk - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    const int nqt = (Lq + 31) / 32;
    int t_begin = 0, wt_begin = 0;
    bool wave_active = true;
    const unsigned char *skip_cls0 = nullptr;
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { t_begin = (kb * BM) / 32; wt_begin = kw0 / 32; }
        if (LENS) {
            if (kb * BM >= len) t_begin = nqt;
            if (kw0 >= len) wave_active = false;
        }
        if (DENSE && mask.cls) skip_cls0 = dense_query_bounds(mask, b, hh, kb * BM, wave, nqt, Lk, t_begin, wt_begin);
    }

    float kr[WT::HALF], vr[WT::HALF];   // the lane's key and value rows (columns (W/2)*half ..)
    {
        const float *kp = k + kv_base + (long long)keyc * rs + half * WT::HALF;
        const float *vp = v + kv_base + (long long)keyc * rs + half * WT::HALF;
#pragma unroll
        for (int j = 0; j < WT::NJ; ++j) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
            if (half * WT::HALF + 4 * j < hd) {
                a = *reinterpret_cast<const f32x4 *>(kp + 4 * j);
                c = *reinterpret_cast<const f32x4 *>(vp + 4 * j);
            }
            kr[4 * j + 0] = a.x; kr[4 * j + 1] = a.y; kr[4 * j + 2] = a.z; kr[4 * j + 3] = a.w;
            vr[4 * j + 0] = c.x; vr[4 * j + 1] = c.y; vr[4 * j + 2] = c.z; vr[4 * j + 3] = c.w;
        }
    }

    const int q_bytes = (int)(((long long)(Lq - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t qrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(q + q_base), 0, q_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t grsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(dout + q_base), 0, q_bytes, 0x00020000);
    unsigned ld_off[WT::NP];   // staging pieces as in sdpa_bwd_dq_f32_d128
    int lds_off[WT::NP];
#pragma unroll
    for (int i = 0; i < WT::NP; ++i) {
        const int pc = tid + 256 * i, row = pc / WT::PPR, col = (pc % WT::PPR) * 4;
        ld_off[i] = col < hd ? (unsigned)(row * rs + col) * 4u : 0x80000000u;
        lds_off[i] = row * WT::LS + col;
    }
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 qst[WT::NP], gst[WT::NP];
    float sst = 0.f;
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i) {
            const int o = (int)(ld_off[i] + t * tile_bytes);
            qst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o, 0, 0));
            gst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o, 0, 0));
        }
        if (tid < 96) {      // threads 0..31: reference maximum, 32..63: 1 / row sum, 64..95: D
            const int row = t * 32 + (tid & 31);
            const long long at = (long long)bh * Lq + row;
            sst = 0.f;
            if (row < Lq) sst = tid < 32 ? stats[2 * at] : (tid < 64 ? stats[2 * at + 1] : D[at]);
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i) {
            const int off = buf * WT::TF + lds_off[i];
            f32x4 s;
            s.x = (qst[i].x * rT) * LOG2E; s.y = (qst[i].y * rT) * LOG2E;
            s.z = (qst[i].z * rT) * LOG2E; s.w = (qst[i].w * rT) * LOG2E;
            *reinterpret_cast<f32x4 *>(Qs + off) = s;
            *reinterpret_cast<f32x4 *>(Gs + off) = gst[i];
        }
        if (tid < 96) Ss[(tid >> 5) * 64 + buf * 32 + (tid & 31)] = sst;
    };

    typename WT::Acc ka, va;   // dK^T and dV^T
    WT::zero(ka);
    WT::zero(va);

    int t = t_begin + (((sp - t_begin) % nsplit) + nsplit) % nsplit;   // the share's first tile at or after t_begin
    if (t < nqt) { load_tile(t); store_tile(0); }
    __syncthreads();

    const int row_lds = ln * WT::LS + half * WT::HALF;
    const unsigned char *cls_col = nullptr;
    if (DENSE && mask.cls) cls_col = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(kw0, Lk - 1) >> 5) * mask.cls_sk;
    const float *mcol = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + keyc * mask.sk : nullptr;
    const int Lqp = (Lq + 31) & ~31, Lkp = (Lk + 31) & ~31;
    __amdgpu_buffer_rsrc_t dsrsrc;
    unsigned ds_voff = 0;
    if (WRITE_DS) {
        dsrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(ds + (long long)bh * Lkp * Lqp), 0, (int)((long long)Lk * Lqp * 4), 0x00020000);
        ds_voff = ((unsigned)key * (unsigned)Lqp + 4u * half) * 4u;
    }

    // tiles the wavefront only stages first, then a loop whose every path stores dS (see sdpa_bwd_dkv_f32_d64)
    int buf = 0;
    const int wt_first = __builtin_amdgcn_readfirstlane(wave_active ? max(wt_begin, t_begin) : nqt);   // the same in every lane
    for (; t < wt_first && t < nqt; t += nsplit, buf ^= 1) {
        if (t + nsplit < nqt) { load_tile(t + nsplit); store_tile(buf ^ 1); }
        __syncthreads();
    }
    wait_vector_memory();   // the loads of the lane's key and value rows: nothing from before the loop is left in flight
    for (; t < nqt; t += nsplit, buf ^= 1) {
        const bool more = (t + nsplit < nqt);
        if (more) load_tile(t + nsplit);
        const int qt0 = t * 32;
        int cls = 2;
        if (DENSE && cls_col) cls = cls_col[(long long)t * mask.cls_sq] & 3;
        if (!(DENSE && cls == 1 && skip_cls0 && dense_block_open(skip_cls0 + (long long)t * mask.cls_sq, mask.cls_sk, t, (Lk + 31) >> 5))) {
            // S[query, key] in the base-2 domain: rows = the tile's queries 8(r/4) + 4*half + r%4, column = the lane's key
            f32x16 p = tile_product_w<WT::NJ>(Qs + buf * WT::TF + row_lds, kr);
            if (DENSE) {
                if (cls == 1) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) p[r] = blocked_score2(p[r]);
                } else if (cls == 2) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int qg = qt0 + 8 * (r >> 2) + 4 * half + (r & 3);
                        const int qc = qg < Lq ? qg : Lq - 1;
                        p[r] = dense_masked2(p[r], mcol[qc * mask.sq]);
                    }
                }
            } else if ((CAUSAL && (kw0 + 31 > qt0)) || (LENS && (kw0 + 32 > len))) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qg = qt0 + 8 * (r >> 2) + 4 * half + (r & 3);
                    bool blocked = false;
                    if (CAUSAL) blocked = blocked || (key > qg);
                    if (LENS) blocked = blocked || (key >= len);
                    if (blocked) p[r] = blocked_score2(p[r]);
                }
            }
            const float *st = Ss + buf * 32 + 4 * half;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 m4 = *reinterpret_cast<const f32x4 *>(st + 8 * g);
                const f32x4 r4 = *reinterpret_cast<const f32x4 *>(st + 64 + 8 * g);
                p[4 * g + 0] = fast_exp2(p[4 * g + 0] - m4.x) * r4.x;
                p[4 * g + 1] = fast_exp2(p[4 * g + 1] - m4.y) * r4.y;
                p[4 * g + 2] = fast_exp2(p[4 * g + 2] - m4.z) * r4.z;
                p[4 * g + 3] = fast_exp2(p[4 * g + 3] - m4.w) * r4.w;
            }
            WT::accumulate(Gs + buf * WT::TF, half, ln, lane, p, va);                // dV^T += dout^T . P
            const f32x16 dp = tile_product_w<WT::NJ>(Gs + buf * WT::TF + row_lds, vr);            // dP = dout . V^T
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 d4 = *reinterpret_cast<const f32x4 *>(st + 128 + 8 * g);
                p[4 * g + 0] = p[4 * g + 0] * (dp[4 * g + 0] - d4.x);
                p[4 * g + 1] = p[4 * g + 1] * (dp[4 * g + 1] - d4.y);
                p[4 * g + 2] = p[4 * g + 2] * (dp[4 * g + 2] - d4.z);
                p[4 * g + 3] = p[4 * g + 3] * (dp[4 * g + 3] - d4.w);
            }
            if (WRITE_DS) {
                // (rows of dS for keys that do not exist lie outside the descriptor: their stores are dropped, and the dQ
                // kernel, whose descriptor ends at the same row, reads them as zeros)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 o = {p[4 * g + 0], p[4 * g + 1], p[4 * g + 2], p[4 * g + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o), dsrsrc, (int)ds_voff, (qt0 + 8 * g) * 4, 0);
                }
            }
            WT::accumulate(Qs + buf * WT::TF, half, ln, lane, p, ka);                // dK^T += Q~^T . dS
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (part) {
        const long long rows = (long long)(total_blocks / nkb) * Lk;
        float *pp = part + (((long long)sp * 2) * rows + (long long)bh * Lk) * HD2;
        WT::store_rows(pp, HD2, kw0, Lk, ka, 1.0f, half, ln, lane, W);
        WT::store_rows(pp + rows * HD2, HD2, kw0, Lk, va, 1.0f, half, ln, lane, W);
        return;
    }
    WT::store_rows(dv + kv_base, rs, kw0, Lk, va, 1.0f, half, ln, lane, hd);
    WT::store_rows(dk + kv_base, rs, kw0, Lk, ka, 0.69314718055994530942f, half, ln, lane, hd);   // Q~ carries log2(e)
}

// out[row][0 .. hd-1] = scale * (share 0 + share 1 + ...) of unscaled partial sums part[share][rows][128] (shares
// share_stride floats apart); 32 lanes per row, four columns each
__global__ __launch_bounds__(256) void sdpa_bwd_merge_d128(const float *__restrict__ part, float *__restrict__ out, int nsplit,
                                                           long long share_stride, long long rows, int H, int L, int hd,
                                                           int token_major, float scale) {
    const long long row = (long long)blockIdx.x * 8 + (threadIdx.x >> 5);
    const int c = threadIdx.x & 31;
    if (row >= rows || 4 * c >= hd) return;
    f32x4 acc = *reinterpret_cast<const f32x4 *>(part + row * HD2 + 4 * c);
    for (int s = 1; s < nsplit; ++s) {
        const f32x4 x = *reinterpret_cast<const f32x4 *>(part + (long long)s * share_stride + row * HD2 + 4 * c);
        acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
    }
    acc.x *= scale; acc.y *= scale; acc.z *= scale; acc.w *= scale;
    const long long bh = row / L, i = row % L, b = bh / H, hh = bh % H;
    const long long at = token_major ? (((b * L + i) * H + hh) * hd) : (row * hd);
    *reinterpret_cast<f32x4 *>(out + at + 4 * c) = acc;
}

// ------------------------------------------------------------------------------------------------ dQ from stored dS
// dQ = (dS . K) * rT with dS read from the scratch tensor sdpa_bwd_dkv_f32_d128<KIND, true> wrote; see
// sdpa_bwd_dq_from_ds_f32_d64.  Four accumulators and one dS tile in flight: three wavefronts per SIMD instead of one.
template <int KIND, int W = 128>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dq_from_ds_f32_d128(const float *__restrict__ k, const float *__restrict__ ds,
                                                                        float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                                        MaskArgs mask, int strict, int nqb, int total_blocks, int lpt,
                                                                        int token_major, int hd, int nsplit = 1,
                                                                        float *__restrict__ part = nullptr, int shares_adjacent = 0) {
    // nsplit > 1: workgroup blockIdx.y takes the key tiles y, y + nsplit, ... and leaves its unscaled sums in
    // part [share][batch*head*Lq][128] for sdpa_bwd_merge_d128
    using WT = WideTile<W>;
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                      // [2][BN][WT::LS]
    int bh, unit;
    int blk = blockIdx.x, sp = blockIdx.y;
    if ((lpt & 1) && shares_adjacent) dl4s_work_order::split_item_at(blockIdx.x, blockIdx.y, gridDim.x, nsplit, blk, sp);
    if (!dl4s_work_order::work_item_at(blk, nqb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, ln = lane & 31;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int qb = nqb - 1 - unit;   // longest rows first
    const int q0 = qb * BM + wave * 32;
    const int qi = q0 + ln;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    int kend = Lk, wkend = Lk;
    bool skip_ones = false;
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { kend = min(kend, qb * BM + BM); wkend = min(wkend, q0 + 32); }
        if (LENS) { kend = min(kend, len); wkend = min(wkend, len); }
        if (DENSE && mask.cls) dense_key_bounds(mask, b, hh, qb * BM, wave, Lq, Lk, kend, wkend, skip_ones);
    }
    const int ntiles = (kend + BN - 1) / BN;

    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    unsigned ld_off[WT::NP];   // staging pieces as in sdpa_bwd_dq_f32_d128
    int lds_off[WT::NP];
#pragma unroll
    for (int i = 0; i < WT::NP; ++i) {
        const int pc = tid + 256 * i, row = pc / WT::PPR, col = (pc % WT::PPR) * 4;
        ld_off[i] = col < hd ? (unsigned)(row * rs + col) * 4u : 0x80000000u;
        lds_off[i] = row * WT::LS + col;
    }
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[WT::NP];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i)
            kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, (int)(ld_off[i] + t * tile_bytes), 0, 0));
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < WT::NP; ++i) *reinterpret_cast<f32x4 *>(Ks + buf * WT::TF + lds_off[i]) = kst[i];
    };

    const int Lqp = (Lq + 31) & ~31, Lkp = (Lk + 31) & ~31;
    const __amdgpu_buffer_rsrc_t dsrsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)(ds + (long long)bh * Lkp * Lqp), 0, (int)((long long)Lk * Lqp * 4), 0x00020000);
    const unsigned ds_voff = ((unsigned)(4 * half) * (unsigned)Lqp + (unsigned)qi) * 4u;
    const unsigned ds_row = (unsigned)Lqp * 4u;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;
    auto visited = [&](int t) {
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        return t * BN < wkend && !(DENSE && skip_ones && cls == 1);
    };
    f32x16 dsn;
    auto load_ds = [&](int t) {
        const unsigned base = (unsigned)(t * BN) * ds_row;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            dsn[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(dsrsrc, (int)ds_voff, (int)(base + (unsigned)(8 * (r >> 2) + (r & 3)) * ds_row), 2));
    };

    typename WT::Acc acc;   // dQ^T
    WT::zero(acc);
#pragma unroll
    for (int i = 0; i < 16; ++i) dsn[i] = 0.f;

    if (sp < ntiles) {
        load_tile(sp);
        store_tile(0);
        if (visited(sp)) load_ds(sp);
    }
    __syncthreads();
    for (int t = sp, buf = 0; t < ntiles; t += nsplit, buf ^= 1) {
        const bool more = (t + nsplit < ntiles);
        const bool now = visited(t);
        f32x16 p = dsn;
        // The slab's rows of the keys Lk ... (padded to 32) are never written, and the row term of the load sits in the
        // scalar offset, which the descriptor's range check does not cover: clear them (their K rows are zeros, but
        // 0 x a stale NaN would not be).
        if (t * BN + BN > Lk) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (t * BN + 8 * (r >> 2) + 4 * half + (r & 3) >= Lk) p[r] = 0.f;
        }
        if (more) {
            load_tile(t + nsplit);
            if (visited(t + nsplit)) load_ds(t + nsplit);
        }
        if (now) WT::accumulate(Ks + buf * WT::TF, half, ln, lane, p, acc);         // dQ^T += K^T . dS^T
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (part) {
        WT::store_rows(part + (((long long)sp * (total_blocks / nqb) + bh) * Lq) * HD2, HD2, q0, Lq, acc, 1.0f, half, ln, lane, W);
        return;
    }
    WT::store_rows(dq + q_base, rs, q0, Lq, acc, rT, half, ln, lane, hd);
}

template <int KIND, int W = 128>
int launch_bwd128(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *dout, const float *stats,
                  const float *D, float *dq, float *dk, float *dv, int B, int H, int Lq, int Lk, float rT, const MaskArgs &m,
                  int strict, int token_major, int hd, long long ds_max_bytes, int no_split = 0) {
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    using WT = WideTile<W>;
    const size_t lds_dq = 4 * WT::TF * sizeof(float);
    const size_t lds_dkv = (4 * WT::TF + 192) * sizeof(float);
    // (the 96-wide tiles stay within the default 64 KiB of dynamic LDS)
    if (lds_dkv > 65536 && dl4s::lds_limit_pending(ctx, dl4s::LDS_BWD_D128, KIND)) {
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dq_f32_d128<KIND, W>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dkv_f32_d128<KIND, false, W>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dkv_f32_d128<KIND, true, W>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv));
        dl4s::lds_limit_done(ctx, dl4s::LDS_BWD_D128, KIND);
    }
    const bool uneven = (causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict;
    // The dK/dV kernel stores dS and a light dQ kernel contracts it with K (see sdpa_backward.hip) whenever the scratch
    // tensor can be had; the two self-contained kernels otherwise.
    {
        const long long Lqp = (Lq + 31) & ~31ll, Lkp = (Lk + 31) & ~31ll;
        const long long slab = Lqp * Lkp * 4;
        const int nqb = (Lq + BM - 1) / BM, nkb = (Lk + BM - 1) / BM;
        const long long total_q = (long long)nqb * B * H, total_k = (long long)nkb * B * H;
        void *dsv = nullptr;
        if (slab < (1ll << 31) && (long long)B * H * slab <= ds_max_bytes && total_q < (1ll << 30) && total_k < (1ll << 30) &&
            dl4s_hip_alloc(ctx, (size_t)((long long)B * H * slab), &dsv) == DL4S_HIP_OK) {
            float *ds = static_cast<float *>(dsv);
            // Launches that leave CUs without a workgroup (dK/dV: one per CU; dQ: two) are split over the walked tiles
            // across workgroups; the counts depend on the extents only.  B4 H8 L512 causal: 186 us unsplit.
            const long long nqt = (Lq + 31) / 32, nkt = (Lk + 31) / 32;
            long long sk = 1, sq = 1;
            // (blocks of different length: two shares also where every CU just has its workgroup, B2 H8 L2048 causal 679 -> 497 us)
            if (!no_split && total_k < (uneven ? 2ll : 1ll) * ctx->cu_count && nqt >= 4)
                sk = std::min(std::min(8ll, nqt / 2), std::max(2ll, (ctx->cu_count + total_k - 1) / total_k));
            if (!no_split && total_q < (uneven ? 4ll : 2ll) * ctx->cu_count && nkt >= 4)
                sq = std::min(std::min(8ll, nkt / 2), std::max(2ll, (2ll * ctx->cu_count + total_q - 1) / total_q));
            const long long krows = (long long)B * H * Lk, qrows = (long long)B * H * Lq;
            const long long part_k = sk > 1 ? sk * 2 * krows * HD2 : 0, part_q = sq > 1 ? sq * qrows * HD2 : 0;
            void *pv = nullptr;
            if (part_k + part_q > 0 && dl4s_hip_alloc(ctx, (size_t)(part_k + part_q) * sizeof(float), &pv) != DL4S_HIP_OK) { sk = sq = 1; pv = nullptr; }
            float *pk = sk > 1 ? static_cast<float *>(pv) : nullptr;
            float *pq = sq > 1 ? static_cast<float *>(pv) + (sk > 1 ? part_k : 0) : nullptr;
            int lpt = (uneven && nkb >= 2) ? 1 : 0;
            if (lpt && total_k <= (long long)ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
            hipLaunchKernelGGL((sdpa_bwd_dkv_f32_d128<KIND, true, W>), dim3((unsigned)((total_k + 7) / 8 * 8), (unsigned)sk), dim3(256), lds_dkv,
                               ctx->stream, q, k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb, (int)total_k, lpt, token_major, hd,
                               ds, (int)sk, pk, ((total_k + 7) / 8 * 8 * sk > (long long)ctx->cu_count) ? 1 : 0);   // (B1 H12 L2048 causal 444 -> 414 us, B1 H8 L4096 913 -> 881 us)
            int rc = dl4s::launch_status("sdpa_bwd_dkv_f32_d128");
            if (rc == DL4S_HIP_OK && pk) {
                const dim3 mg((unsigned)((krows + 7) / 8));
                hipLaunchKernelGGL(sdpa_bwd_merge_d128, mg, dim3(256), 0, ctx->stream, pk, dk, (int)sk, 2 * krows * HD2, krows, H, Lk, hd,
                                   token_major, 0.69314718055994530942f);   // Q~ carries log2(e)
                hipLaunchKernelGGL(sdpa_bwd_merge_d128, mg, dim3(256), 0, ctx->stream, pk + krows * HD2, dv, (int)sk, 2 * krows * HD2, krows, H,
                                   Lk, hd, token_major, 1.0f);
                rc = dl4s::launch_status("sdpa_bwd_merge_d128");
            }
            if (rc == DL4S_HIP_OK) {
                lpt = (uneven && nqb >= 2) ? 1 : 0;
                if (lpt && total_q <= 2ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
                hipLaunchKernelGGL((sdpa_bwd_dq_from_ds_f32_d128<KIND, W>), dim3((unsigned)((total_q + 7) / 8 * 8), (unsigned)sq), dim3(256),
                                   2 * WT::TF * sizeof(float), ctx->stream, k, ds, dq, H, Lq, Lk, rT, m, strict, nqb, (int)total_q,
                                   lpt, token_major, hd, (int)sq, pq, ((total_q + 7) / 8 * 8 * sq > 2ll * ctx->cu_count) ? 1 : 0);
                rc = dl4s::launch_status("sdpa_bwd_dq_from_ds_f32_d128");
                if (rc == DL4S_HIP_OK && pq) {
                    hipLaunchKernelGGL(sdpa_bwd_merge_d128, dim3((unsigned)((qrows + 7) / 8)), dim3(256), 0, ctx->stream, pq, dq, (int)sq,
                                       qrows * HD2, qrows, H, Lq, hd, token_major, rT);
                    rc = dl4s::launch_status("sdpa_bwd_merge_d128");
                }
            }
            int rcf = dl4s_hip_free(ctx, dsv);   // stream-ordered
            if (pv) { const int rcp = dl4s_hip_free(ctx, pv); if (rcf == DL4S_HIP_OK) rcf = rcp; }
            return rc != DL4S_HIP_OK ? rc : rcf;
        }
    }
    {
        const int nqb = (Lq + BM - 1) / BM;
        const long long total = (long long)nqb * B * H;
        DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa backward: %lld workgroups exceed the grid limit", total);
        int lpt = (uneven && nqb >= 2) ? 1 : 0;
        if (lpt && total <= (long long)ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL((sdpa_bwd_dq_f32_d128<KIND, W>), dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dq, ctx->stream, q, k,
                           v, dout, stats, D, dq, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt, token_major, hd);
        const int rc = dl4s::launch_status("sdpa_bwd_dq_f32_d128");
        if (rc != DL4S_HIP_OK) return rc;
    }
    {
        const int nkb = (Lk + BM - 1) / BM;
        const long long total = (long long)nkb * B * H;
        DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa backward: %lld workgroups exceed the grid limit", total);
        int lpt = (uneven && nkb >= 2) ? 1 : 0;
        if (lpt && total <= (long long)ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL((sdpa_bwd_dkv_f32_d128<KIND, false, W>), dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dkv, ctx->stream, q,
                           k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb, (int)total, lpt, token_major, hd);
        return dl4s::launch_status("sdpa_bwd_dkv_f32_d128");
    }
}

}  // namespace

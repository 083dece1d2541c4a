// Gradients of the fused attention for narrow heads (head dims up to 32): the stored-dS route of sdpa_backward.hip on tiles
// of W = 32 or W = 16 columns, with the operand layouts of sdpa_prefill_narrow.h.  Included by sdpa_backward.hip only.
//
//   sdpa_bwd_dkv_f32_narrow     a wavefront owns 32 keys and walks the query tiles: S and dP take W/2 MFMAs each (the two
//                               halves of the wavefront contract d = s and d = W/2 + s), dV^T and dK^T one 32 x 32
//                               accumulator each (row = d, column = key; 16 MFMAs); every dS tile is stored to the scratch
//                               tensor [batch*head][key][query]
//   sdpa_bwd_dq_from_ds_f32_narrow   dQ^T += K^T . dS^T from the stored tiles, one accumulator, 16 MFMAs per tile
// W + 48 MFMAs per 32 x 32 tile of (query, key) pairs instead of 160.  Launches that cannot take the stored-dS route (small
// ones, no scratch) run the 64-wide kernels on zero-padded tiles as before.  The scores are formed in the same order over
// d as in the narrow forward kernels, whose row statistics they are matched against.
#pragma once
#include "sdpa_common.h"

namespace {

template <int NJ>
__device__ __forceinline__ f32x16 tile_product_n(const float *Ab, const float (&br)[4 * NJ]) {
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

// acc (row d = the lane's ln, column = the lane's query or key) += A^T . B: A is a [32][LS] LDS tile read a float at a
// time (row 8(r/4) + r%4 + 4*half, column ln: At already points there), B the accumulator-layout tile b
template <int LS>
__device__ __forceinline__ void tile_accumulate_1(const float *At, const f32x16 &b, f32x16 &acc) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(At[(8 * (r >> 2) + (r & 3)) * LS], b[r], acc, 0, 0, 0);
}

// The 16-wide form of tile_accumulate_1 on 16 x 16 x 4 MFMAs (a 32 x 32 accumulator of a 16-wide head is half empty):
// og[0] holds the columns (keys) 0 .. 15 of the wavefront, og[1] 16 .. 31; lane: column = lane % 16, rows d = 4 * (lane / 16) + i.
// v_permlane16_swap of a register pair (2p, 2p+1) of b puts, for both accumulators at once, the value of row
// 8(p/2) + 2(p%2) + (s&1) + 4(s>>1) into lane 16 s + lane % 16 (see attend_tile_16 in sdpa_prefill_narrow.h).
// At16: the lane's base in the [32][LS] tile, row (s&1) + 4(s>>1), column lane % 16 (s = lane / 16).
template <int LS>
__device__ __forceinline__ void tile_accumulate_16(const float *At16, const f32x16 &b, f32x4 (&og)[2]) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(b[2 * p]), __float_as_uint(b[2 * p + 1]), false, false);
        const float a = At16[(8 * (p >> 1) + 2 * (p & 1)) * LS];
        og[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, __uint_as_float(sw[0]), og[0], 0, 0, 0);
        og[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, __uint_as_float(sw[1]), og[1], 0, 0, 0);
    }
}

// stores the lane's row: register r of acc is d = 8(r/4) + 4*half + r%4
__device__ __forceinline__ void store_row_1(float *p, const f32x16 &acc, const float scale, const int half, const int hd) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int d0 = 8 * g + 4 * half;
        const f32x4 a = {acc[4 * g + 0] * scale, acc[4 * g + 1] * scale, acc[4 * g + 2] * scale, acc[4 * g + 3] * scale};
        if (d0 < hd) *reinterpret_cast<f32x4 *>(p + d0) = a;
    }
}

template <int KIND, int W>
__global__ __launch_bounds__(256, 3) void sdpa_bwd_dkv_f32_narrow(const float *__restrict__ q, const float *__restrict__ k,
                                                                   const float *__restrict__ v, const float *__restrict__ dout,
                                                                   const float *__restrict__ stats, const float *__restrict__ D,
                                                                   float *__restrict__ dk, float *__restrict__ dv, int H, int Lq,
                                                                   int Lk, float rT, MaskArgs mask, int strict, int nkb,
                                                                   int total_blocks, int lpt, int token_major, int hd,
                                                                   float *__restrict__ ds) {
    constexpr int LS = W + 4, TF = BN * LS, NJ = W / 8;
    extern __shared__ __align__(16) float lds[];
    float *Qs = lds;               // [2][BN][LS]  q * rT * log2(e)
    float *Gs = lds + 2 * TF;      // [2][BN][LS]  dout
    float *Ss = lds + 4 * TF;      // per query tile: [2][32] reference maxima, [2][32] 1 / row sums, [2][32] D
    int bh, unit;
    if (!work_item(nkb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, ln = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int kb = unit;                 // under a causal mask the first key block meets the most queries: longest first
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

    float kr[W / 2], vr[W / 2];   // the lane's key and value rows (columns half * W/2 ..)
    {
        const float *kp = k + kv_base + (long long)keyc * rs + half * (W / 2);
        const float *vp = v + kv_base + (long long)keyc * rs + half * (W / 2);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
            if (half * (W / 2) + 4 * j < hd) {
                a = *reinterpret_cast<const f32x4 *>(kp + 4 * j);
                c = *reinterpret_cast<const f32x4 *>(vp + 4 * j);
            }
            kr[4 * j + 0] = a.x; kr[4 * j + 1] = a.y; kr[4 * j + 2] = a.z; kr[4 * j + 3] = a.w;
            vr[4 * j + 0] = c.x; vr[4 * j + 1] = c.y; vr[4 * j + 2] = c.z; vr[4 * j + 3] = c.w;
        }
    }

    // staging of one query tile (the scheme of sdpa_prefill_f32_narrow): W = 32 every thread one piece of q and one of
    // dout; W = 16 wavefronts 0, 1 the q tile and wavefronts 2, 3 the dout tile
    constexpr int CPR = W / 4;
    const int stt = (W == 32) ? tid : (tid & 127);
    const int ld_row = stt / CPR, ld_col = (stt % CPR) * 4;
    const int q_bytes = (int)(((long long)(Lq - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t qrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(q + q_base), 0, q_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t grsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(dout + q_base), 0, q_bytes, 0x00020000);
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    const int lds_off = ld_row * LS + ld_col;
    f32x4 qst, gst;
    float sst = 0.f;
    auto load_tile = [&](int t) {
        const int o = (int)(ld_off + t * tile_bytes);
        if (W == 32) {
            qst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o, 0, 0));
            gst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o, 0, 0));
        } else if (wave < 2) {
            qst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o, 0, 0));
        } else {
            gst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o, 0, 0));
        }
        if (tid < 96) {      // threads 0..31: reference maximum, 32..63: 1 / row sum, 64..95: D
            const int row = t * 32 + (tid & 31);
            const long long at = (long long)bh * Lq + row;
            sst = 0.f;
            if (row < Lq) sst = tid < 32 ? stats[2 * at] : (tid < 64 ? stats[2 * at + 1] : D[at]);
        }
    };
    auto store_tile = [&](int buf) {
        if (W == 32 || wave < 2) {
            f32x4 s;
            s.x = (qst.x * rT) * LOG2E; s.y = (qst.y * rT) * LOG2E; s.z = (qst.z * rT) * LOG2E; s.w = (qst.w * rT) * LOG2E;
            *reinterpret_cast<f32x4 *>(Qs + buf * TF + lds_off) = s;
        }
        if (W == 32 || wave >= 2) *reinterpret_cast<f32x4 *>(Gs + buf * TF + lds_off) = gst;
        if (tid < 96) Ss[(tid >> 5) * 64 + buf * 32 + (tid & 31)] = sst;
    };

    f32x16 ka, va;   // dK^T and dV^T, row d = 8(r/4) + 4*half + r%4
#pragma unroll
    for (int i = 0; i < 16; ++i) { ka[i] = 0.f; va[i] = 0.f; }
    f32x4 kg[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, vg[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};   // W = 16 (tile_accumulate_16)

    if (t_begin < nqt) { load_tile(t_begin); store_tile(0); }
    __syncthreads();

    const int row_lds = ln * LS + half * (W / 2);
    const int col_lds = (4 * half) * LS + ln;
    const int slot = lane >> 4;
    const int col_lds16 = ((slot & 1) + 4 * (slot >> 1)) * LS + (lane & 15);
    const unsigned char *cls_col = nullptr;
    if (DENSE && mask.cls) cls_col = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(kw0, Lk - 1) >> 5) * mask.cls_sk;
    const float *mcol = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + keyc * mask.sk : nullptr;
    const int Lqp = (Lq + 31) & ~31, Lkp = (Lk + 31) & ~31;
    const __amdgpu_buffer_rsrc_t dsrsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)(ds + (long long)bh * Lkp * Lqp), 0, (int)((long long)Lk * Lqp * 4), 0x00020000);
    const unsigned ds_voff = ((unsigned)key * (unsigned)Lqp + 4u * half) * 4u;

    // tiles the wavefront only stages first, then a loop whose every path stores dS (see sdpa_bwd_dkv_f32_d64)
    int t = t_begin;
    const int wt_first = __builtin_amdgcn_readfirstlane(wave_active ? max(wt_begin, t_begin) : nqt);   // the same in every lane
    for (; t < wt_first && t < nqt; ++t) {
        const int buf = (t - t_begin) & 1;
        if (t + 1 < nqt) { load_tile(t + 1); store_tile(buf ^ 1); }
        __syncthreads();
    }
    wait_vector_memory();   // the loads of the lane's key and value rows: nothing from before the loop is left in flight
    for (; t < nqt; ++t) {
        const int buf = (t - t_begin) & 1;
        const bool more = (t + 1 < nqt);
        if (more) load_tile(t + 1);
        const int qt0 = t * 32;
        int cls = 2;
        if (DENSE && cls_col) cls = cls_col[(long long)t * mask.cls_sq] & 3;
        if (!(DENSE && cls == 1 && skip_cls0 && dense_block_open(skip_cls0 + (long long)t * mask.cls_sq, mask.cls_sk, t, (Lk + 31) >> 5))) {
            f32x16 p = tile_product_n<NJ>(Qs + buf * TF + row_lds, kr);     // S, rows = the tile's queries, column = the lane's key
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
            if constexpr (W == 16) tile_accumulate_16<LS>(Gs + buf * TF + col_lds16, p, vg);
            else tile_accumulate_1<LS>(Gs + buf * TF + col_lds, p, va);                      // dV^T += dout^T . P
            const f32x16 dp = tile_product_n<NJ>(Gs + buf * TF + row_lds, vr);               // dP = dout . V^T
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 d4 = *reinterpret_cast<const f32x4 *>(st + 128 + 8 * g);
                p[4 * g + 0] = p[4 * g + 0] * (dp[4 * g + 0] - d4.x);
                p[4 * g + 1] = p[4 * g + 1] * (dp[4 * g + 1] - d4.y);
                p[4 * g + 2] = p[4 * g + 2] * (dp[4 * g + 2] - d4.z);
                p[4 * g + 3] = p[4 * g + 3] * (dp[4 * g + 3] - d4.w);
            }
            // (rows of dS for keys that do not exist lie outside the descriptor: their stores are dropped, and the dQ
            // kernel, whose descriptor ends at the same row, reads them as zeros)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 o = {p[4 * g + 0], p[4 * g + 1], p[4 * g + 2], p[4 * g + 3]};
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o), dsrsrc, (int)ds_voff, (qt0 + 8 * g) * 4, 0);
            }
            if constexpr (W == 16) tile_accumulate_16<LS>(Qs + buf * TF + col_lds16, p, kg);
            else tile_accumulate_1<LS>(Qs + buf * TF + col_lds, p, ka);                      // dK^T += Q~^T . dS
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if constexpr (W == 16) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {      // accumulator g: key kw0 + 16 g + lane % 16, columns 4 * slot ..
            const int kg_ = kw0 + 16 * g + (lane & 15);
            if (kg_ < Lk && 4 * slot < hd) {
                constexpr float LN2 = 0.69314718055994530942f;    // Q~ carries log2(e)
                const f32x4 a = {kg[g].x * LN2, kg[g].y * LN2, kg[g].z * LN2, kg[g].w * LN2};
                *reinterpret_cast<f32x4 *>(dv + kv_base + (long long)kg_ * rs + 4 * slot) = vg[g];
                *reinterpret_cast<f32x4 *>(dk + kv_base + (long long)kg_ * rs + 4 * slot) = a;
            }
        }
    } else if (key < Lk) {
        store_row_1(dv + kv_base + (long long)key * rs, va, 1.0f, half, hd);
        store_row_1(dk + kv_base + (long long)key * rs, ka, 0.69314718055994530942f, half, hd);   // Q~ carries log2(e)
    }
}

template <int KIND, int W>
__global__ __launch_bounds__(256, 4) void sdpa_bwd_dq_from_ds_f32_narrow(const float *__restrict__ k, const float *__restrict__ ds,
                                                                          float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                                          MaskArgs mask, int strict, int nqb, int total_blocks, int lpt,
                                                                          int token_major, int hd) {
    constexpr int LS = W + 4, TF = BN * LS;
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                     // [2][BN][LS]
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

    // the K tile: 8 W pieces of 128 bits, one per thread (W = 32) or per thread of the first two wavefronts (W = 16)
    constexpr int CPR = W / 4;
    const bool stager = (W == 32) || tid < 128;
    const int ld_row = tid / CPR, ld_col = (tid % CPR) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off = (stager && ld_col < hd) ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst;
    auto load_tile = [&](int t) { kst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, (int)(ld_off + t * tile_bytes), 0, 0)); };
    auto store_tile = [&](int buf) {
        if (stager) *reinterpret_cast<f32x4 *>(Ks + buf * TF + ld_row * LS + ld_col) = kst;
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

    f32x16 acc;   // dQ^T, row d = 8(r/4) + 4*half + r%4
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc[i] = 0.f; dsn[i] = 0.f; }

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
        if (visited(0)) load_ds(0);
    }
    __syncthreads();
    const int col_lds = (4 * half) * LS + ln;
    for (int t = 0; t < ntiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1 < ntiles);
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
            load_tile(t + 1);
            if (visited(t + 1)) load_ds(t + 1);
        }
        if (now) tile_accumulate_1<LS>(Ks + buf * TF + col_lds, p, acc);
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (qi < Lq) store_row_1(dq + q_base + (long long)qi * rs, acc, rT, half, hd);
}

// The stored-dS route for narrow heads.  Returns 1 when it ran, 0 when the caller should take the 64-wide kernels (small
// launches, no scratch tensor to be had), a negative status on failure.
template <int KIND, int W>
int launch_bwd_narrow(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *dout, const float *stats,
                      const float *D, float *dq, float *dk, float *dv, int B, int H, int Lq, int Lk, float rT, const MaskArgs &m,
                      int strict, int token_major, int hd, int no_split, long long ds_max_bytes) {
    constexpr int TF = BN * (W + 4);
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    const bool uneven = (causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict;
    const bool dq_small = !no_split && sdpa_bwd_small_launch(ctx, B, H, Lq, uneven, true) && Lk >= 2 * BN;
    const bool dkv_small = !no_split && sdpa_bwd_small_launch(ctx, B, H, Lk, uneven, true) && Lq >= 2 * BN;
    if (dq_small || dkv_small) return 0;
    const long long Lqp = (Lq + 31) & ~31ll, Lkp = (Lk + 31) & ~31ll;
    const long long slab = Lqp * Lkp * 4;
    const int nqb = (Lq + BM - 1) / BM, nkb = (Lk + BM - 1) / BM;
    const long long total_q = (long long)nqb * B * H, total_k = (long long)nkb * B * H;
    void *dsv = nullptr;
    if (!(slab < (1ll << 31) && (long long)B * H * slab <= ds_max_bytes && total_q < (1ll << 30) && total_k < (1ll << 30))) return 0;
    if (dl4s_hip_alloc(ctx, (size_t)((long long)B * H * slab), &dsv) != DL4S_HIP_OK) return 0;
    float *ds = static_cast<float *>(dsv);
    int lpt = (uneven && nkb >= 2) ? 1 : 0;
    if (lpt && total_k <= 5ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
    // 32 floats of LDS beyond the tiles: at W = 16 the lanes that stand for rows d >= 16 read past the last tile
    hipLaunchKernelGGL((sdpa_bwd_dkv_f32_narrow<KIND, W>), dim3((unsigned)((total_k + 7) / 8 * 8)), dim3(256),
                       (size_t)(4 * TF + 192 + 32) * sizeof(float), ctx->stream, q, k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb,
                       (int)total_k, lpt, token_major, hd, ds);
    int rc = dl4s::launch_status("sdpa_bwd_dkv_f32_narrow");
    if (rc == DL4S_HIP_OK) {
        lpt = (uneven && nqb >= 2) ? 1 : 0;
        if (lpt && total_q <= 7ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL((sdpa_bwd_dq_from_ds_f32_narrow<KIND, W>), dim3((unsigned)((total_q + 7) / 8 * 8)), dim3(256),
                           (size_t)(2 * TF + 32) * sizeof(float), ctx->stream, k, ds, dq, H, Lq, Lk, rT, m, strict, nqb, (int)total_q, lpt,
                           token_major, hd);
        rc = dl4s::launch_status("sdpa_bwd_dq_from_ds_f32_narrow");
    }
    const int rcf = dl4s_hip_free(ctx, dsv);   // stream-ordered
    if (rc != DL4S_HIP_OK) return rc;
    return rcf != DL4S_HIP_OK ? rcf : 1;
}

}  // namespace

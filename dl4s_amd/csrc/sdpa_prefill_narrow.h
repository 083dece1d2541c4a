// Fused attention forward for narrow heads (head dims up to 32): the kernels of sdpa_prefill.hip on tiles that are W = 32
// or W = 16 columns wide instead of 64, and a W = 48 form of the main kernel for head dims 36 .. 48 (attend_tile_48).
// Included by sdpa_prefill.hip only.
//
// A 64-wide tile spends 32 MFMA steps on S^T = K . Q^T and 32 on O^T += V^T . P^T whatever the head dim; a model with key
// size 8 (the reference's own test model, Tests/DL4STests/TransformerTests.swift:31) needs a fraction of that:
//   S^T   the two halves of the wavefront contract d = s and d = W/2 + s in step s: W/2 MFMAs (16 or 8 instead of 32)
//   O^T   one 32 x 32 accumulator (row = d, column = query) instead of two: 16 MFMAs instead of 32; V is read a float at a
//         time (row = key, column = the lane's d); rows at or beyond the head dim are computed on whatever follows in LDS
//         and never stored.  The main 16-wide kernel uses two 16 x 16 accumulators instead (attend_tile_16).
// Everything else - the transposed products that keep the weights in the registers they were computed in, the mask in
// registers, the online softmax with a lazy reference maximum, tile skipping, the work order, the token-major layout, the
// row statistics for the gradient kernels - is the 64-wide kernels'.  The summation order over d differs from theirs, so
// the two agree within rounding, not bit for bit.
#pragma once
#include <type_traits>

#include "sdpa_common.h"

namespace {

template <int W> struct NarrowTile {
    static constexpr int LS = W + 4;          // LDS row stride (36, 20, 52): keeps 128-bit reads of consecutive rows on distinct banks
    static constexpr int TF = BN * LS;        // floats per tile
    // Row stride of the V tile in the main kernel.  Its 16 x 16 x 4 MFMA operand reads (W = 16, and the columns 32 .. 47 of
    // W = 48) put the lanes 16 s .. 16 s + 15 on 16 consecutive floats of row r + (s & 1) + 4 (s >> 1): with rows of exactly
    // W floats (16, 48: an odd multiple of 16) the two rows that a half of the wavefront reads land on the two halves of the
    // 32 banks; on the K tile's stride they overlapped in four (W + 4 = 20, 52) and the read took twice as long.
    static constexpr int LSV = (W == 32) ? LS : W;
    static constexpr int TFV = BN * LSV;
    static constexpr int NJ = W / 8;          // 128-bit reads per K row fragment
};

// One 32-key tile for one wavefront (32 queries).  Kb: the lane's K fragment base (row ln, columns half * W/2 ..);
// Vb: row 4 * half, column ln.
template <int KIND, int W>
__device__ __forceinline__ void attend_tile_narrow(const float *Kb, const float *Vb, const float (&qr)[W / 2], f32x16 &o0,
                                                   float &m_run, float &m_use, float &l_run, const int k0, const int q0,
                                                   const int qi, const int half, const int Lk, const int len, const float *mrow,
                                                   const long long msk, const int cls) {
    constexpr int LS = NarrowTile<W>::LS;
    f32x16 s0 = masked_scores<KIND, NarrowTile<W>::NJ>(Kb, qr, k0, q0, qi, half, Lk, len, mrow, msk, cls);

    // online softmax with a lazy reference maximum (see attend_tile in sdpa_prefill.hip)
    const float tmax = max_across_halves(max_of_16(s0));
    const bool upd = tmax - m_run > 8.0f;      // also right at m_run = -inf: +inf, or NaN for tmax = -inf
    if (__any(upd)) {
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = (m_run == m_new) ? 1.0f : fast_exp2(m_run - m_new);
        m_run = m_new;
        m_use = (m_new == -INFINITY) ? 0.f : m_new;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) o0[i] *= alpha;
    }
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = fast_exp2(s0[r] - m_use);
        psum += s0[r];
    }
    l_run += psum;

    // O^T += V^T . P^T: A operand = V[key 8(r/4) + 4*half + r%4][d = ln]
#pragma unroll
    for (int r = 0; r < 16; ++r) o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(Vb[(8 * (r >> 2) + (r & 3)) * LS], s0[r], o0, 0, 0, 0);
}

// The 16-wide tile in the main kernel: O^T on 16 x 16 x 4 MFMAs, so that no accumulator row is idle (a 32 x 32 accumulator
// of a 16-wide head is half empty: 16 MFMAs of 64 cycles against 16 of 32 cycles here).  og[0] holds the queries q0 .. q0+15,
// og[1] q0+16 .. q0+31; lane: column = lane % 16, rows d = 4 * (lane / 16) + i.  The weights leave the score product with
// lane = query (lane % 32) and 16 keys in registers; v_permlane16_swap of a register pair (2p, 2p+1) puts, for both groups
// at once, the weight of key 8(p/2) + 2(p%2) + (s&1) + 4(s>>1) of query lane % 16 (+16) into lane 16 s + lane % 16 - the B
// operand of one MFMA step per group, with V read at that key's row as the A operand of both.
// Vt: the lane's V base, row (s&1) + 4(s>>1), column lane % 16 (s = lane / 16).
template <int KIND>
__device__ __forceinline__ void attend_tile_16(const float *Kb, const float *Vt, const float (&qr)[8], f32x4 (&og)[2], float &m_run,
                                               float &m_use, float &l_run, const int k0, const int q0, const int qi, const int half,
                                               const int ln, const int Lk, const int len, const float *mrow, const long long msk,
                                               const int cls) {
    constexpr int LSV = NarrowTile<16>::LSV;
    f32x16 s0 = masked_scores<KIND, 2>(Kb, qr, k0, q0, qi, half, Lk, len, mrow, msk, cls);
    const float tmax = max_across_halves(max_of_16(s0));
    const bool upd = tmax - m_run > 8.0f;      // also right at m_run = -inf: +inf, or NaN for tmax = -inf
    if (__any(upd)) {
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = (m_run == m_new) ? 1.0f : fast_exp2(m_run - m_new);
        m_run = m_new;
        m_use = (m_new == -INFINITY) ? 0.f : m_new;
        l_run *= alpha;
        // the lane's own factor belongs to the group its query is in; the other group's comes from the lane 16 away
        const float other = __shfl_xor(alpha, 16, 64);
        const float a0 = ln < 16 ? alpha : other, a1 = ln < 16 ? other : alpha;
        og[0].x *= a0; og[0].y *= a0; og[0].z *= a0; og[0].w *= a0;
        og[1].x *= a1; og[1].y *= a1; og[1].z *= a1; og[1].w *= a1;
    }
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = fast_exp2(s0[r] - m_use);
        psum += s0[r];
    }
    l_run += psum;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(s0[2 * p]), __float_as_uint(s0[2 * p + 1]), false, false);
        const float va = Vt[(8 * (p >> 1) + 2 * (p & 1)) * LSV];
        og[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[0]), og[0], 0, 0, 0);
        og[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[1]), og[1], 0, 0, 0);
    }
}

// The 48-wide tile of the main kernel (head dims 36 .. 48): S^T takes 24 MFMAs, the columns 0 .. 31 of O^T one 32 x 32
// accumulator like the 32-wide tile (Vb: row 4 * half, column lane % 32), the columns 32 .. 47 two 16 x 16 accumulators like
// attend_tile_16 (Vt: row of the lane's MFMA slot, column 32 + lane % 16): 48 MFMA units per tile against the 64 of the
// 64-wide kernel these head dims ran on.
template <int KIND>
__device__ __forceinline__ void attend_tile_48(const float *Kb, const float *Vb, const float *Vt, const float (&qr)[24], f32x16 &o0,
                                               f32x4 (&og)[2], float &m_run, float &m_use, float &l_run, const int k0, const int q0,
                                               const int qi, const int half, const int ln, const int Lk, const int len,
                                               const float *mrow, const long long msk, const int cls) {
    constexpr int LSV = NarrowTile<48>::LSV;
    f32x16 s0 = masked_scores<KIND, 6>(Kb, qr, k0, q0, qi, half, Lk, len, mrow, msk, cls);
    const float tmax = max_across_halves(max_of_16(s0));
    const bool upd = tmax - m_run > 8.0f;      // also right at m_run = -inf: +inf, or NaN for tmax = -inf
    if (__any(upd)) {
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = (m_run == m_new) ? 1.0f : fast_exp2(m_run - m_new);
        m_run = m_new;
        m_use = (m_new == -INFINITY) ? 0.f : m_new;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) o0[i] *= alpha;
        const float other = __shfl_xor(alpha, 16, 64);
        const float a0 = ln < 16 ? alpha : other, a1 = ln < 16 ? other : alpha;
        og[0].x *= a0; og[0].y *= a0; og[0].z *= a0; og[0].w *= a0;
        og[1].x *= a1; og[1].y *= a1; og[1].z *= a1; og[1].w *= a1;
    }
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = fast_exp2(s0[r] - m_use);
        psum += s0[r];
    }
    l_run += psum;
#pragma unroll
    for (int r = 0; r < 16; ++r) o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(Vb[(8 * (r >> 2) + (r & 3)) * LSV], s0[r], o0, 0, 0, 0);
#pragma unroll
    for (int p = 0; p < 8; ++p) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(s0[2 * p]), __float_as_uint(s0[2 * p + 1]), false, false);
        const float va = Vt[(8 * (p >> 1) + 2 * (p & 1)) * LSV];
        og[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[0]), og[0], 0, 0, 0);
        og[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[1]), og[1], 0, 0, 0);
    }
}

// Stores the lane's query row: register r of o0 is d = 8(r/4) + 4*half + r%4.
__device__ __forceinline__ void store_row_narrow(float *op, const f32x16 &o0, const float inv, const int half, const int hd) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int d0 = 8 * g + 4 * half;
        const f32x4 a = {o0[4 * g + 0] * inv, o0[4 * g + 1] * inv, o0[4 * g + 2] * inv, o0[4 * g + 3] * inv};
        if (d0 < hd) *reinterpret_cast<f32x4 *>(op + d0) = a;
    }
}

template <int KIND, int W>
__global__ __launch_bounds__(256, 4) void sdpa_prefill_f32_narrow(const float *__restrict__ q, const float *__restrict__ k,
                                                                   const float *__restrict__ v, float *__restrict__ out, int H,
                                                                   int Lq, int Lk, float rT, MaskArgs mask, int strict, int nqb,
                                                                   int total_blocks, int lpt, int token_major,
                                                                   float *__restrict__ stats, int hd) {
    constexpr int LS = NarrowTile<W>::LS, TF = NarrowTile<W>::TF, LSV = NarrowTile<W>::LSV, TFV = NarrowTile<W>::TFV;
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;              // [2][BN][LS]
    float *Vs = lds + 2 * TF;     // [2][BN][LSV]

    int bh, unit;
    if (!work_item(nqb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
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
    const int rs = token_major ? H * hd : hd;   // hd: the tensors' head dim, a multiple of 4 up to W; tiles are zero beyond it
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

    float qr[W / 2];   // Q[qi][half * W/2 + s] * rT (one rounding, the reference's q / temperature) * log2(e)
    {
        const float *qp = q + q_base + (long long)qic * rs + half * (W / 2);
#pragma unroll
        for (int j = 0; j < W / 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * (W / 2) + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E; qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E; qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // global -> LDS staging.  W = 32: every thread moves one 128-bit piece of the K tile and one of the V tile (row tid/8,
    // column 4 * (tid%8)).  W = 16: wavefronts 0, 1 move the K tile and wavefronts 2, 3 the V tile (row t/4, column
    // 4 * (t%4) with t = tid % 128).  W = 48: 384 pieces per tile - every thread piece tid of both tiles, the threads of
    // wavefronts 0, 1 also piece tid + 256.  Rows at or beyond Lk and columns at or beyond hd lie outside the descriptor: zeros.
    constexpr int CPR = W / 4;                       // 128-bit pieces per tile row
    const int st = (W == 16) ? (tid & 127) : tid;
    const int ld_row = st / CPR, ld_col = (st % CPR) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    const int lds_off = ld_row * LS + ld_col, lds_off_v = ld_row * LSV + ld_col;
    const int ld_row2 = (tid + 256) / CPR, ld_col2 = ((tid + 256) % CPR) * 4;      // W = 48, wavefronts 0, 1
    const unsigned ld_off2 = ld_col2 < hd ? (unsigned)(ld_row2 * rs + ld_col2) * 4u : 0x80000000u;
    const int lds_off2 = ld_row2 * LS + ld_col2, lds_off2_v = ld_row2 * LSV + ld_col2;
    f32x4 kst, vst, kst2, vst2;
    auto load_tile = [&](int t) {
        const int o = (int)(ld_off + t * tile_bytes);
        if (W != 16) {
            kst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
            vst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
            if (W == 48 && wave < 2) {
                const int o2 = (int)(ld_off2 + t * tile_bytes);
                kst2 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o2, 0, 0));
                vst2 = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o2, 0, 0));
            }
        } else if (wave < 2) {
            kst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
        } else {
            kst = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
        }
    };
    auto store_tile = [&](int buf) {
        if (W != 16) {
            *reinterpret_cast<f32x4 *>(Ks + buf * TF + lds_off) = kst;
            *reinterpret_cast<f32x4 *>(Vs + buf * TFV + lds_off_v) = vst;
            if (W == 48 && wave < 2) {
                *reinterpret_cast<f32x4 *>(Ks + buf * TF + lds_off2) = kst2;
                *reinterpret_cast<f32x4 *>(Vs + buf * TFV + lds_off2_v) = vst2;
            }
        } else {
            if (wave < 2) *reinterpret_cast<f32x4 *>(Ks + buf * TF + lds_off) = kst;
            else *reinterpret_cast<f32x4 *>(Vs + buf * TFV + lds_off_v) = kst;
        }
    };

    f32x16 o0;   // O^T, row d = 8(r/4) + 4*half + r%4
#pragma unroll
    for (int i = 0; i < 16; ++i) o0[i] = 0.f;
    f32x4 og[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};   // W = 16: O^T on two 16 x 16 accumulators (attend_tile_16); W = 48: its columns 32 .. 47
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    const int k_lds = ln * LS + half * (W / 2);
    const int v_lds = (4 * half) * LSV + ln;
    const int slot = lane >> 4;
    const int v_lds16 = ((slot & 1) + 4 * (slot >> 1)) * LSV + (W == 48 ? 32 : 0) + (lane & 15);
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    auto tile_step = [&](const int t, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const bool more = (t + 1 < ntiles);
        if (more) load_tile(t + 1);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (k0 < wkend && !(DENSE && skip_ones && cls == 1)) {
            if constexpr (W == 16)
                attend_tile_16<KIND>(Ks + buf * TF + k_lds, Vs + buf * TFV + v_lds16, qr, og, m_run, m_use, l_run, k0, q0, qi, half, ln, Lk,
                                     len, mrow, mask.sk, cls);
            else if constexpr (W == 48)
                attend_tile_48<KIND>(Ks + buf * TF + k_lds, Vs + buf * TFV + v_lds, Vs + buf * TFV + v_lds16, qr, o0, og, m_run, m_use, l_run,
                                     k0, q0, qi, half, ln, Lk, len, mrow, mask.sk, cls);
            else
                attend_tile_narrow<KIND, W>(Ks + buf * TF + k_lds, Vs + buf * TFV + v_lds, qr, o0, m_run, m_use, l_run, k0, q0, qi, half, Lk,
                                            len, mrow, mask.sk, cls);
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        if (t + 1 < ntiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    }

    const float l_tot = sum_across_halves(l_run);
    const float inv = 1.0f / l_tot;
    if (stats && half == 0 && qi < Lq) {
        stats[2 * ((long long)bh * Lq + qi)] = m_use;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    if constexpr (W != 16) {
        if (qi < Lq) store_row_narrow(out + q_base + (long long)qi * rs, o0, inv, half, hd);
    }
    if constexpr (W != 32) {
        // group g of the lane: query q0 + 16 g + lane % 16, columns (32 +) 4 * slot ..; the reciprocal sum of that query is the
        // lane's own when the lane's query lies in the group, else the one of the lane 16 away
        const float other = __shfl_xor(inv, 16, 64);
        const int d0 = (W == 48 ? 32 : 0) + 4 * slot;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int qg = q0 + 16 * g + (lane & 15);
            const float f = ((ln < 16) == (g == 0)) ? inv : other;
            const f32x4 a = {og[g].x * f, og[g].y * f, og[g].z * f, og[g].w * f};
            if (qg < Lq && d0 < hd) *reinterpret_cast<f32x4 *>(out + q_base + (long long)qg * rs + d0) = a;
        }
    }
}

// Small launches: one workgroup = 32 queries, its key tiles dealt round-robin to the 4 wavefronts through
// wavefront-private LDS tiles, the four partial results merged at the end (see sdpa_prefill_split_f32_d64).
template <int KIND, int W>
__global__ __launch_bounds__(256, 2) void sdpa_prefill_split_f32_narrow(const float *__restrict__ q, const float *__restrict__ k,
                                                                         const float *__restrict__ v, float *__restrict__ out,
                                                                         int H, int Lq, int Lk, float rT, MaskArgs mask, int strict,
                                                                         int nqb, int total_blocks, int token_major,
                                                                         float *__restrict__ stats, int hd, int order) {
    constexpr int LS = NarrowTile<W>::LS, TF = NarrowTile<W>::TF;
    constexpr int REGION = 2 * TF;     // a wavefront's K tile and V tile; later its partial result [18][64]
    static_assert(REGION >= 18 * 64, "the merge records must fit a wavefront's tile region");
    extern __shared__ __align__(16) float lds[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, half = lane >> 5, ln = lane & 31;
    float *Ks = lds + wave * REGION;
    float *Vs = Ks + TF;

    int bh, unit;
    if (!work_item(nqb, total_blocks, order & 1, bh, unit, order >> 1)) return;
    const int qb = nqb - 1 - unit;
    const int b = bh / H, hh = bh % H;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int q0 = qb * 32;
    const int qi = q0 + ln;
    const int qic = qi < Lq ? qi : Lq - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    int kend = Lk;
    bool skip_ones = false;
    if (!strict && !(LENS && len <= 0)) {
        if (DENSE && mask.cls) {
            const int blk = min(q0, Lq - 1) >> 5;
            const unsigned char *row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)blk * mask.cls_sq;
            skip_ones = dense_block_open(row, mask.cls_sk, blk, (Lk + 31) >> 5);
            kend = dense_key_bound(row, mask.cls_sk, blk, Lk);
        }
        if (CAUSAL) kend = min(kend, q0 + 32);
        if (LENS) kend = min(kend, len);
    }
    const int ntiles = (kend + BN - 1) / BN;

    float qr[W / 2];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * (W / 2);
#pragma unroll
        for (int j = 0; j < W / 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * (W / 2) + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E; qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E; qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // the wavefront stages its own tiles: W/8 pieces of 128 bits per lane and tensor, piece c = lane + 64 i is row c / (W/4),
    // column 4 * (c % (W/4))
    constexpr int CPR = W / 4, NP = W / 8;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const int ld_row = lane / CPR, ld_col = (lane % CPR) * 4;       // piece i is 64 / CPR rows further down
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned piece_bytes = (unsigned)(64 / CPR) * rs * 4u, tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[NP], vst[NP];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int o = (int)(ld_off + t * tile_bytes + i * piece_bytes);
            kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
            vst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int off = (i * (64 / CPR) + ld_row) * LS + ld_col;
            *reinterpret_cast<f32x4 *>(Ks + off) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + off) = vst[i];
        }
    };

    f32x16 o0;
#pragma unroll
    for (int i = 0; i < 16; ++i) o0[i] = 0.f;
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    const int k_lds = ln * LS + half * (W / 2);
    const int v_lds = (4 * half) * LS + ln;
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    if (wave < ntiles) {
        load_tile(wave);
        store_tile();
    }
    for (int t = wave; t < ntiles; t += SPLIT_WAVES) {
        const bool more = (t + SPLIT_WAVES < ntiles);
        if (more) load_tile(t + SPLIT_WAVES);
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (!(DENSE && skip_ones && cls == 1))
            attend_tile_narrow<KIND, W>(Ks + k_lds, Vs + v_lds, qr, o0, m_run, m_use, l_run, t * BN, q0, qi, half, Lk, len, mrow, mask.sk, cls);
        if (more) store_tile();
    }

    // Merge the four partial results (reference maximum, row sum, O^T) in wavefront order: every wavefront leaves its
    // partial result in its own (dead) tile region, and behind the one barrier wavefront w folds the accumulator registers
    // 4w .. 4w + 3 of the four (8 of the 32 columns) and stores them - see sdpa_prefill_split_f32_d64.
    {
        const float l_part = sum_across_halves(l_run);
        float *mine = lds + wave * REGION;   // rows 0..15 = o0 registers, row 16 = m_run, row 17 = row sum
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[r * 64 + lane] = o0[r];
        mine[16 * 64 + lane] = m_run;
        mine[17 * 64 + lane] = l_part;
    }
    __syncthreads();
    float m_all = lds[16 * 64 + lane];
#pragma unroll
    for (int x = 1; x < SPLIT_WAVES; ++x) m_all = fmaxf(m_all, lds[x * REGION + 16 * 64 + lane]);
    const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
    float l_tot = 0.f, acc[4];
#pragma unroll
    for (int x = 0; x < SPLIT_WAVES; ++x) {
        const float *part = lds + x * REGION;
        const float mx = part[16 * 64 + lane];
        const float fx = (mx == -INFINITY) ? 1.0f : fast_exp2(mx - m_ref);
        const float *rows = part + (4 * wave) * 64 + lane;
        if (x == 0) {
            l_tot = part[17 * 64 + lane] * fx;
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = rows[r * 64] * fx;
        } else {
            l_tot += part[17 * 64 + lane] * fx;
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += rows[r * 64] * fx;
        }
    }
    const float inv = 1.0f / l_tot;
    if (stats && wave == 0 && half == 0 && qi < Lq) {
        stats[2 * ((long long)bh * Lq + qi)] = m_ref;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    const int d0 = 8 * wave + 4 * half;      // store_row_narrow's group `wave`
    if (qi < Lq && d0 < hd) {
        const f32x4 a = {acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
        *reinterpret_cast<f32x4 *>(out + q_base + (long long)qi * rs + d0) = a;
    }
}

// The launch rules of launch_d64 (sdpa_prefill.hip).  32 floats of LDS beyond the tiles: at W = 16 the lanes that stand for
// rows d >= 16 of O^T read up to 11 floats past the last V tile.
template <int KIND, int W>
int launch_narrow(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk,
                  float rT, const MaskArgs &m, int strict, int token_major, int no_split, float *stats, int hd) {
    constexpr int TF = NarrowTile<W>::TF, TFV = NarrowTile<W>::TFV;
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    const bool uneven = (causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict;
    const long long waves = (long long)B * H * ((Lq + 31) / 32);
    // (from 1024 keys on up to sixteen wavefronts per CU: B1 H8 L8192 d32 causal 382 -> 292 us, B1 H16 L4096 203 -> 161 us,
    // B3 H16 L2048 145 -> 129 us, without a mask 3 - 7 %; with short rows the 128-query kernel wins from eight on: B16 H16 L256
    // 20 us against 24 us)
    if (!no_split && (waves < 8ll * ctx->cu_count || (Lk >= 1024 && waves < 16ll * ctx->cu_count)) && Lk >= 2 * BN) {
        const int nqb32 = (Lq + 31) / 32;
        const long long total32 = (long long)nqb32 * B * H;
        DL4S_REQUIRE(total32 < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total32);
        int order = 0;
        if (uneven && nqb32 >= 2) order = 1 | (total32 <= 2ll * ctx->cu_count ? (ctx->cu_count / 8) << 1 : 0);
        hipLaunchKernelGGL((sdpa_prefill_split_f32_narrow<KIND, W>), dim3((unsigned)((total32 + 7) / 8 * 8)), dim3(256),
                           (size_t)(SPLIT_WAVES * 2 * TF + 32) * sizeof(float), ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb32,
                           (int)total32, token_major, stats, hd, order);
        return dl4s::launch_status("sdpa_prefill_split_f32_narrow");
    }
    const int nqb = (Lq + BM - 1) / BM;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    const int lpt = (uneven && nqb >= 2) ? 1 : 0;
    // every second round of the CUs reversed as well, on launches of any size: these short workgroups (16 or 32 columns)
    // gain from it well beyond the four per CU that are resident at once (B5 H16 L2048 d32 causal 216 -> 191 us, B6
    // 248 -> 222 us, B8 299 -> 295 us; d16 133 -> 119, 154 -> 138, 188 -> 180 us), where the 64-wide kernel starts to lose
    const int lpt_arg = lpt | (lpt ? (ctx->cu_count / 8) << 1 : 0);
    hipLaunchKernelGGL((sdpa_prefill_f32_narrow<KIND, W>), dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), (size_t)(2 * TF + 2 * TFV + 32) * sizeof(float),
                       ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt_arg, token_major, stats, hd);
    return dl4s::launch_status("sdpa_prefill_f32_narrow");
}

// The 48-column form of the main kernel for head dims 36 .. 48 on launches large enough for it (small ones run the 64-wide
// key-split kernel)
template <int KIND>
int launch_narrow48_main(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk,
                         float rT, const MaskArgs &m, int strict, int token_major, float *stats, int hd) {
    constexpr int TF = NarrowTile<48>::TF, TFV = NarrowTile<48>::TFV;
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    const bool uneven = (causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict;
    const int nqb = (Lq + BM - 1) / BM;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    const int lpt = (uneven && nqb >= 2) ? 1 : 0;
    // (reversed rounds up to five workgroups per CU, like the 64-wide kernel: B5 H16 L2048 d48 296 -> 289 us, beyond it loses)
    const int lpt_arg = lpt | ((lpt && total <= 5ll * ctx->cu_count) ? (ctx->cu_count / 8) << 1 : 0);
    hipLaunchKernelGGL((sdpa_prefill_f32_narrow<KIND, 48>), dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), (size_t)(2 * TF + 2 * TFV + 32) * sizeof(float),
                       ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt_arg, token_major, stats, hd);
    return dl4s::launch_status("sdpa_prefill_f32_narrow");
}

}  // namespace

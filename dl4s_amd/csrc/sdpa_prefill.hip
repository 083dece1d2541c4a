// Fused attention forward for gfx950: out = softmax((q * rT) . k^T - mask * 1e9) . v
//
// sdpa_prefill_f32_d64 is the hot kernel (head dim 64; smaller head dims padded with zero columns).  One workgroup = 4 wavefronts = 128
// queries of one (batch, head); each wavefront owns 32 queries and walks the keys in LDS tiles of
// 32.  Both contractions run on v_mfma_f32_32x32x2_f32 and are set up TRANSPOSED so that the
// probabilities never leave the registers they were computed in:
//
//   S^T[key, query] = K[key, :] . Q[query, :]      A operand = K (from LDS), B operand = Q (registers)
//   O^T[d,   query] = V[key, d]^T . P^T[key, query] A operand = V (from LDS), B operand = P (the S^T
//                                                   accumulator registers, used as they are)
//
// In the 32x32 accumulator layout lane l holds column (l % 32) = one query and 16 rows = 16 keys,
// which is exactly the B-operand layout of the second contraction (k = l / 32, n = l % 32) once
// the key order inside a tile is permuted consistently for V.  The row maximum and row sum are
// therefore 16 in-lane operations plus one exchange with lane l ^ 32.
//
// The scale is applied to Q once (q * rT), as the reference does before its first matrix product
// (NN/Models/Transformer/ScaledDotProductAttention.swift:53), followed by a factor log2(e) so that the scores live in
// the base-2 exponent domain; the mask is applied in registers (the base-2 image of s - m * 1e9, ibid. :55-57) before
// the running maximum; normalisation by the row sum is deferred to the end.  Keys beyond Lk contribute nothing;
// queries beyond Lq are computed and not stored.
//
// Kernels in this file: sdpa_prefill_f32_d64 (above), sdpa_prefill_split_f32_d64 (small launches: the keys of a
// 32-query block split over the 4 wavefronts of a workgroup), sdpa_generic_f32 (head dims the MFMA kernels do not take);
// sdpa_prefill_f32_d128 for head dims above 64 up to 128 is in sdpa_prefill_d128.h.  The two 64-wide MFMA kernels can
// also leave the two row statistics the backward pass needs (sdpa_backward.hip).
#include <type_traits>

#include "sdpa_common.h"
#include "sdpa_prefill_d128.h"
#include "sdpa_prefill_w96.h"
#include "sdpa_prefill_wide.h"
#include "sdpa_prefill_narrow.h"

namespace {

// One 32-key tile for one wavefront (32 queries): S^T = K.Q^T, mask, online softmax update, O^T += V^T.P^T.
// Kb / Vb point at the lane's K and V fragment bases of the tile in LDS; mrow is the lane's row of a dense mask
// (element stride msk along keys), cls the tile's mask class.
template <int KIND>
__device__ __forceinline__ void attend_tile(const float *Kb, const float *Vb, const float (&qr)[32], f32x16 &o0, f32x16 &o1,
                                            float &m_run, float &m_use, float &l_run, const int k0, const int q0, const int qi,
                                            const int half, const int Lk, const int len, const float *mrow, const long long msk,
                                            const int cls) {
    f32x16 s0 = masked_scores<KIND>(Kb, qr, k0, q0, qi, half, Lk, len, mrow, msk, cls);

    // ---- online softmax: lane (query ln) sees 16 of the 32 keys, lane ^ 32 the other 16.
    // Vector-ALU instructions do not overlap the matrix pipe on a SIMD (measured: their cycles add to the MFMA
    // cycles), so the reduction is kept to about four instructions per score: max3, one fma + exp2, one add.
    // The reference maximum m_run only moves -- and the accumulators are only rescaled -- when a tile's maximum
    // would give a weight above 2^8; any per-row factor 2^(max - m_run) left in the weights cancels in the
    // final division by the row sum.
    const float tmax = max_across_halves(max_of_16(s0));
    // tmax above m_run by more than 8; with m_run = -inf the difference is +inf for any other tmax and NaN for tmax = -inf
    const bool upd = tmax - m_run > 8.0f;
    if (__any(upd)) {
        const float m_new = fmaxf(m_run, tmax);
        // lanes whose maximum did not move keep factor 1 (also when it is still -inf: -inf - -inf would be NaN)
        const float alpha = (m_run == m_new) ? 1.0f : fast_exp2(m_run - m_new);
        m_run = m_new;
        m_use = (m_new == -INFINITY) ? 0.f : m_new;      // a row of -inf so far: weights 0, not NaN
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) { o0[i] *= alpha; o1[i] *= alpha; }
    }
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s0[r] = fast_exp2(s0[r] - m_use);
        psum += s0[r];
    }
    l_run += psum;

    // ---- O^T += V^T . P^T.  Row = key (+ 4*half, folded into v_lds), columns 2*ln, 2*ln+1.
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const f32x2 vv = *reinterpret_cast<const f32x2 *>(Vb + (8 * (r >> 2) + (r & 3)) * LSTR);
        o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, s0[r], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, s0[r], o1, 0, 0, 0);
    }
}

// Four workgroups per CU (128 registers, 34 KiB of LDS each).  The structured kinds fit by themselves; the dense-mask
// kind needs 138 registers unbounded and spills 7 outside the MFMA chains to fit, which pays: dense causal B8 H16 L2048
// 588 -> 567 us, every tile visited 1079 -> 1061 us, B8 H16 L1024 all tiles 288 -> 278 us.
template <int KIND>
__device__ __forceinline__ void prefill_block_d64(const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                                                  float *__restrict__ out, const int H, const int Lq, const int Lk, const float rT,
                                                  const MaskArgs &mask, const int strict, const int nqb, const int total_blocks,
                                                  const int lpt, const int token_major, float *__restrict__ stats, const int hd) {
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                     // [2][BN][LSTR]
    float *Vs = lds + 2 * TILE_FLOATS;   // [2][BN][LSTR]

    int bh, unit;   // unit 0 = the last (longest) query block of the pair
    if (!work_item(nqb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H;
    const int hh = bh % H;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: lets the per-wavefront tile conditions branch on scalars
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int ln = lane & 31;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int qb = nqb - 1 - unit;  // longest rows first
    const int q0 = qb * BM + wave * 32;  // first query of this wavefront
    const int qi = q0 + ln;
    const int qic = qi < Lq ? qi : Lq - 1;

    int len = Lk;
    if (LENS) len = mask.lengths[b];

    // Tensor layout: [B,H,L,64] (row stride 64) or, token-major, [B,L,H,64] (row stride H*64): the projections of
    // MultiHeadAttention come out token-major, so reading them in place saves the four permuteAxes copies.
    // hd = the tensors' head dim (a multiple of 4, at most 64): rows are hd floats long; columns hd..63 of every tile are
    // zeros, which leaves scores and outputs unchanged
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    // Keys this workgroup / wavefront has to visit.  Skipping is exact when every row keeps at least one
    // unblocked key (true unless len == 0) and K, V are finite at blocked keys.
    int kend = Lk, wkend = Lk;
    bool skip_ones = false;   // dense masks: this wavefront's all-ones tiles have weight exactly zero
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) {
            kend = min(kend, qb * BM + BM);
            wkend = min(wkend, q0 + 32);
        }
        if (LENS) {
            kend = min(kend, len);
            wkend = min(wkend, len);
        }
        if (DENSE && mask.cls) dense_key_bounds(mask, b, hh, qb * BM, wave, Lq, Lk, kend, wkend, skip_ones);
    }
    const int ntiles = (kend + BN - 1) / BN;

    // Q fragment: lane holds Q[qi][half*32 + s] * rT (one rounding, like the reference's q / temperature) times log2(e):
    // the scores then come out of the MFMAs in the base-2 exponent domain and the weights are exp2(s - max), one
    // subtraction per score and -- as in the reference -- the subtraction before anything can overflow.
    float qr[32];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E;
            qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E;
            qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // global -> LDS staging: thread covers rows (i*16 + tid/16), 4 floats at column (tid%16)*4.  K and V are read with
    // buffer loads whose whole byte offset is in the vector operand (the only part the hardware range-checks): rows at
    // or beyond Lk fall outside the descriptor's range and read as zeros (their scores are then set to -inf by the key
    // bound below), so the loop needs neither address arithmetic beyond one add nor clamps.
    const int ld_row = tid >> 4;
    const int ld_col = (tid & 15) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);   // extent of this pair's rows; the host keeps it below 2^31
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    // columns at or beyond hd: an offset outside every descriptor (they stay below 2^31 bytes), i.e. zeros
    const unsigned ld_off0 = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;   // unsigned: sums may pass 2^31
    const unsigned ld_off1 = ld_off0 + 16u * rs * 4u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[2], vst[2];
    auto load_tile = [&](int t) {
        const int o0 = (int)(ld_off0 + t * tile_bytes), o1 = (int)(ld_off1 + t * tile_bytes);
        kst[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o0, 0, 0));
        vst[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o0, 0, 0));
        kst[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o1, 0, 0));
        vst[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o1, 0, 0));
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int off = buf * TILE_FLOATS + (i * 16 + ld_row) * LSTR + ld_col;
            *reinterpret_cast<f32x4 *>(Ks + off) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + off) = vst[i];
        }
    };

    f32x16 o0, o1;  // O^T rows d = 2*m + {0,1}
#pragma unroll
    for (int i = 0; i < 16; ++i) { o0[i] = 0.f; o1[i] = 0.f; }
    float m_run = -INFINITY;   // reference maximum of the row, base-2 exponent domain (see the softmax step)
    float m_use = 0.f;         // m_run, or 0 while m_run is -inf
    float l_run = 0.f;

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    const int k_lds = ln * LSTR + half * 32;        // K fragment base: row ln, columns half*32..
    const int v_lds = (4 * half) * LSTR + 2 * ln;   // V fragment base: row 4*half (+ const), columns 2*ln, 2*ln+1

    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;   // wavefronts past Lq store nothing

    // the classes of 64 key tiles at a time, one per lane, read ahead of the loop: a class byte fetched inside a tile step
    // would put a global load's latency on every step's critical path
    int clsv = 2;
    auto load_classes = [&](const int t0) {
        const int t = t0 + lane;
        clsv = t < ntiles ? (int)cls_row[(long long)t * mask.cls_sk] : 2;
    };
    if (DENSE && cls_row) load_classes(0);

    // one key tile; the LDS buffer index is a compile-time constant (the loop is unrolled by two), so every LDS address
    // in the step is a per-thread base plus a literal
    auto tile_step = [&](const int t, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const bool more = (t + 1 < ntiles);
        if (more) load_tile(t + 1);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) {
            if ((t & 63) == 0 && t > 0) load_classes(t);
            cls = __builtin_amdgcn_readlane(clsv, t & 63) & 3;
        }

        if (k0 < wkend && !(DENSE && skip_ones && cls == 1)) {
            attend_tile<KIND>(Ks + buf * TILE_FLOATS + k_lds, Vs + buf * TILE_FLOATS + v_lds, qr, o0, o1, m_run, m_use, l_run, k0, q0,
                              qi, half, Lk, len, mrow, mask.sk, cls);
        }

        if (more) store_tile(buf ^ 1);
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        if (t + 1 < ntiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    }

    // ---- normalise and store.  Register r of o0/o1 is d = 2*(8(r/4) + 4*half + r%4) + {0,1}.
    const float l_tot = sum_across_halves(l_run);
    const float inv = 1.0f / l_tot;
    // row statistics for the backward pass, [B,H,Lq,2]: the reference maximum m and 1 / sum_j 2^(s_j - m), so that a weight
    // is 2^(s - m) * that (kept apart: m can be of the order of the 1e9 mask penalty, where a float cannot also hold log2 l)
    if (stats && half == 0 && qi < Lq) {
        stats[2 * ((long long)bh * Lq + qi)] = m_use;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    if (qi < Lq) {
        float *op = out + q_base + (long long)qi * rs + 8 * half;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            f32x4 a, c;
            a.x = o0[4 * g + 0] * inv; a.y = o1[4 * g + 0] * inv;
            a.z = o0[4 * g + 1] * inv; a.w = o1[4 * g + 1] * inv;
            c.x = o0[4 * g + 2] * inv; c.y = o1[4 * g + 2] * inv;
            c.z = o0[4 * g + 3] * inv; c.w = o1[4 * g + 3] * inv;
            if (8 * half + 16 * g < hd) *reinterpret_cast<f32x4 *>(op + 16 * g) = a;
            if (8 * half + 16 * g + 4 < hd) *reinterpret_cast<f32x4 *>(op + 16 * g + 4) = c;
        }
    }
}

// Two kernels over the one body: the default launch, and the launch that visits every key tile (DL4S_SDPA_STRICT) under
// a name of its own, so that a profile of a program that makes both kinds of call keeps their durations apart (the
// strict launch of a causal problem issues twice the MFMAs).
template <int KIND>
__global__ __launch_bounds__(256, 4) void sdpa_prefill_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                const float *__restrict__ v, float *__restrict__ out, int H, int Lq,
                                                                int Lk, float rT, MaskArgs mask, int nqb, int total_blocks, int lpt,
                                                                int token_major, float *__restrict__ stats, int hd) {
    prefill_block_d64<KIND>(q, k, v, out, H, Lq, Lk, rT, mask, 0, nqb, total_blocks, lpt, token_major, stats, hd);
}
template <int KIND>
__global__ __launch_bounds__(256, 4) void sdpa_prefill_strict_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                       const float *__restrict__ v, float *__restrict__ out, int H,
                                                                       int Lq, int Lk, float rT, MaskArgs mask, int nqb,
                                                                       int total_blocks, int lpt, int token_major,
                                                                       float *__restrict__ stats, int hd) {
    prefill_block_d64<KIND>(q, k, v, out, H, Lq, Lk, rT, mask, 1, nqb, total_blocks, lpt, token_major, stats, hd);
}

// Variant for launches with too few wavefronts to fill the GPU (fewer 32-query wavefronts than about two per SIMD):
// one workgroup = 32 queries of one (batch, head), and its 4 wavefronts share the keys, wavefront w taking the 32-key
// tiles w, w + 4, w + 8, ... through a wavefront-private LDS tile (no workgroup barrier in the loop).  At the end the
// four partial results (reference maximum, row sum, O^T) are merged through LDS, each wavefront finishing 16 of the 64 columns.
// Same tile arithmetic as the kernel above; the summation order over keys differs, so results agree with it within
// rounding, not bit for bit.  Which of the two kernels runs depends on the extents only, never on the mask.
template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_prefill_split_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                      const float *__restrict__ v, float *__restrict__ out,
                                                                      int H, int Lq, int Lk, float rT, MaskArgs mask,
                                                                      int strict, int nqb, int total_blocks, int token_major,
                                                                      float *__restrict__ stats, int hd, int order) {
    extern __shared__ __align__(16) float lds[];
    // every argument the block's first loads depend on is asked for at once: fetched as the code first needs them, the
    // arguments arrive in three round trips, one behind the other, before the first row is requested
    asm volatile("" ::"s"(q), "s"(k), "s"(v), "s"(out), "s"(H), "s"(Lq), "s"(Lk), "s"(rT), "s"(nqb), "s"(total_blocks),
                 "s"(token_major), "s"(hd), "s"(order), "s"(strict), "s"(stats));
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: lets the per-wavefront tile conditions branch on scalars
    const int lane = tid & 63;
    const int half = lane >> 5;
    const int ln = lane & 31;
    float *Ks = lds + wave * 2 * TILE_FLOATS;   // this wavefront's K tile, then its V tile
    float *Vs = Ks + TILE_FLOATS;

    int bh, unit;
    if (!work_item(nqb, total_blocks, order & 1, bh, unit, order >> 1)) return;
    const int qb = nqb - 1 - unit;   // longest rows first
    const int b = bh / H;
    const int hh = bh % H;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int q0 = qb * 32;
    const int qi = q0 + ln;
    const int qic = qi < Lq ? qi : Lq - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    // hd = the tensors' head dim (a multiple of 4, at most 64): rows are hd floats long; columns hd..63 of every tile are
    // zeros, which leaves scores and outputs unchanged
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    int kend = Lk;
    bool skip_ones = false;   // dense masks: the block's all-ones tiles have weight exactly zero
    if (!strict && !(LENS && len <= 0)) {
        if (DENSE && mask.cls) {   // trailing all-ones tiles of an open block
            const int blk = min(q0, Lq - 1) >> 5;
            const unsigned char *row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)blk * mask.cls_sq;
            skip_ones = dense_block_open(row, mask.cls_sk, blk, (Lk + 31) >> 5);
            kend = dense_key_bound(row, mask.cls_sk, blk, Lk);
        }
        if (CAUSAL) kend = min(kend, q0 + 32);
        if (LENS) kend = min(kend, len);
    }
    const int ntiles = (kend + BN - 1) / BN;

    float qr[32];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            qr[4 * j + 0] = (t.x * rT) * LOG2E;
            qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E;
            qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // the wavefront stages its own tiles: lane covers rows (i*4 + lane/16), 4 floats at column (lane%16)*4
    const int ld_row = lane >> 4;
    const int ld_col = (lane & 15) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned row4_bytes = 4u * rs * 4u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[8], vst[8];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int o = (int)(ld_off + t * tile_bytes + i * row4_bytes);
            kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
            vst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int off = (i * 4 + ld_row) * LSTR + ld_col;
            *reinterpret_cast<f32x4 *>(Ks + off) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + off) = vst[i];
        }
    };

    f32x16 o0, o1;
#pragma unroll
    for (int i = 0; i < 16; ++i) { o0[i] = 0.f; o1[i] = 0.f; }
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    const int k_lds = ln * LSTR + half * 32;
    const int v_lds = (4 * half) * LSTR + 2 * ln;
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    // LDS operations of one wavefront execute in order, so the tile can be overwritten right after the reads of the
    // previous one were issued: no barrier, the prefetch of the next tile sits in registers meanwhile.
    if (wave < ntiles) {
        load_tile(wave);
        store_tile();
    }
    // the classes of this wavefront's next 64 tiles, one per lane, read ahead of the loop (a class byte fetched inside a
    // step would put a global load's latency on every step's critical path)
    int clsv = 2;
    auto load_classes = [&](const int t0) {
        const int t = t0 + SPLIT_WAVES * lane;
        clsv = t < ntiles ? (int)cls_row[(long long)t * mask.cls_sk] : 2;
    };
    if (DENSE && cls_row) load_classes(wave);
    for (int t = wave, j = 0; t < ntiles; t += SPLIT_WAVES, ++j) {
        const bool more = (t + SPLIT_WAVES < ntiles);
        if (more) load_tile(t + SPLIT_WAVES);
        int cls = 2;
        if (DENSE && cls_row) {
            if ((j & 63) == 0 && j > 0) load_classes(t);
            cls = __builtin_amdgcn_readlane(clsv, j & 63) & 3;
        }
        if (!(DENSE && skip_ones && cls == 1))
            attend_tile<KIND>(Ks + k_lds, Vs + v_lds, qr, o0, o1, m_run, m_use, l_run, t * BN, q0, qi, half, Lk, len, mrow, mask.sk, cls);
        if (more) store_tile();
    }

    // ---- merge the four partial results.  Every wavefront leaves (m_run, row sum, O^T) in its own LDS region (its
    // tiles are dead by now, and the LDS operations of one wavefront execute in order: no barrier before the writes);
    // after the barrier wavefront w folds the four partial results of the accumulator registers 4w .. 4w + 3 (16 of the
    // 64 output columns) in the order 0, 1, 2, 3 and stores them.  A partial result with m_run = -inf has seen no finite
    // score: its sums are zeros (or NaN, which must survive), so it is added with factor 1.
    {
        const float l_part = sum_across_halves(l_run);
        float *mine = lds + wave * 2 * TILE_FLOATS;   // [34][64]: rows 0..31 = o0/o1 registers, row 32 = m_run, row 33 = row sum
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            mine[(2 * r) * 64 + lane] = o0[r];
            mine[(2 * r + 1) * 64 + lane] = o1[r];
        }
        mine[32 * 64 + lane] = m_run;
        mine[33 * 64 + lane] = l_part;
    }
    __syncthreads();
    float m_all = lds[32 * 64 + lane];
#pragma unroll
    for (int x = 1; x < SPLIT_WAVES; ++x) m_all = fmaxf(m_all, lds[x * 2 * TILE_FLOATS + 32 * 64 + lane]);
    const float m_ref = (m_all == -INFINITY) ? 0.f : m_all;
    float l_tot = 0.f, acc[8];
#pragma unroll
    for (int x = 0; x < SPLIT_WAVES; ++x) {
        const float *part = lds + x * 2 * TILE_FLOATS;
        const float mx = part[32 * 64 + lane];
        const float fx = (mx == -INFINITY) ? 1.0f : fast_exp2(mx - m_ref);
        const float *rows = part + (8 * wave) * 64 + lane;   // rows 8w .. 8w + 7 = o0[4w], o1[4w], o0[4w + 1], ...
        if (x == 0) {
            l_tot = part[33 * 64 + lane] * fx;
#pragma unroll
            for (int r = 0; r < 8; ++r) acc[r] = rows[r * 64] * fx;
        }
        else {
            l_tot += part[33 * 64 + lane] * fx;
#pragma unroll
            for (int r = 0; r < 8; ++r) acc[r] += rows[r * 64] * fx;
        }
    }
    const float inv = 1.0f / l_tot;
    if (stats && wave == 0 && half == 0 && qi < Lq) {
        stats[2 * ((long long)bh * Lq + qi)] = m_ref;
        stats[2 * ((long long)bh * Lq + qi) + 1] = inv;
    }
    if (qi < Lq) {
        float *op = out + q_base + (long long)qi * rs + 8 * half + 16 * wave;
        f32x4 a, c;
        a.x = acc[0] * inv; a.y = acc[1] * inv; a.z = acc[2] * inv; a.w = acc[3] * inv;
        c.x = acc[4] * inv; c.y = acc[5] * inv; c.z = acc[6] * inv; c.w = acc[7] * inv;
        if (8 * half + 16 * wave < hd) *reinterpret_cast<f32x4 *>(op) = a;
        if (8 * half + 16 * wave + 4 < hd) *reinterpret_cast<f32x4 *>(op + 4) = c;
    }
}

// Plain fused kernel for head dims other than 64 (up to 256): one wavefront per query row, two passes over
// the keys like the reference's softmax (max, then exp / sum), keys handled 64 at a time through LDS.
__global__ __launch_bounds__(64) void sdpa_generic_f32(const float *__restrict__ q, const float *__restrict__ k,
                                                        const float *__restrict__ v, float *__restrict__ out, int H,
                                                        int Lq, int Lk, int dk, int dv, float rT, MaskArgs mask,
                                                        float *__restrict__ stats) {
    __shared__ float qs[GEN_MAXD];
    __shared__ float ps[64];
    const int row = blockIdx.x;  // over B*H*Lq
    const int qi = row % Lq;
    const int bh = row / Lq;
    const int b = bh / H, hh = bh % H;
    const int lane = threadIdx.x;
    for (int c = lane; c < dk; c += 64) qs[c] = q[(long long)row * dk + c] * rT;
    __syncthreads();
    const float *kp = k + (long long)bh * Lk * dk;
    const float *vp = v + (long long)bh * Lk * dv;
    int len = Lk;
    if (mask.kind == DL4S_MASK_KEY_LENGTHS || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS) len = mask.lengths[b];
    auto score = [&](int j) { return plain_score(qs, kp + (long long)j * dk, dk, mask, b, hh, qi, j, len); };
    float mx = -INFINITY;
    for (int j = lane; j < Lk; j += 64) mx = fmaxf(mx, score(j));
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float acc[GEN_MAXD / 64];
    for (int i = 0; i < GEN_MAXD / 64; ++i) acc[i] = 0.f;
    float sum = 0.f;
    for (int j0 = 0; j0 < Lk; j0 += 64) {
        const int j = j0 + lane;
        float p = 0.f;
        if (j < Lk) p = expf(score(j) - mx);   // -inf - -inf = NaN for an all -inf row, like the reference
        sum += p;
        ps[lane] = p;
        __syncthreads();
        const int n = min(64, Lk - j0);
        for (int i = 0; i < GEN_MAXD / 64; ++i) {
            const int c = lane + 64 * i;
            if (c < dv)
                for (int jj = 0; jj < n; ++jj) acc[i] += ps[jj] * vp[(long long)(j0 + jj) * dv + c];
        }
        __syncthreads();
    }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    const float inv = 1.0f / sum;
    for (int i = 0; i < GEN_MAXD / 64; ++i) {
        const int c = lane + 64 * i;
        if (c < dv) out[(long long)row * dv + c] = acc[i] * inv;
    }
    if (stats && lane == 0) {     // row statistics for the backward pass: a weight is exp(s - mx) * inv
        stats[2 * (long long)row] = mx;
        stats[2 * (long long)row + 1] = inv;
    }
}

template <int KIND>
int launch_d64(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq,
               int Lk, float rT, const MaskArgs &m, int strict, int token_major, int no_split, float *stats, int hd) {
    // narrow heads: tiles of 16 or 32 columns
    if (hd <= 16) return launch_narrow<KIND, 16>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, no_split, stats, hd);
    if (hd <= 32) return launch_narrow<KIND, 32>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, no_split, stats, hd);
    // Too few 32-query wavefronts to give every SIMD about two: split the keys of each query block over 4 wavefronts.
    // The choice depends on the extents only, so every mask kind of one problem runs the same kernel.
    const long long waves = (long long)B * H * ((Lq + 31) / 32);
    if (!no_split && waves < 8ll * ctx->cu_count && Lk >= 2 * BN) {
        const int nqb32 = (Lq + 31) / 32;
        const long long total32 = (long long)nqb32 * B * H;
        DL4S_REQUIRE(total32 < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total32);
        const size_t lds_split = (size_t)SPLIT_WAVES * 2 * TILE_FLOATS * sizeof(float);
        if (dl4s::lds_limit_pending(ctx, dl4s::LDS_PREFILL_SPLIT, KIND)) {
            DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_prefill_split_f32_d64<KIND>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_split));
            dl4s::lds_limit_done(ctx, dl4s::LDS_PREFILL_SPLIT, KIND);
        }
        // Rows of different length (causal masks, dense masks with tile skipping): longest first, and when the launch fits
        // the chip at once (two workgroups per CU) every second round of the CUs reversed, which pairs long rows with
        // short ones on a CU.  B4 H8 L512 causal: 24.3 us pair-major, 19.5 us longest first, 17.6 us with the reversal.
        constexpr bool causal_kind32 = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
        int split_order = 0;
        if ((causal_kind32 || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb32 >= 2)
            split_order = 1 | (total32 <= 2ll * ctx->cu_count ? (ctx->cu_count / 8) << 1 : 0);
        hipLaunchKernelGGL(sdpa_prefill_split_f32_d64<KIND>, dim3((unsigned)((total32 + 7) / 8 * 8)), dim3(256), lds_split,
                           ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb32, (int)total32, token_major, stats, hd, split_order);
        return dl4s::launch_status("sdpa_prefill_split_f32_d64");
    }
    // head dims 36 .. 48: the 48-column form of the narrow kernel (48 MFMA units per tile instead of 64) - unless the call
    // leaves row statistics: the gradient kernels form the scores again in the 64-column order, and the statistics must
    // belong to those scores to the last bit
    if (hd <= 48 && !stats) return launch_narrow48_main<KIND>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd);
    const int nqb = (Lq + BM - 1) / BM;
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    // longest-first order for causal masks.  Measured on B8 H16 L2048 causal with the order applied to groups of
    // 16 (= the whole run) / 8 / 4 / 1 pairs: 120 / 111 / 107 / 87 TFLOP/s and 754 / 391 / 263 / 248 MiB of L2 fills
    // (the floor is 192 MiB): the kernel is MFMA-bound, the fills stay far below what the memory side delivers, so
    // balance wins over L2 reuse.
    const int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb >= 2) ? 1 : 0;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    const int chunk = (int)((total + 7) / 8);
    const size_t lds_bytes = 4 * TILE_FLOATS * sizeof(float);
    if (dl4s::lds_limit_pending(ctx, dl4s::LDS_PREFILL, KIND)) {
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_prefill_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_prefill_strict_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        dl4s::lds_limit_done(ctx, dl4s::LDS_PREFILL, KIND);
    }
    // a launch that fits the chip at once (four workgroups per CU), or nearly: little or nothing is left for the
    // dispatcher to balance, so every second round of the CUs is reversed as well (B2 H16 L2048 causal: 203 -> 161 us,
    // B4 H16 L1024: 106 -> 88 us; with exactly four per CU B4 H16 L2048 319 -> 277 us, B1 H16 L8192 1251 -> 1038 us,
    // B8 H16 L1024 165 -> 151 us; five per CU B5 H16 L2048 379 -> 362 us; from six per CU on it loses: B8 H16 L2048
    // 540 -> 555 us, B2 H16 L8192 2.03 -> 2.13 ms)
    const int lpt_arg = lpt | ((lpt && total <= 5ll * ctx->cu_count) ? (ctx->cu_count / 8) << 1 : 0);
    if (strict) {
        hipLaunchKernelGGL(sdpa_prefill_strict_f32_d64<KIND>, dim3(chunk * 8), dim3(256), lds_bytes, ctx->stream, q, k, v, out, H,
                           Lq, Lk, rT, m, nqb, (int)total, lpt_arg, token_major, stats, hd);
        return dl4s::launch_status("sdpa_prefill_strict_f32_d64");
    }
    hipLaunchKernelGGL(sdpa_prefill_f32_d64<KIND>, dim3(chunk * 8), dim3(256), lds_bytes, ctx->stream, q, k, v, out, H,
                       Lq, Lk, rT, m, nqb, (int)total, lpt_arg, token_major, stats, hd);
    return dl4s::launch_status("sdpa_prefill_f32_d64");
}

}  // namespace

namespace {
int sdpa_forward_locked(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, float *stats, int64_t B,
                        int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv, float inv_temperature, const dl4s_mask_desc *mask,
                        uint32_t flags);

// Head dims the MFMA kernels do not take as they are (key dim != value dim, not a multiple of 4, tensors off the 16-byte
// grid), up to 256: the operands are copied into tensors of one padded head dim - zero columns change neither scores nor
// outputs - the MFMA kernels run on the copies and the output's own columns are copied back.  Four streaming passes for
// a kernel that is 30 - 40 times faster than the one-wavefront-per-row fallback (B8 H16 L2048 d72: 42 ms there).
// Returns DL4S_HIP_EOOM without side effects when the copies cannot be allocated (the caller falls back).
int sdpa_forward_padded(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, float *stats, int64_t B,
                        int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv, float inv_temperature, const dl4s_mask_desc *mask,
                        uint32_t flags) {
    const int64_t dp = (std::max(dk, dv) + 3) / 4 * 4;
    const int64_t qrows = B * H * Lq, krows = B * H * Lk;
    void *bufs[4] = {nullptr, nullptr, nullptr, nullptr};
    const size_t sizes[4] = {(size_t)(qrows * dp) * 4, (size_t)(krows * dp) * 4, (size_t)(krows * dp) * 4, (size_t)(qrows * dp) * 4};
    for (int i = 0; i < 4; ++i)
        if (dl4s_hip_alloc(ctx, sizes[i], &bufs[i]) != DL4S_HIP_OK) {
            for (int j = 0; j < i; ++j) (void)dl4s_hip_free(ctx, bufs[j]);
            return DL4S_HIP_EOOM;
        }
    float *qp = static_cast<float *>(bufs[0]), *kp = static_cast<float *>(bufs[1]), *vp = static_cast<float *>(bufs[2]),
          *op = static_cast<float *>(bufs[3]);
    const auto copy = [&](const float *src, float *dst, long long rows, int64_t ds, int64_t dd) {
        launch_copy_rows(ctx, src, dst, rows, ds, dd);
    };
    copy(q, qp, qrows, dk, dp);
    copy(k, kp, krows, dk, dp);
    copy(v, vp, krows, dv, dp);
    int rc = dl4s::launch_status("copy_rows_f32");
    if (rc == DL4S_HIP_OK)
        rc = sdpa_forward_locked(ctx, qp, kp, vp, op, stats, B, H, Lq, Lk, dp, dp, inv_temperature, mask, flags);
    if (rc == DL4S_HIP_OK) {
        copy(op, out, qrows, dp, dv);
        rc = dl4s::launch_status("copy_rows_f32");
    }
    // the pool hands a block out again only to work enqueued later on the same stream
    for (int i = 0; i < 4; ++i) (void)dl4s_hip_free(ctx, bufs[i]);
    return rc;
}

int sdpa_forward(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, float *stats, int64_t B, int64_t H,
                 int64_t Lq, int64_t Lk, int64_t dk, int64_t dv, float inv_temperature, const dl4s_mask_desc *mask, uint32_t flags) {
    DL4S_CHECK_CTX(ctx);
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    return sdpa_forward_locked(ctx, q, k, v, out, stats, B, H, Lq, Lk, dk, dv, inv_temperature, mask, flags);
}

int sdpa_forward_locked(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, float *stats, int64_t B,
                        int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv, float inv_temperature, const dl4s_mask_desc *mask,
                        uint32_t flags) {
    DL4S_REQUIRE(B >= 0 && H >= 0 && Lq >= 0 && Lk >= 0 && dk >= 0 && dv >= 0, DL4S_HIP_EINVALID_ARG,
                 "sdpa: negative extent");
    if (B * H * Lq * dv == 0) return DL4S_HIP_OK;  // nothing to write
    DL4S_REQUIRE(q && k && v && out, DL4S_HIP_EINVALID_ARG, "sdpa: NULL tensor pointer");
    DL4S_REQUIRE(Lk > 0, DL4S_HIP_ESHAPE, "sdpa: keyCount is 0 (softmax over an empty axis)");
    DL4S_REQUIRE(dk > 0, DL4S_HIP_ESHAPE, "sdpa: keyDim is 0");
    DL4S_REQUIRE(B * H * (Lq > Lk ? Lq : Lk) * (dk > dv ? dk : dv) < (1ll << 40) && Lq < (1ll << 30) && Lk < (1ll << 30),
                 DL4S_HIP_EUNSUPPORTED, "sdpa: extents too large");
    // head dims that are multiples of 4 up to 64 run on the MFMA kernels (tiles padded with zero columns), as long as
    // every row starts on a 16-byte boundary
    const bool mfma_path = dk == dv && dk <= HD && dk % 4 == 0 &&
                           ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                             reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    // head dims above 64 up to 128: the 128-wide MFMA kernel
    const bool aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                           reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const bool mfma128_path = dk == dv && dk > HD && dk <= HD2 && dk % 4 == 0 && aligned;
    const int strict = (flags & DL4S_SDPA_STRICT) ? 1 : 0;
    const int token_major = (flags & DL4S_SDPA_TOKEN_MAJOR) ? 1 : 0;
    const int no_split = (flags & DL4S_SDPA_NO_KEY_SPLIT) ? 1 : 0;
    // head dims above 64 up to 96: the 96-wide kernel, which on launches that fill the GPU without a key split also takes
    // even head dims that are not a multiple of 4 as they are (rows on the 8-byte grid)
    const bool aligned8 = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                            reinterpret_cast<uintptr_t>(out)) & 7) == 0;
    const bool w96_path = dk == dv && dk > HD && dk <= W96 &&
                          ((dk % 4 == 0 && aligned) ||
                           (dk % 2 == 0 && aligned8 && !token_major && ((Lq + BM - 1) / BM) * B * H >= 2ll * ctx->cu_count &&
                            // with row statistics only where the gradient call's rule lands on the MFMA kernels as well (it
                            // pads such head dims, sdpa_padded_route): the statistics have the MFMA kernels' base-2 form
                            (!stats || sdpa_padded_route(false, B, H, Lq, Lk, dk, dv)))) &&
                          Lk * (token_major ? H : 1) * dk * 4 < (1ll << 30);   // its 32-bit K/V offsets; beyond: the routes below
    // head dims above 128 up to 256: the 192- and 256-wide kernels (the gradient call evaluates sdpa_wide_route on the same
    // arguments)
    const bool wide_as_is = dk == dv && aligned && dk > HD2 && dk <= 256 && dk % 4 == 0;   // never copied, whichever kernel it runs
    const bool wide_path = wide_as_is && sdpa_wide_route(H, Lk, dk, token_major);
    // The 128-wide kernel on a launch that leaves CUs without their two workgroups: the key tiles of every block are dealt
    // to several workgroups, whose partial results a second kernel adds up (B4 H8 L512 d128: 73 us unsplit).  The count
    // depends on the extents only.
    int nsplit128 = 1;
    size_t part_bytes = 0;
    if ((mfma128_path || (w96_path && dk % 4 == 0)) && !no_split) {
        const long long blocks = ((Lq + BM - 1) / BM) * B * H, nkt = (Lk + BN - 1) / BN;
        // the count that leaves the fewest rounds of the CUs per share (sdpa_key_shares); two where every CU just has one block
        // (blocks of different length then pair up long with short through the order of their workgroups: B2 H8 L2048 d256
        // causal 570 -> 353 us; without a mask 569 -> 609 us - the count depends on the extents only, so that every mask kind of
        // a problem adds in one order)
        if (blocks < 2ll * ctx->cu_count && nkt >= 4) {
            const long long want = sdpa_key_shares(blocks, nkt, ctx->cu_count, 0.02);
            const size_t bytes = (size_t)want * B * H * Lq * PART2_STRIDE * sizeof(float);
            if (want > 1 && bytes <= (size_t(256) << 20)) { nsplit128 = (int)want; part_bytes = bytes; }
        }
    }
    // the wide kernels run one workgroup per CU: the same split on launches that leave CUs without one
    if (wide_path && !no_split) {
        const long long blocks = ((Lq + BM - 1) / BM) * B * H, nkt = (Lk + BN - 1) / BN;
        // the count that leaves the fewest rounds of the CUs per share (sdpa_key_shares); two where every CU just has one block
        // (blocks of different length then pair up long with short through the order of their workgroups: B2 H8 L2048 d256
        // causal 570 -> 353 us; without a mask 569 -> 609 us - the count depends on the extents only, so that every mask kind of
        // a problem adds in one order)
        if (blocks < 2ll * ctx->cu_count && nkt >= 4) {
            const long long want = sdpa_key_shares(blocks, nkt, ctx->cu_count, 0.045);
            const size_t bytes = (size_t)want * B * H * Lq * PARTW_STRIDE * sizeof(float);
            if (want > 1 && bytes <= (size_t(256) << 20)) { nsplit128 = (int)want; part_bytes = bytes; }
        }
    }
    MaskArgs m{};
    void *part128 = nullptr;
    {
        const int rc = build_mask_args(ctx, mask, B, H, Lq, Lk, mfma_path || mfma128_path || w96_path || wide_path, m, part_bytes, &part128);
        if (rc != DL4S_HIP_OK) return rc;
    }
    DL4S_REQUIRE((flags & ~(uint32_t)(DL4S_SDPA_STRICT | DL4S_SDPA_TOKEN_MAJOR | DL4S_SDPA_NO_KEY_SPLIT)) == 0, DL4S_HIP_EINVALID_ARG,
                 "sdpa: unknown flag bits 0x%x", flags);
    if (mfma_path) {
        // the MFMA kernel addresses one (batch, head) pair's K/V rows through a 32-bit byte offset
        // (half of that for head dims below 64, whose padding columns use offsets from 2^31 up that must not wrap)
        DL4S_REQUIRE(Lk * (token_major ? H : 1) * dk * 4 < (dk == HD ? (1ll << 31) : (1ll << 30)), DL4S_HIP_EUNSUPPORTED,
                     "sdpa: the K/V rows of one (batch, head) pair span more than 2 GiB (1 GiB for head dims below 64)");
        switch (m.kind) {
            case DL4S_MASK_NONE: return launch_d64<DL4S_MASK_NONE>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, no_split, stats, (int)dk);
            case DL4S_MASK_DENSE_F32: return launch_d64<DL4S_MASK_DENSE_F32>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, no_split, stats, (int)dk);
            case DL4S_MASK_CAUSAL: return launch_d64<DL4S_MASK_CAUSAL>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, no_split, stats, (int)dk);
            case DL4S_MASK_KEY_LENGTHS: return launch_d64<DL4S_MASK_KEY_LENGTHS>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, no_split, stats, (int)dk);
            default: return launch_d64<DL4S_MASK_CAUSAL_OR_KEY_LENGTHS>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, no_split, stats, (int)dk);
        }
    }
    if (w96_path) {
        if (dk % 4 == 0)
            return launch_w96<4>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128,
                                 static_cast<float *>(part128));
        return launch_w96<2>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk);
    }
    if (mfma128_path) {
        DL4S_REQUIRE(Lk * (token_major ? H : 1) * dk * 4 < (dk == HD2 ? (1ll << 31) : (1ll << 30)), DL4S_HIP_EUNSUPPORTED,
                     "sdpa: the K/V rows of one (batch, head) pair span more than 2 GiB (1 GiB for padded head dims)");
        switch (m.kind) {
            case DL4S_MASK_NONE: return launch_d128<DL4S_MASK_NONE>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, static_cast<float *>(part128));
            case DL4S_MASK_DENSE_F32: return launch_d128<DL4S_MASK_DENSE_F32>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, static_cast<float *>(part128));
            case DL4S_MASK_CAUSAL: return launch_d128<DL4S_MASK_CAUSAL>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, static_cast<float *>(part128));
            case DL4S_MASK_KEY_LENGTHS: return launch_d128<DL4S_MASK_KEY_LENGTHS>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, static_cast<float *>(part128));
            default: return launch_d128<DL4S_MASK_CAUSAL_OR_KEY_LENGTHS>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, static_cast<float *>(part128));
        }
    }
    if (wide_path) {
        float *partw = static_cast<float *>(part128);
        if (dk <= 160) return launch_wide<160>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, partw);
        if (dk <= 192) return launch_wide<192>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, partw);
        return launch_wide<256>(ctx, q, k, v, out, B, H, Lq, Lk, inv_temperature, m, strict, token_major, stats, (int)dk, nsplit128, partw);
    }
    DL4S_REQUIRE(!token_major, DL4S_HIP_EUNSUPPORTED, "sdpa: the token-major layout needs equal head dims that are a multiple of 4, at most 128, and 16-byte aligned tensors");
    // Large enough to pay for four copies: the MFMA kernels on padded copies of the operands.  When row statistics are
    // asked for there is no falling back to the plain kernel: the gradient call decides by the same rule and reads the
    // statistics in the MFMA kernels' form.
    if (sdpa_padded_route(wide_as_is, B, H, Lq, Lk, dk, dv)) {
        const int rc = sdpa_forward_padded(ctx, q, k, v, out, stats, B, H, Lq, Lk, dk, dv, inv_temperature, mask, flags);
        if (stats || (rc != DL4S_HIP_EOOM && rc != DL4S_HIP_EUNSUPPORTED)) return rc;   // else: the plain kernel below
    }
    DL4S_REQUIRE(dk <= GEN_MAXD && dv <= GEN_MAXD && dv > 0, DL4S_HIP_EUNSUPPORTED,
                 "sdpa: head dims (%lld, %lld) above %d are not implemented", (long long)dk, (long long)dv, GEN_MAXD);
    const long long rows = B * H * Lq;
    DL4S_REQUIRE(rows < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "sdpa: too many rows for the plain kernel");
    hipLaunchKernelGGL(sdpa_generic_f32, dim3((unsigned)rows), dim3(64), 0, ctx->stream, q, k, v, out, (int)H, (int)Lq,
                       (int)Lk, (int)dk, (int)dv, inv_temperature, m, stats);
    return dl4s::launch_status("sdpa_generic_f32");
}
}  // namespace

extern "C" int dl4s_hip_sdpa_fwd_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out,
                                     int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv,
                                     float inv_temperature, const dl4s_mask_desc *mask, uint32_t flags) {
    return sdpa_forward(ctx, q, k, v, out, nullptr, B, H, Lq, Lk, dk, dv, inv_temperature, mask, flags);
}

extern "C" int dl4s_hip_sdpa_fwd_stats_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out,
                                           float *stats, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t d,
                                           float inv_temperature, const dl4s_mask_desc *mask, uint32_t flags) {
    DL4S_REQUIRE(stats || B * H * Lq == 0, DL4S_HIP_EINVALID_ARG, "sdpa: stats pointer is NULL");
    return sdpa_forward(ctx, q, k, v, out, stats, B, H, Lq, Lk, d, d, inv_temperature, mask, flags);
}

// ---- tile classes of a dense mask, prepared once for many attention calls
namespace {
// number of class bytes of a dense mask broadcastable to [B,H,Lq,Lk]
int mask_class_count(const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk, long long &total) {
    DL4S_REQUIRE(mask && mask->kind == DL4S_MASK_DENSE_F32, DL4S_HIP_EINVALID_ARG, "mask classes: the descriptor is not a dense mask");
    const int64_t full[4] = {B, H, Lq, Lk};
    for (int i = 0; i < 4; ++i)
        DL4S_REQUIRE(full[i] > 0 && (mask->shape[i] == 1 || mask->shape[i] == full[i]), DL4S_HIP_ESHAPE,
                     "mask classes: mask axis %d has size %lld, expected 1 or %lld", i, (long long)mask->shape[i], (long long)full[i]);
    total = (mask->shape[0] == 1 ? 1 : B) * (mask->shape[1] == 1 ? 1 : H) * (mask->shape[2] == 1 ? 1 : (Lq + 31) / 32) *
            (mask->shape[3] == 1 ? 1 : (Lk + 31) / 32);
    DL4S_REQUIRE(total < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "mask classes: more than 2^31 tiles");
    return DL4S_HIP_OK;
}
}  // namespace

extern "C" int dl4s_hip_mask_classes_size(const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk, size_t *out_bytes) {
    DL4S_REQUIRE(out_bytes, DL4S_HIP_EINVALID_ARG, "mask classes: NULL argument");
    long long total = 0;
    const int rc = mask_class_count(mask, B, H, Lq, Lk, total);
    if (rc != DL4S_HIP_OK) return rc;
    *out_bytes = (size_t)total;
    return DL4S_HIP_OK;
}

extern "C" int dl4s_hip_mask_classify_f32(dl4s_hip_ctx *ctx, const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                                          uint8_t *classes) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(classes, DL4S_HIP_EINVALID_ARG, "mask classes: NULL argument");
    long long total = 0;
    int rc = mask_class_count(mask, B, H, Lq, Lk, total);
    if (rc != DL4S_HIP_OK) return rc;
    DL4S_REQUIRE(mask->dense, DL4S_HIP_EINVALID_ARG, "mask classes: dense mask pointer is NULL");
    MaskArgs m{};
    dl4s_mask_desc plain = *mask;
    plain.classes = nullptr;
    rc = build_mask_args(ctx, &plain, B, H, Lq, Lk, false, m);
    if (rc != DL4S_HIP_OK) return rc;
    const int MB = m.sb ? (int)B : 1, MH = m.sh ? (int)H : 1;
    const int nqt = m.sq ? (int)((Lq + 31) / 32) : 1, nkt = m.sk ? (int)((Lk + 31) / 32) : 1;
    hipLaunchKernelGGL(sdpa_mask_classify, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, ctx->stream, m, MB, MH, nqt, nkt, (int)Lq,
                       (int)Lk, total, classes);
    return dl4s::launch_status("sdpa_mask_classify");
}

// ---- a dense mask whose values are exactly those of a structured kind
namespace {
// One workgroup per mask batch entry: the number of leading zeros of the entry's designated row (the only row of a mask
// without a query axis, the last query's row otherwise), as the valid key count the structured kinds would need to
// reproduce the mask.  Under the causal rule a count that reaches the last query blocks nothing beyond what the rule
// blocks already: it is recorded as Lk.  ok[0] is set to 1 for the verification pass.
__global__ __launch_bounds__(256) void sdpa_mask_structure_lengths(MaskArgs m, int Lq, int Lk, int causal, int *lengths, int *ok) {
    __shared__ int first_one;
    const int bm = blockIdx.x;
    if (threadIdx.x == 0) first_one = Lk;
    __syncthreads();
    const float *row = m.dense + bm * m.sb + (causal ? (long long)(Lq - 1) * m.sq : 0);
    const int jmax = causal ? min(Lk, Lq) : Lk;     // beyond the last query the causal rule blocks anyway
    int mine = Lk;
    for (int j = threadIdx.x; j < jmax; j += 256)
        if (row[j * m.sk] != 0.0f) { mine = j; break; }
    if (mine < Lk) atomicMin(&first_one, mine);
    __syncthreads();
    if (threadIdx.x == 0) {
        lengths[bm] = first_one >= jmax ? Lk : first_one;
        if (bm == 0) ok[0] = 1;
    }
}
// Every element against the structured kind's rule: 1 where key j >= lengths[b] or (causal) j > query i, else 0.
__global__ __launch_bounds__(256) void sdpa_mask_structure_verify(MaskArgs m, int MB, int nq, int Lk, int causal, const int *lengths,
                                                                  int *ok) {
    const long long total = (long long)MB * nq * Lk;
    bool bad = false;
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
        const int j = (int)(e % Lk);
        const int i = (int)((e / Lk) % nq);
        const int bm = (int)(e / Lk / nq);
        const float want = (j >= lengths[bm] || (causal && j > i)) ? 1.0f : 0.0f;
        bad = bad || !(m.dense[bm * m.sb + i * m.sq + j * m.sk] == want);
    }
    if (bad) ok[0] = 0;
}
}  // namespace

extern "C" int dl4s_hip_mask_describe_f32(dl4s_hip_ctx *ctx, const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                                          int32_t *lengths, dl4s_mask_desc *out) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(mask && out && lengths, DL4S_HIP_EINVALID_ARG, "mask describe: NULL argument");
    DL4S_NOT_WHILE_CAPTURING(ctx);
    *out = *mask;
    if (mask->kind != DL4S_MASK_DENSE_F32) return DL4S_HIP_OK;
    long long tiles = 0;
    int rc = mask_class_count(mask, B, H, Lq, Lk, tiles);      // validates the shape
    if (rc != DL4S_HIP_OK) return rc;
    DL4S_REQUIRE(mask->dense, DL4S_HIP_EINVALID_ARG, "mask describe: dense mask pointer is NULL");
    // the structured kinds know no head axis, and a query axis only through the causal rule
    const bool has_b = mask->shape[0] != 1, has_h = mask->shape[1] != 1, has_q = mask->shape[2] != 1, has_k = mask->shape[3] != 1;
    if (has_h || (!has_k && Lk > 1) || B > 65536 || Lq >= (1ll << 30) || Lk >= (1ll << 30)) return DL4S_HIP_OK;
    const int causal = has_q ? 1 : 0;
    const int MB = has_b ? (int)B : 1;
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    rc = dl4s::ensure_scratch(ctx, 256);
    if (rc != DL4S_HIP_OK) return rc;
    int *ok = static_cast<int *>(ctx->scratch);
    MaskArgs m{};
    dl4s_mask_desc plain = *mask;
    plain.classes = nullptr;
    rc = build_mask_args(ctx, &plain, B, H, Lq, Lk, false, m);
    if (rc != DL4S_HIP_OK) return rc;
    // one workgroup per batch element (a mask without a batch axis has stride 0 there: every element reads the one entry)
    hipLaunchKernelGGL(sdpa_mask_structure_lengths, dim3((unsigned)B), dim3(256), 0, ctx->stream, m, (int)Lq, (int)Lk, causal, lengths, ok);
    rc = dl4s::launch_status("sdpa_mask_structure_lengths");
    if (rc != DL4S_HIP_OK) return rc;
    const int nq = has_q ? (int)Lq : 1;
    const long long total = (long long)MB * nq * Lk;
    const unsigned grid = (unsigned)std::min<long long>((total + 255) / 256, 4096);
    hipLaunchKernelGGL(sdpa_mask_structure_verify, dim3(grid), dim3(256), 0, ctx->stream, m, MB, nq, (int)Lk, causal, lengths, ok);
    rc = dl4s::launch_status("sdpa_mask_structure_verify");
    if (rc != DL4S_HIP_OK) return rc;
    std::vector<int32_t> host((size_t)MB + 1);
    DL4S_HIP_TRY(hipMemcpyAsync(host.data(), lengths, sizeof(int32_t) * MB, hipMemcpyDeviceToHost, ctx->stream));
    DL4S_HIP_TRY(hipMemcpyAsync(host.data() + MB, ok, sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (!host[(size_t)MB]) return DL4S_HIP_OK;      // not a structured mask: *out is the dense descriptor
    bool all_open = true;
    for (int b = 0; b < MB; ++b) all_open = all_open && host[(size_t)b] >= Lk;
    dl4s_mask_desc d{};
    d.kind = all_open ? (causal ? DL4S_MASK_CAUSAL : DL4S_MASK_NONE) : (causal ? DL4S_MASK_CAUSAL_OR_KEY_LENGTHS : DL4S_MASK_KEY_LENGTHS);
    d.lengths = all_open ? nullptr : lengths;
    *out = d;
    return DL4S_HIP_OK;
}

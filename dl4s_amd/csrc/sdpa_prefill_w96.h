// Fused attention forward for head dims above 64 and up to 96: the scheme of sdpa_prefill_f32_d128
// (sdpa_prefill_d128.h) on tiles that are 96 columns wide, and with a second staging form for head dims that are even
// but not a multiple of 4 (rows on an 8-byte grid: 64-bit loads and stores), which the other MFMA kernels only take
// through zero-padded copies of the operands.  Included by sdpa_prefill.hip only.
//
//   S^T[key, query] = K[key, :] . Q[query, :]        48 MFMA steps: step s contracts d = 48*half + s
//   O^T[d,   query] = V[key, d]^T . P^T[key, query]   three accumulators: accumulator c row i is d = 32*c + i; V is read
//                                                    a float at a time (consecutive lanes, consecutive columns), and
//                                                    register r of accumulator c is d = 32c + 8(r/4) + 4*half + r%4:
//                                                    four consecutive outputs per 128-bit (or two 64-bit) stores
//
// 96 MFMAs per 32 x 32 tile of (query, key) pairs against the 128-wide kernel's 128: a head dim of 96 costs three
// quarters, and one of 70 runs without the four streaming copies.  Head dims up to 80 run the W = 80 form (below).  One workgroup = 4 wavefronts = 128 queries of one
// (batch, head) pair, K/V in double-buffered LDS tiles of 32 keys on a 100-float row stride (2 x 2 x 32 x 100 floats =
// 50 KiB).  Mask kinds, tile skipping, the work order, the token-major layout (head dims that are multiples of 4) and
// the row statistics are those of the other forward kernels.  Small launches (head dims that are multiples of 4) are
// split over the keys across workgroups like the 128-wide kernel: share y of n takes the key tiles y, y + n, ... and
// sdpa_prefill_merge_d128 adds the shares up.
#pragma once
#include "sdpa_common.h"

namespace {

constexpr int W96 = 96;
constexpr int LSTR96 = W96 + 4;            // 100 = 4 mod 32: the bank spread of the other tile widths
constexpr int TILE96_FLOATS = BN * LSTR96;

// VEC: floats per staging access, 4 (head dim a multiple of 4, tensors on the 16-byte grid) or 2 (head dim even, 8-byte grid)
// W: 96, or 80 for head dims up to 80: the same tiles in LDS (columns from the head dim up are zeros either way), but the
// score product contracts 40 steps per half (d = 40*half + s) and the columns 64 .. 79 of O^T live in two 16 x 16
// accumulators on v_mfma_f32_16x16x4_f32 (queries 0-15 and 16-31 of the wavefront; lane: column = lane % 16, rows
// d = 64 + 4 * (lane / 16) + i), fed through v_permlane16_swap like attend_tile_16 (sdpa_prefill_narrow.h): 80 MFMA units
// per tile instead of 96.
// Three workgroups per CU with 128-bit staging (168 registers; the kinds that need a few more spill 4 to 21 outside the MFMA
// chains and still gain: B8 H16 L2048 d96 causal 846 -> 827 us, key lengths 1109 -> 1081 us, dense causal 922 -> 891 us), two
// with 64-bit staging, whose address arithmetic does not fit (d90 causal 880 us against 905 us at three).
template <int KIND, int VEC, int W = 96>
__global__ __launch_bounds__(256, VEC == 4 ? 3 : 2) void sdpa_prefill_f32_w96(const float *__restrict__ q, const float *__restrict__ k,
                                                                const float *__restrict__ v, float *__restrict__ out, int H, int Lq,
                                                                int Lk, float rT, MaskArgs mask, int strict, int nqb, int total_blocks,
                                                                int lpt, int token_major, float *__restrict__ stats, int hd,
                                                                int nsplit, float *__restrict__ part, int shares_adjacent) {
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                       // [2][BN][LSTR96]
    float *Vs = lds + 2 * TILE96_FLOATS;   // [2][BN][LSTR96]
    int bh, unit;
    // key split with blocks of different length: see sdpa_prefill_f32_d128
    int blk = ((lpt & 1) && (blockIdx.y & 1) && !shares_adjacent) ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;
    int sp = blockIdx.y;     // this workgroup's share of the key tiles: sp, sp + nsplit, ...
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

    // Q fragment: Q[qi][(W/2)*half + s] * rT (one rounding, like the reference's q / temperature) * log2(e); zeros beyond hd
    float qr[W / 2];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * (W / 2);
#pragma unroll
        for (int j = 0; j < W / 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            const int c0 = half * (W / 2) + 4 * j;
            if (VEC == 4) {
                if (c0 < hd) t = *reinterpret_cast<const f32x4 *>(qp + 4 * j);
            } else {
                if (c0 < hd) { const f32x2 a = *reinterpret_cast<const f32x2 *>(qp + 4 * j); t.x = a.x; t.y = a.y; }
                if (c0 + 2 < hd) { const f32x2 a = *reinterpret_cast<const f32x2 *>(qp + 4 * j + 2); t.z = a.x; t.w = a.y; }
            }
            qr[4 * j + 0] = (t.x * rT) * LOG2E;
            qr[4 * j + 1] = (t.y * rT) * LOG2E;
            qr[4 * j + 2] = (t.z * rT) * LOG2E;
            qr[4 * j + 3] = (t.w * rT) * LOG2E;
        }
    }

    // global -> LDS staging: a tile is 32 rows of 96 / VEC pieces; thread tid moves the pieces tid, tid + 256, ...
    // (3 of 128 bits or 6 of 64 bits for K and as many for V).  Buffer loads with the whole byte offset in the
    // range-checked vector operand: rows past Lk and columns past hd read as zeros.
    constexpr int PPR = W96 / VEC;            // pieces per tile row
    constexpr int NP = BN * PPR / 256;        // pieces per thread
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    unsigned ld_off[NP];
    int lds_off[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int p = tid + 256 * i, row = p / PPR, col = (p % PPR) * VEC;
        ld_off[i] = col < hd ? (unsigned)(row * rs + col) * 4u : 0x80000000u;
        lds_off[i] = row * LSTR96 + col;
    }
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    using piece_t = typename std::conditional<VEC == 4, f32x4, f32x2>::type;
    piece_t kst[NP], vst[NP];
    auto load_tile = [&](int t) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int o = (int)(ld_off[i] + t * tile_bytes);
            if constexpr (VEC == 4) {
                kst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, o, 0, 0));
                vst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, o, 0, 0));
            } else {
                kst[i] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(krsrc, o, 0, 0));
                vst[i] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(vrsrc, o, 0, 0));
            }
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            *reinterpret_cast<piece_t *>(Ks + buf * TILE96_FLOATS + lds_off[i]) = kst[i];
            *reinterpret_cast<piece_t *>(Vs + buf * TILE96_FLOATS + lds_off[i]) = vst[i];
        }
    };

    constexpr int NC = W == 96 ? 3 : 2;    // 32 x 32 accumulators
    f32x16 o[3];
#pragma unroll
    for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[c][i] = 0.f;
    f32x4 og[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};   // W = 80: the columns 64 .. 79
    float m_run = -INFINITY, m_use = 0.f, l_run = 0.f;

    if (sp < ntiles) { load_tile(sp); store_tile(0); }
    __syncthreads();

    const int k_lds = ln * LSTR96 + half * (W / 2);     // K fragment base: row ln, columns (W/2)*half ..
    const int v_lds = (4 * half) * LSTR96 + ln;          // V operand base: row 4*half (+ const), column ln (+ 32c)
    const int slot = lane >> 4;
    const int v_lds16 = ((slot & 1) + 4 * (slot >> 1)) * LSTR96 + 64 + (lane & 15);   // W = 80: row of the lane's MFMA slot, column 64 + lane % 16
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    for (int t = sp, buf = 0; t < ntiles; t += nsplit, buf ^= 1) {
        const bool more = (t + nsplit < ntiles);
        if (more) load_tile(t + nsplit);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (k0 < wkend && !(DENSE && skip_ones && cls == 1)) {
            f32x16 s0 = masked_scores<KIND, W / 8>(Ks + buf * TILE96_FLOATS + k_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
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
                if constexpr (W == 80) {    // the other group's factor comes from the lane 16 away
                    const float other = __shfl_xor(alpha, 16, 64);
                    const float a0 = ln < 16 ? alpha : other, a1 = ln < 16 ? other : alpha;
                    og[0].x *= a0; og[0].y *= a0; og[0].z *= a0; og[0].w *= a0;
                    og[1].x *= a1; og[1].y *= a1; og[1].z *= a1; og[1].w *= a1;
                }
            }
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s0[r] = fast_exp2(s0[r] - m_use);
                psum += s0[r];
            }
            l_run += psum;
            const float *Vb = Vs + buf * TILE96_FLOATS + v_lds;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float *vr = Vb + (8 * (r >> 2) + (r & 3)) * LSTR96;
                o[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[0], s0[r], o[0], 0, 0, 0);
                o[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[32], s0[r], o[1], 0, 0, 0);
                if constexpr (W == 96) o[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(vr[64], s0[r], o[2], 0, 0, 0);
            }
            if constexpr (W == 80) {
                const float *Vt = Vs + buf * TILE96_FLOATS + v_lds16;
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(s0[2 * p]), __float_as_uint(s0[2 * p + 1]), false, false);
                    const float va = Vt[(8 * (p >> 1) + 2 * (p & 1)) * LSTR96];
                    og[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[0]), og[0], 0, 0, 0);
                    og[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(va, __uint_as_float(sw[1]), og[1], 0, 0, 0);
                }
            }
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- normalise and store
    const float l_tot = sum_across_halves(l_run);
    if (part) {   // this share's weighted sums as they are, with their reference maximum and row sum
        if (qi < Lq) {
            float *pp = part + (((long long)sp * (total_blocks / nqb) + bh) * Lq + qi) * PART2_STRIDE;
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x4 a = {o[c][4 * g + 0], o[c][4 * g + 1], o[c][4 * g + 2], o[c][4 * g + 3]};
                    *reinterpret_cast<f32x4 *>(pp + 32 * c + 8 * g + 4 * half) = a;
                }
            if (half == 0) { pp[HD2] = m_run; pp[HD2 + 1] = l_tot; }
        }
        if constexpr (W == 80) {     // the 16 x 16 accumulators: query q0 + 16 g + lane % 16, columns 64 + 4 * slot ..
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const int qg = q0 + 16 * g + (lane & 15);
                if (qg < Lq)
                    *reinterpret_cast<f32x4 *>(part + (((long long)sp * (total_blocks / nqb) + bh) * Lq + qg) * PART2_STRIDE + 64 + 4 * slot) = og[g];
            }
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
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * c + 8 * g + 4 * half;
                const f32x4 a = {o[c][4 * g + 0] * inv, o[c][4 * g + 1] * inv, o[c][4 * g + 2] * inv, o[c][4 * g + 3] * inv};
                if (VEC == 4) {
                    if (d0 < hd) *reinterpret_cast<f32x4 *>(op + d0) = a;
                } else {
                    const f32x2 lo = {a.x, a.y}, hi = {a.z, a.w};
                    if (d0 < hd) *reinterpret_cast<f32x2 *>(op + d0) = lo;
                    if (d0 + 2 < hd) *reinterpret_cast<f32x2 *>(op + d0 + 2) = hi;
                }
            }
    }
    if constexpr (W == 80) {
        // the reciprocal sum of a group's query is the lane's own when its query lies in the group, else the lane's 16 away
        const float other = __shfl_xor(inv, 16, 64);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const int qg = q0 + 16 * g + (lane & 15), d0 = 64 + 4 * slot;
            const float f = ((ln < 16) == (g == 0)) ? inv : other;
            const f32x4 a = {og[g].x * f, og[g].y * f, og[g].z * f, og[g].w * f};
            if (qg < Lq) {
                float *op = out + q_base + (long long)qg * rs;
                if (VEC == 4) {
                    if (d0 < hd) *reinterpret_cast<f32x4 *>(op + d0) = a;
                } else {
                    const f32x2 lo = {a.x, a.y}, hi = {a.z, a.w};
                    if (d0 < hd) *reinterpret_cast<f32x2 *>(op + d0) = lo;
                    if (d0 + 2 < hd) *reinterpret_cast<f32x2 *>(op + d0 + 2) = hi;
                }
            }
        }
    }
}

template <int KIND, int VEC, int W>
int launch_w96_kind(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk,
                    float rT, const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit, float *part) {
    const int nqb = (Lq + BM - 1) / BM;
    const long long total = (long long)nqb * B * H;
    DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa: %lld workgroups exceed the grid limit", total);
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb >= 2) ? 1 : 0;
    if (lpt && total <= 5ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
    const size_t lds_bytes = 4 * TILE96_FLOATS * sizeof(float);   // 50 KiB: within the default limit
    if (nsplit <= 1 || !part || VEC != 4) { nsplit = 1; part = nullptr; }
    hipLaunchKernelGGL((sdpa_prefill_f32_w96<KIND, VEC, W>), dim3((unsigned)((total + 7) / 8 * 8), (unsigned)nsplit), dim3(256), lds_bytes,
                       ctx->stream, q, k, v, out, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt, token_major, stats, hd, nsplit, part,
                       ((total + 7) / 8 * 8 * nsplit > (VEC == 4 ? 3ll : 2ll) * ctx->cu_count) ? 1 : 0);   // (beyond what is resident at once)
    const int st = dl4s::launch_status("sdpa_prefill_f32_w96");
    if (st != DL4S_HIP_OK || nsplit == 1) return st;
    const long long rows = (long long)B * H * Lq;
    hipLaunchKernelGGL(sdpa_prefill_merge_d128, dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, ctx->stream, part, out, stats, nsplit, rows,
                       H, Lq, hd, token_major);
    return dl4s::launch_status("sdpa_prefill_merge_d128");
}

template <int VEC, int W>
int launch_w96_width(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk, float rT,
                     const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit, float *part) {
    switch (m.kind) {
        case DL4S_MASK_NONE: return launch_w96_kind<DL4S_MASK_NONE, VEC, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_DENSE_F32: return launch_w96_kind<DL4S_MASK_DENSE_F32, VEC, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_CAUSAL: return launch_w96_kind<DL4S_MASK_CAUSAL, VEC, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        case DL4S_MASK_KEY_LENGTHS: return launch_w96_kind<DL4S_MASK_KEY_LENGTHS, VEC, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
        default: return launch_w96_kind<DL4S_MASK_CAUSAL_OR_KEY_LENGTHS, VEC, W>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
    }
}

// head dims up to 80 on the 80-column form, the others on all 96 (the gradient kernels choose by the same rule, so that they
// form the scores in the summation order of the call that left the row statistics)
template <int VEC>
int launch_w96(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, int B, int H, int Lq, int Lk, float rT,
               const MaskArgs &m, int strict, int token_major, float *stats, int hd, int nsplit = 1, float *part = nullptr) {
    if (hd <= 80) return launch_w96_width<VEC, 80>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
    return launch_w96_width<VEC, 96>(ctx, q, k, v, out, B, H, Lq, Lk, rT, m, strict, token_major, stats, hd, nsplit, part);
}

}  // namespace

// Shared by the attention forward and backward kernels for gfx950: tile constants of the 64-wide kernels, the mask
// descriptor as the kernels see it, the dense-mask tile classifier, the masked score tile and the plain-kernel helpers.
#pragma once
#include "common.h"

#include <algorithm>
#include "work_order.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 64;       // head dim of the MFMA kernel
constexpr int BM = 128;      // queries per workgroup
constexpr int BN = 32;       // keys per LDS tile
constexpr int LSTR = 68;     // LDS row stride in floats: 64 + 4 keeps 128-bit reads of 8 rows on distinct banks
constexpr int TILE_FLOATS = BN * LSTR;
constexpr float LOG2E = 1.44269504088896340736f;
// the 128-wide kernels (head dims above 64 up to 128)
constexpr int HD2 = 128;
constexpr int LSTR2 = HD2 + 4;   // 132 = 4 mod 32: the same bank spread as LSTR
constexpr int TILE2_FLOATS = BN * LSTR2;
constexpr int SPLIT_WAVES = 4;   // wavefronts that share the key tiles of a 32-query block in the kernels for small launches

struct MaskArgs {
    int kind;
    const float *dense;
    long long sb, sh, sq, sk;  // element strides of the dense mask, 0 on broadcast axes
    const int *lengths;
    // dense masks, optional: one class per 32-query x 32-key tile (0 = all zeros, 1 = all ones, 2 = anything else),
    // laid out [slab][q tile][k tile] with slab / tile strides 0 on the mask's broadcast axes
    // Bit 2 (value 4) of a class: every query row of the tile has a zero among the tile's 32 keys.  A 32-query block with
    // such a tile is "open": each of its rows keeps an unblocked key, so its all-ones tiles have weight exactly zero (like
    // the tiles a structured mask blocks) and may be skipped.
    const unsigned char *cls;
    int cls_sb, cls_sh, cls_sq, cls_sk;
};

// Classifies the 32 x 32 tiles of a dense mask so that the attention kernel only reads mask values where a tile is
// neither all zeros nor all ones.  One wavefront per tile; elements outside [Lq, Lk] count as matching.  Bit 2 of the
// class says that every row of the tile (inside Lq) has a zero in this tile.
__global__ __launch_bounds__(256) void sdpa_mask_classify(MaskArgs m, int MB, int MH, int nqt, int nkt, int Lq, int Lk,
                                                          long long total, unsigned char *cls) {
    const long long tile = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tile >= total) return;
    const int lane = threadIdx.x & 63;
    const int kt = (int)(tile % nkt);
    const int qt = (int)((tile / nkt) % nqt);
    const int hm = (int)((tile / nkt / nqt) % MH);
    const int bm = (int)(tile / nkt / nqt / MH);
    const int col = kt * 32 + (lane & 31);
    const int nrow = m.sq ? 32 : 1, ncol_ok = (m.sk ? col < Lk : (lane & 31) == 0);
    bool all0 = true, all1 = true, rows_open = true;
    const float *base = m.dense + bm * m.sb + hm * m.sh;
    // lanes 0..31 take row 2*it, lanes 32..63 row 2*it + 1; all 16 loads are issued before the first is looked at
    float x[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) {
        const int r = 2 * it + (lane >> 5);
        const int row = qt * 32 + r;
        x[it] = __builtin_nanf("");     // neither 0 nor 1: an element that does not exist
        if (r < nrow && ncol_ok && (!m.sq || row < Lq)) x[it] = base[row * m.sq + col * m.sk];
    }
#pragma unroll
    for (int it = 0; it < 16; ++it) {
        const int r = 2 * it + (lane >> 5);
        const bool exists = r < nrow && ncol_ok && (!m.sq || qt * 32 + r < Lq);
        const bool zero = exists && x[it] == 0.0f;
        if (exists) {
            all0 = all0 && zero;
            all1 = all1 && (x[it] == 1.0f);
        }
        const unsigned long long zeros = __ballot(zero);
        const bool row0 = 2 * it < nrow && (!m.sq || qt * 32 + 2 * it < Lq), row1 = 2 * it + 1 < nrow && (!m.sq || qt * 32 + 2 * it + 1 < Lq);
        if (row0 && (unsigned)zeros == 0u) rows_open = false;
        if (row1 && (unsigned)(zeros >> 32) == 0u) rows_open = false;
    }
    const int z = __all(all0), o = __all(all1);
    if (lane == 0) cls[tile] = (unsigned char)((z ? 0 : (o ? 1 : 2)) | (rows_open ? 4 : 0));
}

// Whether a 32-query block is known to be open (see MaskArgs): looked up in its first key tile and in the tile on the
// diagonal, which covers causal, padding and band masks.  cls_row: the block's row of tile classes.
__device__ __forceinline__ bool dense_block_open(const unsigned char *cls_row, const int cls_sk, const int qt, const int nkt) {
    if (!cls_row || !cls_sk) return false;
    return ((cls_row[0] | cls_row[min(qt, nkt - 1)]) & 4) != 0;
}

// Dense masks, tile skipping: how many leading keys a 32-query block has to visit.  Its key tiles from there on are all
// ones while the block is open, so their weights are exactly zero.  cls_row: the block's row of tile classes, qt: its
// index.  The same value in every lane.
__device__ __forceinline__ int dense_key_bound(const unsigned char *cls_row, const int cls_sk, const int qt, const int Lk) {
    const int nkt = (Lk + 31) >> 5;
    if (!dense_block_open(cls_row, cls_sk, qt, nkt)) return Lk;
    const int lane = threadIdx.x & 63;
    for (int base = (nkt - 1) & ~63; base >= 0; base -= 64) {
        const int t = base + lane;
        const bool need = t < nkt && (cls_row[t] & 3) != 1;
        const unsigned long long bal = __ballot(need);
        if (bal) return __builtin_amdgcn_readfirstlane(min(Lk, (base + 64 - (int)__builtin_clzll(bal)) * 32));
    }
    return min(Lk, 32);   // not reached: an open block has a tile that is not all ones
}

// Dense masks, tile skipping, seen from a 32-key block (key tile kt): the first 32-query tile it has to visit; the
// tiles before are all ones in open query blocks.  nqt when no tile needs a visit.  cls0: the (batch, head) slab's
// classes.
__device__ __forceinline__ int dense_query_begin(const MaskArgs &m, const unsigned char *cls0, const int kt, const int nqt, const int nkt) {
    if (!cls0 || !m.cls_sk) return 0;
    if (!m.cls_sq) return (dense_block_open(cls0, m.cls_sk, 0, nkt) && (cls0[kt] & 3) == 1) ? nqt : 0;   // one mask row for every query
    const int lane = threadIdx.x & 63;
    for (int base = 0; base < nqt; base += 64) {
        const int t = base + lane;
        bool need = false;
        if (t < nqt) {
            const unsigned char *row = cls0 + (long long)t * m.cls_sq;
            need = !(dense_block_open(row, m.cls_sk, t, nkt) && (row[kt] & 3) == 1);
        }
        const unsigned long long bal = __ballot(need);
        if (bal) return __builtin_amdgcn_readfirstlane(base + (int)__builtin_ctzll(bal));
    }
    return nqt;
}

// Dense masks, tile skipping, for a workgroup of BM / 32 wavefronts that owns the queries first .. first + BM - 1 (one
// 32-query block per wavefront; `sub` = this wavefront's block): kend = the keys the workgroup has to visit (the largest
// bound of its blocks), wkend = this wavefront's own bound, skip_ones = whether its all-ones tiles may be skipped.
__device__ __forceinline__ void dense_key_bounds(const MaskArgs &m, const int b, const int hh, const int first, const int sub,
                                                 const int Lq, const int Lk, int &kend, int &wkend, bool &skip_ones) {
    const unsigned char *cls0 = m.cls + (long long)b * m.cls_sb + hh * m.cls_sh;
    int kmax = 0;
#pragma unroll
    for (int w = 0; w < BM / 32; ++w) {
        const int blk = min(first + w * 32, Lq - 1) >> 5;
        const unsigned char *row = cls0 + (long long)blk * m.cls_sq;
        const int bound = dense_key_bound(row, m.cls_sk, blk, Lk);
        kmax = max(kmax, bound);
        if (w == sub) {
            wkend = bound;
            skip_ones = dense_block_open(row, m.cls_sk, blk, (Lk + 31) >> 5);
        }
    }
    kend = kmax;
}

// The same seen from a workgroup that owns the keys first .. first + BM - 1: t_begin = the first query tile the workgroup
// has to visit, wt_begin = this wavefront's own.  Returns the (batch, head) slab's tile classes for the per-tile test.
__device__ __forceinline__ const unsigned char *dense_query_bounds(const MaskArgs &m, const int b, const int hh, const int first,
                                                                   const int sub, const int nqt, const int Lk, int &t_begin,
                                                                   int &wt_begin) {
    const unsigned char *cls0 = m.cls + (long long)b * m.cls_sb + hh * m.cls_sh;
    int tmin = nqt;
#pragma unroll
    for (int w = 0; w < BM / 32; ++w) {
        const int kt = min(first + w * 32, Lk - 1) >> 5;
        const int begin = dense_query_begin(m, cls0, kt, nqt, (Lk + 31) >> 5);
        tmin = min(tmin, begin);
        if (w == sub) wt_begin = begin;
    }
    t_begin = tmin;
    return cls0;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// s_waitcnt vmcnt(0): every vector memory operation the wavefront has issued is complete.  Placed in front of a loop it
// also tells the compiler so: a load left pending on some path into the loop would otherwise make it wait, inside the
// loop, for everything issued up to the first use of that load's result - the loop's own prefetches included.
__device__ __forceinline__ void wait_vector_memory() { __builtin_amdgcn_s_waitcnt(0x0F70); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

// The value of lane l and the value of lane l ^ 32 in both lanes: v_permlane32_swap exchanges the upper half of its first
// operand with the lower half of its second, so (x, x) becomes (the lower half's values twice, the upper half's twice) - one
// instruction where a shuffle through the LDS crossbar costs an address computation, the round trip and its wait.
__device__ __forceinline__ void both_halves(const float x, float &lower, float &upper) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lower = __uint_as_float(sw[0]);
    upper = __uint_as_float(sw[1]);
}
// fmaxf(x, xor32(x)) and x + xor32(x) (the sum of two floats does not depend on their order: the same bits in both lanes)
// (the maximum is formed as max3(-inf, a, b): a two-operand maximum of values the compiler cannot prove canonical - register
// contents that come from an MFMA or a lane exchange - costs one quieting instruction per operand, the three-operand form none)
__device__ __forceinline__ float max_across_halves(const float x) {
    float a, b;
    both_halves(x, a, b);
    return fmaxf(fmaxf(-INFINITY, a), b);
}
// The largest of 16 scores, NaN ignored; -inf when all of them are NaN.
__device__ __forceinline__ float max_of_16(const f32x16 &s) {
    float t = fmaxf(fmaxf(-INFINITY, s[0]), s[1]);
#pragma unroll
    for (int r = 2; r < 16; r += 2) t = fmaxf(fmaxf(t, s[r]), s[r + 1]);
    return t;
}
__device__ __forceinline__ float sum_across_halves(const float x) {
    float a, b;
    both_halves(x, a, b);
    return a + b;
}

// Work item of this workgroup (see work_order.h).  Returns false for padding workgroups.
__device__ __forceinline__ bool work_item(const int nunits, const int total_blocks, const int lpt, int &bh, int &unit,
                                          const int snake = 0) {
    return dl4s_work_order::work_item_at((int)blockIdx.x, nunits, total_blocks, lpt, bh, unit, snake);
}

// The penalty of a dense mask value in the base-2 exponent domain, fl(fl(m * 1e9) * log2 e).  The reference subtracts
// fl(m * 1e9) from the natural-domain score (ScaledDotProductAttention.swift:55-57).  Where that is finite but its product
// with log2 e is not (|m * 1e9| above 2.36e38) the penalty stays at the largest finite float: a row blocked by such values
// then comes out uniform, as the reference's does, instead of NaN.  (Different penalties in that last sliver of the float
// range count as equal here.)
__device__ __forceinline__ float dense_penalty2(const float mval) {
    const float pen = __fmul_rn(mval, 1e9f);
    const float pen2 = __fmul_rn(pen, LOG2E);
    return (__builtin_isinf(pen2) && !__builtin_isinf(pen)) ? __builtin_copysignf(3.402823466e38f, pen) : pen2;
}

// A score blocked by a mask value of exactly 1 (every structured kind, and the masks TransformerUtil.swift:29-50 builds).
// The reference forms fl(s - 1e9) in the natural domain; floats next to 1e9 are 64 apart, so that is -1e9 + 64 n with
// n = s / 64 rounded to nearest-even: the score survives only as its bucket on a grid of 64.  Next to an unblocked key
// that is a weight of exactly zero whatever n is, but in a row with every key blocked the buckets decide: the keys of the
// highest bucket share the row (the next bucket weighs e^-64 of that, nothing in fp32); scores within (-32, 32) fall
// into one bucket and the row is uniform.  Subtracting 1e9 log2(e) from the base-2 score would sort the keys into other
// buckets (floats there are 128 apart, 88.7 in the natural domain), so the reference's bucket is formed from the score
// itself and carried on the base-2 grid: -PEN2 + 128 n, exact in fp32, with 2^-128 between buckets.  s2 is the score
// times log2(e); its last bits differ from the reference's, which matters only for a score within rounding of a bucket
// edge.  NaN and infinities pass through as they do through the subtraction.
constexpr float PEN2 = 1442695040.0f;   // fl(1e9 * log2(e)), a multiple of 128
__device__ __forceinline__ float blocked_score2(const float s2) {
    const float n = __builtin_rintf(__fmul_rn(s2, 0.69314718055994530942f / 64.0f));
    return __builtin_fmaf(n, 128.0f, -PEN2);
}
// s2 under a dense mask value: the bucket form for a value of exactly 1, the scaled penalty for any other
__device__ __forceinline__ float dense_masked2(const float s2, const float mval) {
    return mval == 1.0f ? blocked_score2(s2) : __fsub_rn(s2, dense_penalty2(mval));
}

// S^T = K . Q^T for one 32-key tile of one wavefront (lane = query qi = q0 + lane % 32, 16 of the 32 keys per lane:
// accumulator register r is key k0 + 8(r/4) + 4*half + r%4), then the mask, in registers.  Kb is the lane's K fragment
// base in LDS; qr the lane's Q fragment, already scaled by (1/T) log2(e): the scores are in the base-2 exponent domain.
// NJ: 128-bit reads per K row fragment (head dim / 8: 8 for the 64-wide kernels, 16 for the 128-wide one)
template <int KIND, int NJ = 8>
__device__ __forceinline__ f32x16 masked_scores(const float *Kb, const float (&qr)[4 * NJ], const int k0, const int q0, const int qi,
                                                const int half, const int Lk, const int len, const float *mrow,
                                                const long long msk, const int cls) {
    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);
    // ---- S^T = K . Q^T for one 32-key tile
    // (one dependent accumulation chain keeps the matrix pipe full; the first MFMA takes a literal zero)
    f32x16 s0;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const f32x4 a0 = *reinterpret_cast<const f32x4 *>(Kb + 4 * j);
        if (j == 0) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, qr[0], zero, 0, 0, 0);
        } else {
            s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, qr[4 * j + 0], s0, 0, 0, 0);
        }
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, qr[4 * j + 1], s0, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, qr[4 * j + 2], s0, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, qr[4 * j + 3], s0, 0, 0, 0);
    }

    // ---- mask, in registers.  Accumulator register r is key k0 + 8(r/4) + 4*half + r%4.
    if (DENSE) {
        if (cls == 1) {           // every element of the tile is 1: the penalty is a constant
#pragma unroll
            for (int r = 0; r < 16; ++r) s0[r] = blocked_score2(s0[r]);
        } else if (cls == 2) {    // mixed tile: read the mask values (class 0 = all zeros needs nothing)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kg = k0 + 8 * (r >> 2) + 4 * half + (r & 3);
                const int kc = kg < Lk ? kg : Lk - 1;
                s0[r] = dense_masked2(s0[r], mrow[kc * msk]);
            }
        }
    } else if ((CAUSAL && (k0 + BN - 1 > q0)) || (LENS && (k0 + BN > len))) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int kg = k0 + 8 * (r >> 2) + 4 * half + (r & 3);
            bool blocked = false;
            if (CAUSAL) blocked = blocked || (kg > qi);
            if (LENS) blocked = blocked || (kg >= len);
            if (blocked) s0[r] = blocked_score2(s0[r]);
        }
    }
    if (k0 + BN > Lk) {           // keys past the end of the tensor take no part
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int kg = k0 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (kg >= Lk) s0[r] = -INFINITY;
        }
    }
    return s0;
}

// Plain kernels (head dims other than 64).  The score of (query qi, key j) is the sequential dot product of the scaled
// query row with the key row, then the mask, every step rounded like the reference's generic engine.
constexpr int GEN_MAXD = 256;
__device__ __forceinline__ float plain_masked(float s, const MaskArgs &mask, const int b, const int hh, const int qi, const int j,
                                              const int len) {
    switch (mask.kind) {
        case DL4S_MASK_DENSE_F32: {
            const float mval = mask.dense[b * mask.sb + hh * mask.sh + qi * mask.sq + j * mask.sk];
            s = __fsub_rn(s, __fmul_rn(mval, 1e9f));
            break;
        }
        case DL4S_MASK_CAUSAL: if (j > qi) s = __fsub_rn(s, 1e9f); break;
        case DL4S_MASK_KEY_LENGTHS: if (j >= len) s = __fsub_rn(s, 1e9f); break;
        case DL4S_MASK_CAUSAL_OR_KEY_LENGTHS: if (j > qi || j >= len) s = __fsub_rn(s, 1e9f); break;
        default: break;
    }
    return s;
}
__device__ __forceinline__ float plain_score(const float *qs, const float *krow, const int dk, const MaskArgs &mask, const int b,
                                             const int hh, const int qi, const int j, const int len) {
    float s = 0.f;
    for (int c = 0; c < dk; ++c) s = __fadd_rn(s, __fmul_rn(qs[c], krow[c]));
    return plain_masked(s, mask, b, hh, qi, j, len);
}

// Validates a mask descriptor against [B,H,Lq,Lk], fills the kernels' view of it and, for dense masks on the MFMA
// kernels, launches the tile classifier (its result lives in the context's scratch block until the next call that uses it).
// Head dims the MFMA kernels do not take as they are (not a multiple of 4, key dim != value dim, q / k / v / out off the
// 16-byte grid), up to 256, on a problem large enough to pay for streaming copies: the kernels run on zero-padded copies.
// The forward call that leaves row statistics and the gradient call evaluate this on the same arguments, so both land
// on the same kind of kernel.
// Head dims above 128 up to 256 that the 192- and 256-wide forward kernels take as they are (the tensors 16-byte aligned
// besides): a multiple of 4 whose K/V rows of one (batch, head) pair stay inside the kernels' 32-bit byte offsets.
// Gradient launches of the 64-wide and narrower classes that count as small (one 32-row block per workgroup, the tiles along
// the other axis split over its wavefronts; the narrow classes run these on 64-wide padded tiles) for L rows along the axis
// the workgroups own.  64-wide: fewer 32-row blocks than four per CU.  (The bound was eight per CU: between four and eight
// the 128-row kernels are faster - B1 H16 L2048 d64 without a mask 490 -> 370 us, B8 H16 L256 99 -> 66 us, B3 H16 L1024 causal
// 263 -> 223 us.)  One case keeps the 32-row kernels up to eight per CU: blocks of different length, at most one 128-row
// workgroup per CU and 2048 rows or more - there the longest block sets the time of the 128-row launch (B1 H16 L2048
// causal 328 us against 369 us, B1 H8 L4096 584 against 717 us).  Narrow classes, whose own 128-row kernels do not pay for
// padding: fewer than two per CU, four with blocks of different length from 512 rows on (B3 H16 L1024 d32 causal 244 -> 130
// us, B1 H16 L1024 d32 without a mask 138 -> 115 us, B8 H16 L128 d16 27 -> 20 us; B1 H8 L2048 d32 causal stays at 161 us
// against 213 us on the 128-row kernels).
inline bool sdpa_bwd_small_launch(const dl4s_hip_ctx *ctx, int64_t B, int64_t H, int64_t L, bool uneven, bool narrow) {
    const long long blocks32 = (long long)B * H * ((L + 31) / 32), blocks128 = (long long)B * H * ((L + 127) / 128);
    if (narrow) return blocks32 < 2ll * ctx->cu_count || (uneven && L >= 512 && blocks32 < 4ll * ctx->cu_count);
    return blocks32 < 4ll * ctx->cu_count || (uneven && L >= 2048 && blocks128 <= ctx->cu_count && blocks32 < 8ll * ctx->cu_count);
}

// Shares of the key tiles per query block on a forward launch with fewer blocks than two per CU (the 96-wide and wider
// kernels): the even count w up to 8 with the least ceil(blocks * w / CUs) / w * (1 + per_share * w) - rounds of the CUs per
// share, times what a share costs in partial records and in the merge (measured: 2 % per share on the 96- and 128-wide
// kernels, 4 to 5 % on the 160- to 256-wide ones) - taking a larger count only for 5 % less.  256 blocks on 256 CUs: 2; 192: 4
// (three rounds of quarter shares against two rounds of halves: B1 H12 L2048 d128 without a mask 267 -> 219 us, causal
// 218 -> 160 us); 160: 8 / 4 (B1 H10 L2048 d128 266 -> 203 us, d256 593 -> 487 us); 128: 2; 96: 8; 64 and 48: 4.  Odd counts lose
// on every shape measured.  From the extents only: every mask kind of a problem adds in one order.
inline long long sdpa_key_shares(long long blocks, long long nkt, int cu, double per_share) {
    long long best = 2;
    double best_cost = 1e30;
    for (long long w = 2; w <= 8 && w <= nkt / 2; w += 2) {
        const double cost = (double)((blocks * w + cu - 1) / cu) / (double)w * (1.0 + per_share * (double)w);
        if (cost < 0.95 * best_cost) { best_cost = cost; best = w; }
    }
    return best;
}

inline bool sdpa_wide_route(int64_t H, int64_t Lk, int64_t d, int token_major) {
    return d > HD2 && d <= 256 && d % 4 == 0 && Lk * (token_major ? H : 1) * d * 4 < ((d == 160 || d == 192 || d == 256) ? (1ll << 31) : (1ll << 30));
}

inline bool sdpa_padded_route(bool mfma_as_is, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv) {
    const int64_t dmax = dk > dv ? dk : dv;
    return !mfma_as_is && dk > 0 && dv > 0 && dmax <= 256 && (double)B * H * Lq * Lk * (double)dmax >= (double)(1ll << 24);
}

// rows x d_src -> rows x d_dst: the common columns copied, the rest of a wider destination zeroed
__global__ void copy_rows_f32(const float *__restrict__ src, float *__restrict__ dst, long long rows, int d_src, int d_dst) {
    const long long n = rows * d_dst;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long r = i / d_dst;
        const int c = (int)(i - r * d_dst);
        dst[i] = c < d_src ? src[r * d_src + c] : 0.0f;
    }
}
inline void launch_copy_rows(dl4s_hip_ctx *ctx, const float *src, float *dst, long long rows, int64_t d_src, int64_t d_dst) {
    const long long n = rows * d_dst;
    const unsigned grid = (unsigned)std::min<long long>((n + 1023) / 1024, 65536);
    hipLaunchKernelGGL(copy_rows_f32, dim3(grid), dim3(256), 0, ctx->stream, src, dst, rows, (int)d_src, (int)d_dst);
}

// extra_bytes / extra: the caller's own share of the scratch block (partial results), placed behind the mask classes so
// that one sizing of the block covers both (growing it later would move the classes away from under m.cls).
inline int build_mask_args(dl4s_hip_ctx *ctx, const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                           bool classify, MaskArgs &m, size_t extra_bytes = 0, void **extra = nullptr) {
    m = MaskArgs{};
    if (extra) *extra = nullptr;
    m.kind = mask ? mask->kind : DL4S_MASK_NONE;
    switch (m.kind) {
        case DL4S_MASK_NONE: break;
        case DL4S_MASK_DENSE_F32: {
            DL4S_REQUIRE(mask->dense, DL4S_HIP_EINVALID_ARG, "sdpa: dense mask pointer is NULL");
            const int64_t full[4] = {B, H, Lq, Lk};
            long long stride = 1, st[4];
            for (int i = 3; i >= 0; --i) {
                DL4S_REQUIRE(mask->shape[i] == 1 || mask->shape[i] == full[i], DL4S_HIP_ESHAPE,
                             "sdpa: mask axis %d has size %lld, expected 1 or %lld", i, (long long)mask->shape[i],
                             (long long)full[i]);
                st[i] = mask->shape[i] == 1 ? 0 : stride;
                stride *= mask->shape[i];
            }
            m.dense = mask->dense;
            m.sb = st[0]; m.sh = st[1]; m.sq = st[2]; m.sk = st[3];
            break;
        }
        case DL4S_MASK_KEY_LENGTHS:
        case DL4S_MASK_CAUSAL_OR_KEY_LENGTHS:
            DL4S_REQUIRE(mask->lengths, DL4S_HIP_EINVALID_ARG, "sdpa: lengths pointer is NULL");
            m.lengths = mask->lengths;
            break;
        case DL4S_MASK_CAUSAL: break;
        default: return dl4s::set_error(DL4S_HIP_EINVALID_ARG, "sdpa: unknown mask kind %d", m.kind);
    }
    if (m.kind == DL4S_MASK_DENSE_F32 && classify) {
        const int64_t MB = m.sb ? B : 1, MH = m.sh ? H : 1;
        const int64_t nqt = m.sq ? (Lq + 31) / 32 : 1, nkt = m.sk ? (Lk + 31) / 32 : 1;
        const long long total = MB * MH * nqt * nkt;
        if (total < (1ll << 31)) {
            const unsigned char *cls = mask->classes;   // prepared by dl4s_hip_mask_classify_f32 for this mask and these extents
            if (!cls) {
                const size_t cls_bytes = ((size_t)total + 255) / 256 * 256;
                const int rc = dl4s::ensure_scratch(ctx, cls_bytes + extra_bytes);
                if (rc != DL4S_HIP_OK) return rc;
                unsigned char *own = static_cast<unsigned char *>(ctx->scratch);
                if (extra && extra_bytes) { *extra = own + cls_bytes; extra_bytes = 0; }
                hipLaunchKernelGGL(sdpa_mask_classify, dim3((unsigned)((total + 3) / 4)), dim3(256), 0, ctx->stream, m, (int)MB,
                                   (int)MH, (int)nqt, (int)nkt, (int)Lq, (int)Lk, total, own);
                const int st = dl4s::launch_status("sdpa_mask_classify");
                if (st != DL4S_HIP_OK) return st;
                cls = own;
            }
            m.cls = cls;
            m.cls_sk = m.sk ? 1 : 0;
            m.cls_sq = m.sq ? (int)nkt : 0;
            m.cls_sh = m.sh ? (int)(nqt * nkt) : 0;
            m.cls_sb = m.sb ? (int)(MH * nqt * nkt) : 0;
        }
    }
    if (extra && extra_bytes) {   // no classes in the block: the caller's share starts at its base
        const int rc = dl4s::ensure_scratch(ctx, extra_bytes);
        if (rc != DL4S_HIP_OK) return rc;
        *extra = ctx->scratch;
    }
    return DL4S_HIP_OK;
}

}  // namespace

// Gradients of the fused attention for gfx950 (64-wide tiles: head dims up to 64, padded with zero columns): given dout = d(loss)/d(out) of
//   out = softmax((q * rT) . k^T - mask * 1e9) . v
// compute dq, dk, dv.  With p = the softmax weights and D_i = sum_d dout[i][d] * out[i][d] (= sum_j dp_ij p_ij):
//   dv = p^T . dout,   dp = dout . v^T,   ds = p * (dp - D),   dq = (ds . k) * rT,   dk = ds^T . (q * rT)
// which is what the reference's reverse-mode closures compute for the forward graph of
// NN/Models/Transformer/ScaledDotProductAttention.swift:43-64 (Tensor/Operators/Matrix.swift:139-174,
// Binary.swift:235-300, Unary.swift:33-55, Reduce.swift:35-62), up to the order of the floating-point operations.
//
// The weights are not stored by the forward pass: they are recomputed tile by tile as p = 2^(s - m) / l, where s is the
// base-2 score exactly as the forward kernel forms it and (m, 1/l) the two row statistics that
// dl4s_hip_sdpa_fwd_stats_f32 leaves per row (the forward pass's reference maximum and the reciprocal of its row sum).
// Two kernels, both deterministic (no atomics):
//   sdpa_bwd_dq_f32_d64    a wavefront owns 32 queries and walks the keys like the forward kernel
//                          (S^T, dP^T in the accumulator layout lane = query; dQ^T += K^T . dS^T)
//   sdpa_bwd_dkv_f32_d64   a wavefront owns 32 keys and walks the queries (S, dP with lane = key;
//                          dV^T += dO^T . P, dK^T += Q^T . dS)
// Large launches form the scores and dP once: the dK/dV kernel also stores its dS tiles to a scratch tensor
// [batch*head][key][query] (a lane of its accumulator layout holds four consecutive queries of one key: 128-bit stores)
// and sdpa_bwd_dq_from_ds_f32_d64 only contracts them with K (a lane of ITS accumulator layout is one query and 16 keys:
// 16 coalesced 32-bit loads) - five products issued for five, and the scratch tensor is written once and read once.
// The two-kernel form above, which forms the scores and dP in both kernels (seven products for five), stays as the route
// for launches whose scratch tensor would be too large to allocate.
// All five products of each run on v_mfma_f32_32x32x2_f32 with the operand layouts of the forward kernel.  Small launches
// run the _split_ forms of the two (one 32-row block per workgroup, its tiles split over the four wavefronts); head dims
// above 64 up to 128 run the 128-wide forms in sdpa_backward_d128.h; head dims the MFMA kernels do not take run the
// plain kernels at the end of the file.
#include "sdpa_common.h"
#include "sdpa_backward_d128.h"
#include "sdpa_backward_narrow.h"

#include <cstdlib>

namespace {

constexpr float LN2 = 0.69314718055994530942f;
// Upper bound of the dS scratch tensor of the large-launch route (B * H * Lk * Lq floats): beyond it the self-contained
// kernels run.  B8 H16 L2048 needs 2 GiB.
constexpr long long DS_SCRATCH_MAX_BYTES = 24ll << 30;
// The environment variable DL4S_HIP_BWD_SCRATCH_MAX_BYTES lowers (or raises) the bound for a process, e.g. to keep the
// gradient call's footprint small; 0 always takes the self-contained kernels.
inline long long ds_scratch_max_bytes() {
    const char *e = getenv("DL4S_HIP_BWD_SCRATCH_MAX_BYTES");
    if (!e || !*e) return DS_SCRATCH_MAX_BYTES;
    char *end = nullptr;
    const long long v = strtoll(e, &end, 10);
    return (end && *end == 0 && v >= 0) ? v : DS_SCRATCH_MAX_BYTES;
}

// D[b,h,i] = sum_d dout[i][d] * out[i][d]; 16 lanes per row, four rows per wavefront
__global__ __launch_bounds__(256) void sdpa_bwd_rowdot(const float *__restrict__ out, const float *__restrict__ dout,
                                                       float *__restrict__ D, int H, int Lq, long long rows, int token_major, int hd) {
    const long long r = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int c = (threadIdx.x & 15) * 4;
    float acc = 0.f;
    if (r < rows && c < hd) {
        const long long bh = r / Lq, qi = r % Lq;
        const long long off = token_major ? (((bh / H) * Lq + qi) * H + bh % H) * hd : r * hd;
        const f32x4 a = *reinterpret_cast<const f32x4 *>(out + off + c);
        const f32x4 g = *reinterpret_cast<const f32x4 *>(dout + off + c);
        acc = a.x * g.x + a.y * g.y + a.z * g.z + a.w * g.w;
    }
    acc += __shfl_xor(acc, 8, 64);
    acc += __shfl_xor(acc, 4, 64);
    acc += __shfl_xor(acc, 2, 64);
    acc += __shfl_xor(acc, 1, 64);
    if (r < rows && (threadIdx.x & 15) == 0) D[r] = acc;
}

// 32 x 32 product tile in the transposed accumulator layout of the forward kernel: A rows from LDS (lane reads row
// lane % 32, 128-bit reads at columns half*32 + 4j), B from the lane's 32 registers.
__device__ __forceinline__ f32x16 tile_product(const float *Ab, const float (&br)[32]) {
    f32x16 acc;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
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

// acc0/acc1 (rows d = 2m, 2m+1; column = the lane's query or key) += A^T . B where A is a [32][64] LDS tile read
// through 64-bit loads (row 8(r/4) + r%4 + 4*half, columns 2*lane%32 + {0,1}: At already points there) and B the
// accumulator-layout tile b.
__device__ __forceinline__ void tile_accumulate_t(const float *At, const f32x16 &b, f32x16 &acc0, f32x16 &acc1) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const f32x2 a = *reinterpret_cast<const f32x2 *>(At + (8 * (r >> 2) + (r & 3)) * LSTR);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b[r], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b[r], acc1, 0, 0, 0);
    }
}

// Stores the transposed accumulators (register r of acc0/acc1 is d = 2*(8(r/4) + 4*half + r%4) + {0,1}) of the lane's
// row to p[row][0..63], scaled; p points at the lane's first column, of which ncols (a multiple of 4, may be <= 0) exist.
__device__ __forceinline__ void store_row_t(float *p, const f32x16 &acc0, const f32x16 &acc1, const float scale, const int ncols) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        f32x4 a, c;
        a.x = acc0[4 * g + 0] * scale; a.y = acc1[4 * g + 0] * scale;
        a.z = acc0[4 * g + 1] * scale; a.w = acc1[4 * g + 1] * scale;
        c.x = acc0[4 * g + 2] * scale; c.y = acc1[4 * g + 2] * scale;
        c.z = acc0[4 * g + 3] * scale; c.w = acc1[4 * g + 3] * scale;
        if (16 * g < ncols) *reinterpret_cast<f32x4 *>(p + 16 * g) = a;
        if (16 * g + 4 < ncols) *reinterpret_cast<f32x4 *>(p + 16 * g + 4) = c;
    }
}

// ------------------------------------------------------------------------------------------------ dQ
template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dq_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                               const float *__restrict__ v, const float *__restrict__ dout,
                                                               const float *__restrict__ stats, const float *__restrict__ D,
                                                               float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                               MaskArgs mask, int strict, int nqb, int total_blocks, int lpt,
                                                               int token_major, int hd) {
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                     // [2][BN][LSTR]
    float *Vs = lds + 2 * TILE_FLOATS;   // [2][BN][LSTR]
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
    const int rs = token_major ? H * hd : hd;   // hd: the tensors' head dim, a multiple of 4 up to 64; tiles are zero beyond it
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    // the same tiles as the forward pass visits (skipped tiles have weight exactly 0, hence gradient 0)
    int kend = Lk, wkend = Lk;
    bool skip_ones = false;   // dense masks: this wavefront's all-ones tiles have weight exactly zero
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { kend = min(kend, qb * BM + BM); wkend = min(wkend, q0 + 32); }
        if (LENS) { kend = min(kend, len); wkend = min(wkend, len); }
        if (DENSE && mask.cls) dense_key_bounds(mask, b, hh, qb * BM, wave, Lq, Lk, kend, wkend, skip_ones);
    }
    const int ntiles = (kend + BN - 1) / BN;

    float qr[32], gr[32];   // lane's Q fragment (scaled as in the forward pass) and dout fragment
    {
        const float *qp = q + q_base + (long long)qic * rs + half * 32;
        const float *gp = dout + q_base + (long long)qic * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) {
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

    const int ld_row = tid >> 4, ld_col = (tid & 15) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off0 = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;   // beyond hd: outside the descriptor, zeros
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
            const int off = buf * TILE_FLOATS + (i * 16 + ld_row) * LSTR + ld_col;
            *reinterpret_cast<f32x4 *>(Ks + off) = kst[i];
            *reinterpret_cast<f32x4 *>(Vs + off) = vst[i];
        }
    };

    f32x16 a0, a1;   // dQ^T rows d = 2m + {0,1}
#pragma unroll
    for (int i = 0; i < 16; ++i) { a0[i] = 0.f; a1[i] = 0.f; }

    if (ntiles > 0) { load_tile(0); store_tile(0); }
    __syncthreads();

    const int row_lds = ln * LSTR + half * 32;        // row-fragment base (S^T and dP^T products)
    const int col_lds = (4 * half) * LSTR + 2 * ln;   // transposed-fragment base (dQ^T product)
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
            f32x16 p = masked_scores<KIND>(Ks + buf * TILE_FLOATS + row_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = fast_exp2(p[r] - m_i) * rl_i;                   // the forward pass's weights
            const f32x16 dp = tile_product(Vs + buf * TILE_FLOATS + row_lds, gr);               // dP^T = V . dout^T
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = p[r] * (dp[r] - D_i);                           // dS^T
            tile_accumulate_t(Ks + buf * TILE_FLOATS + col_lds, p, a0, a1);                     // dQ^T += K^T . dS^T
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (qi < Lq) store_row_t(dq + q_base + (long long)qi * rs + 8 * half, a0, a1, rT, hd - 8 * half);
}

// ------------------------------------------------------------------------------------------------ dK, dV
// WRITE_DS: every visited 32 x 32 tile of dS is also stored to ds [batch*head][Lkp][Lqp] (Lkp, Lqp = the key and query
// counts rounded up to 32), for sdpa_bwd_dq_from_ds_f32_d64.  Rows of keys at or beyond Lk are stored as zeros.
template <int KIND, bool WRITE_DS = false>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dkv_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                const float *__restrict__ v, const float *__restrict__ dout,
                                                                const float *__restrict__ stats, const float *__restrict__ D,
                                                                float *__restrict__ dk, float *__restrict__ dv, int H, int Lq,
                                                                int Lk, float rT, MaskArgs mask, int strict, int nkb,
                                                                int total_blocks, int lpt, int token_major, int hd,
                                                                float *__restrict__ ds = nullptr) {
    extern __shared__ __align__(16) float lds[];
    float *Qs = lds;                       // [2][BN][LSTR]  q * rT * log2(e)
    float *Gs = lds + 2 * TILE_FLOATS;     // [2][BN][LSTR]  dout
    float *Ss = lds + 4 * TILE_FLOATS;     // per query tile: [2][32] reference maxima, [2][32] 1 / row sums, [2][32] D
    int bh, unit;
    if (!work_item(nkb, total_blocks, lpt & 1, bh, unit, lpt >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, ln = lane & 31;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int kb = unit;                 // under a causal mask the first key block meets the most queries: longest first
    const int kw0 = kb * BM + wave * 32; // first key of this wavefront
    const int key = kw0 + ln;
    const int keyc = key < Lk ? key : Lk - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;   // hd: the tensors' head dim, a multiple of 4 up to 64; tiles are zero beyond it
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    // Query tiles this workgroup / wavefront has to visit: under a causal mask only queries at or after its first key;
    // keys at or beyond the valid length have weight 0 everywhere.  Same exactness conditions as the forward pass.
    const int nqt = (Lq + 31) / 32;
    int t_begin = 0, wt_begin = 0;
    bool wave_active = true;
    const unsigned char *skip_cls0 = nullptr;   // dense masks with tile skipping: the (batch, head) slab's tile classes
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) { t_begin = (kb * BM) / 32; wt_begin = kw0 / 32; }
        if (LENS) {
            if (kb * BM >= len) t_begin = nqt;
            if (kw0 >= len) wave_active = false;
        }
        if (DENSE && mask.cls) skip_cls0 = dense_query_bounds(mask, b, hh, kb * BM, wave, nqt, Lk, t_begin, wt_begin);
    }

    float kr[32], vr[32];   // the lane's key and value rows (columns half*32 ..)
    {
        const float *kp = k + kv_base + (long long)keyc * rs + half * 32;
        const float *vp = v + kv_base + (long long)keyc * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) {
                a = *reinterpret_cast<const f32x4 *>(kp + 4 * j);
                c = *reinterpret_cast<const f32x4 *>(vp + 4 * j);
            }
            kr[4 * j + 0] = a.x; kr[4 * j + 1] = a.y; kr[4 * j + 2] = a.z; kr[4 * j + 3] = a.w;
            vr[4 * j + 0] = c.x; vr[4 * j + 1] = c.y; vr[4 * j + 2] = c.z; vr[4 * j + 3] = c.w;
        }
    }

    // staging of one query tile: q (scaled when it is written to LDS), dout, and the tile's row statistics.  Rows at or
    // beyond Lq read as zeros; their reciprocal row sum is taken as 0, which makes their weights 0.
    const int ld_row = tid >> 4, ld_col = (tid & 15) * 4;
    const int q_bytes = (int)(((long long)(Lq - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t qrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(q + q_base), 0, q_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t grsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(dout + q_base), 0, q_bytes, 0x00020000);
    const unsigned ld_off0 = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;   // beyond hd: outside the descriptor, zeros
    const unsigned ld_off1 = ld_off0 + 16u * rs * 4u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 qst[2], gst[2];
    float sst = 0.f;
    auto load_tile = [&](int t) {
        const int o0 = (int)(ld_off0 + t * tile_bytes), o1 = (int)(ld_off1 + t * tile_bytes);
        qst[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o0, 0, 0));
        gst[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o0, 0, 0));
        qst[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o1, 0, 0));
        gst[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o1, 0, 0));
        if (tid < 96) {      // threads 0..31: reference maximum, 32..63: 1 / row sum, 64..95: D
            const int row = t * 32 + (tid & 31);
            const long long at = (long long)bh * Lq + row;
            sst = 0.f;
            if (row < Lq) sst = tid < 32 ? stats[2 * at] : (tid < 64 ? stats[2 * at + 1] : D[at]);
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int off = buf * TILE_FLOATS + (i * 16 + ld_row) * LSTR + ld_col;
            f32x4 s;
            s.x = (qst[i].x * rT) * LOG2E; s.y = (qst[i].y * rT) * LOG2E;
            s.z = (qst[i].z * rT) * LOG2E; s.w = (qst[i].w * rT) * LOG2E;
            *reinterpret_cast<f32x4 *>(Qs + off) = s;
            *reinterpret_cast<f32x4 *>(Gs + off) = gst[i];
        }
        if (tid < 96) Ss[(tid >> 5) * 64 + buf * 32 + (tid & 31)] = sst;
    };

    f32x16 k0a, k1a, v0a, v1a;   // dK^T and dV^T rows d = 2m + {0,1}
#pragma unroll
    for (int i = 0; i < 16; ++i) { k0a[i] = 0.f; k1a[i] = 0.f; v0a[i] = 0.f; v1a[i] = 0.f; }

    if (t_begin < nqt) { load_tile(t_begin); store_tile(0); }
    __syncthreads();

    const int row_lds = ln * LSTR + half * 32;
    const int col_lds = (4 * half) * LSTR + 2 * ln;
    const unsigned char *cls_col = nullptr;
    if (DENSE && mask.cls) cls_col = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(kw0, Lk - 1) >> 5) * mask.cls_sk;
    const float *mcol = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + keyc * mask.sk : nullptr;
    // dS slab of this (batch, head) pair: row = key, column = query; the lane stores four consecutive queries of its key
    const int Lqp = (Lq + 31) & ~31, Lkp = (Lk + 31) & ~31;
    __amdgpu_buffer_rsrc_t dsrsrc;
    unsigned ds_voff = 0;
    if (WRITE_DS) {
        dsrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(ds + (long long)bh * Lkp * Lqp), 0, (int)((long long)Lk * Lqp * 4), 0x00020000);
        ds_voff = ((unsigned)key * (unsigned)Lqp + 4u * half) * 4u;
    }

    // Tiles before the wavefront's first one (causal masks), and every tile of a wavefront without a valid key, are only
    // staged.  The loop over the tiles the wavefront computes on is kept free of that test: with the dS stores on every
    // path through its body the compiler can tell that they follow the next tile's loads, and the wait before the LDS
    // writes covers the loads alone instead of the stores' round trip to memory.
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
            // S[query, key] in the base-2 domain: rows = the tile's queries 8(r/4) + 4*half + r%4, column = the lane's key
            f32x16 p = tile_product(Qs + buf * TILE_FLOATS + row_lds, kr);
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
            tile_accumulate_t(Gs + buf * TILE_FLOATS + col_lds, p, v0a, v1a);                   // dV^T += dout^T . P
            const f32x16 dp = tile_product(Gs + buf * TILE_FLOATS + row_lds, vr);               // dP = dout . V^T
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
            tile_accumulate_t(Qs + buf * TILE_FLOATS + col_lds, p, k0a, k1a);                   // dK^T += Q~^T . dS
        }
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (key < Lk) {
        store_row_t(dv + kv_base + (long long)key * rs + 8 * half, v0a, v1a, 1.0f, hd - 8 * half);
        store_row_t(dk + kv_base + (long long)key * rs + 8 * half, k0a, k1a, LN2, hd - 8 * half);   // Q~ carries log2(e): dK = Q~^T dS ln 2
    }
}

// ------------------------------------------------------------------------------------------------ dQ from stored dS
// dQ = (dS . K) * rT with dS read from the scratch tensor sdpa_bwd_dkv_f32_d64<KIND, true> wrote: a wavefront owns 32
// queries and walks the key tiles the forward pass visits (the dK/dV kernel visits - and writes - exactly those: both
// follow the forward pass's rule, tile by tile).  Per tile and wavefront: 16 coalesced 32-bit loads (lane = query, the
// 16 keys of the accumulator layout) and 32 MFMAs against the K tile in LDS; no scores, no exponentials, no mask values.
template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dq_from_ds_f32_d64(const float *__restrict__ k, const float *__restrict__ ds,
                                                                       float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                                       MaskArgs mask, int strict, int nqb, int total_blocks, int lpt,
                                                                       int token_major, int hd) {
    extern __shared__ __align__(16) float lds[];
    float *Ks = lds;                     // [2][BN][LSTR]
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

    const int ld_row = tid >> 4, ld_col = (tid & 15) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off0 = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned ld_off1 = ld_off0 + 16u * rs * 4u;
    const unsigned tile_bytes = (unsigned)BN * rs * 4u;
    f32x4 kst[2];
    auto load_tile = [&](int t) {
        kst[0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, (int)(ld_off0 + t * tile_bytes), 0, 0));
        kst[1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(krsrc, (int)(ld_off1 + t * tile_bytes), 0, 0));
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) *reinterpret_cast<f32x4 *>(Ks + buf * TILE_FLOATS + (i * 16 + ld_row) * LSTR + ld_col) = kst[i];
    };

    // dS slab of the pair, [key][query]: register r of the lane is key k0 + 8(r/4) + 4*half + r%4, query qi
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

    f32x16 a0, a1;   // dQ^T rows d = 2m + {0,1}
#pragma unroll
    for (int i = 0; i < 16; ++i) { a0[i] = 0.f; a1[i] = 0.f; dsn[i] = 0.f; }

    if (ntiles > 0) {
        load_tile(0);
        store_tile(0);
        if (visited(0)) load_ds(0);
    }
    __syncthreads();
    const int col_lds = (4 * half) * LSTR + 2 * ln;
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
        if (now) tile_accumulate_t(Ks + buf * TILE_FLOATS + col_lds, p, a0, a1);               // dQ^T += K^T . dS^T
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    if (qi < Lq) store_row_t(dq + q_base + (long long)qi * rs + 8 * half, a0, a1, rT, hd - 8 * half);
}

// ------------------------------------------------------------------------------------------------ small launches
// Too few 32-row blocks to give every SIMD about two wavefronts (the forward pass's rule): a workgroup is ONE 32-query
// block (dQ) or ONE 32-key block (dK, dV) whose tiles along the other axis are dealt round-robin to its 4 wavefronts.
// Each wavefront stages its own tiles in its own LDS region (the LDS operations of one wavefront execute in order, so
// the loop has no workgroup barrier); the four partial gradient blocks are added in wavefront order at the end.
template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dq_split_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                     const float *__restrict__ v, const float *__restrict__ dout,
                                                                     const float *__restrict__ stats, const float *__restrict__ D,
                                                                     float *__restrict__ dq, int H, int Lq, int Lk, float rT,
                                                                     MaskArgs mask, int strict, int nqb, int total_blocks, int order,
                                                                     int token_major, int hd) {
    extern __shared__ __align__(16) float lds[];
    // (the arguments in one trip to memory instead of several, one behind the other, before the first row is requested)
    asm volatile("" ::"s"(q), "s"(k), "s"(v), "s"(dout), "s"(stats), "s"(D), "s"(dq), "s"(H), "s"(Lq), "s"(Lk), "s"(rT), "s"(strict),
                 "s"(nqb), "s"(total_blocks), "s"(order), "s"(token_major), "s"(hd));
    int bh, unit;
    if (!work_item(nqb, total_blocks, order & 1, bh, unit, order >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, ln = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float *Ks = lds + wave * 2 * TILE_FLOATS, *Vs = Ks + TILE_FLOATS;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int qb = nqb - 1 - unit;   // longest rows first
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

    float qr[32], gr[32];
    {
        const float *qp = q + q_base + (long long)qic * rs + half * 32;
        const float *gp = dout + q_base + (long long)qic * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f}, g = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) {
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

    // the wavefront stages its own tiles: lane covers rows (i*4 + lane/16), 4 floats at column (lane%16)*4
    const int ld_row = lane >> 4, ld_col = (lane & 15) * 4;
    const int kv_bytes = (int)(((long long)(Lk - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(k + kv_base), 0, kv_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(v + kv_base), 0, kv_bytes, 0x00020000);
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned row4_bytes = 4u * rs * 4u, tile_bytes = (unsigned)BN * rs * 4u;
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

    f32x16 a0, a1;
#pragma unroll
    for (int i = 0; i < 16; ++i) { a0[i] = 0.f; a1[i] = 0.f; }
    const int row_lds = ln * LSTR + half * 32;
    const int col_lds = (4 * half) * LSTR + 2 * ln;
    const float *mrow = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + qic * mask.sq : nullptr;
    const unsigned char *cls_row = nullptr;
    if (DENSE && mask.cls) cls_row = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(q0, Lq - 1) >> 5) * mask.cls_sq;

    if (wave < ntiles) { load_tile(wave); store_tile(); }
    for (int t = wave; t < ntiles; t += 4) {
        const bool more = (t + 4 < ntiles);
        if (more) load_tile(t + 4);
        const int k0 = t * BN;
        int cls = 2;
        if (DENSE && cls_row) cls = cls_row[t * mask.cls_sk] & 3;
        if (!(DENSE && skip_ones && cls == 1)) {
            f32x16 p = masked_scores<KIND>(Ks + row_lds, qr, k0, q0, qi, half, Lk, len, mrow, mask.sk, cls);
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = fast_exp2(p[r] - m_i) * rl_i;
            const f32x16 dp = tile_product(Vs + row_lds, gr);
#pragma unroll
            for (int r = 0; r < 16; ++r) p[r] = p[r] * (dp[r] - D_i);
            tile_accumulate_t(Ks + col_lds, p, a0, a1);
        }
        if (more) store_tile();
    }

    // Add the four partial dQ^T blocks in wavefront order.  Every wavefront leaves its block in its own LDS region (its
    // tiles are dead, and the LDS operations of one wavefront execute in order: no barrier before the writes); behind the
    // barrier wavefront w adds the accumulator registers 4w .. 4w + 3 of the four blocks (16 of the 64 columns) and
    // stores them.
    float *mine = lds + wave * 2 * TILE_FLOATS;   // [32][64]: row 2r = a0[r], row 2r + 1 = a1[r]
#pragma unroll
    for (int r = 0; r < 16; ++r) { mine[(2 * r) * 64 + lane] = a0[r]; mine[(2 * r + 1) * 64 + lane] = a1[r]; }
    __syncthreads();
    float sum[8];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const float *rows = lds + x * 2 * TILE_FLOATS + (8 * wave) * 64 + lane;
#pragma unroll
        for (int i = 0; i < 8; ++i) sum[i] = x == 0 ? rows[i * 64] : sum[i] + rows[i * 64];
    }
    if (qi < Lq) {
        float *p = dq + q_base + (long long)qi * rs + 8 * half + 16 * wave;
        const int ncols = hd - 8 * half - 16 * wave;
        const f32x4 lo = {sum[0] * rT, sum[1] * rT, sum[2] * rT, sum[3] * rT}, hi = {sum[4] * rT, sum[5] * rT, sum[6] * rT, sum[7] * rT};
        if (0 < ncols) *reinterpret_cast<f32x4 *>(p) = lo;
        if (4 < ncols) *reinterpret_cast<f32x4 *>(p + 4) = hi;
    }
}

template <int KIND>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dkv_split_f32_d64(const float *__restrict__ q, const float *__restrict__ k,
                                                                      const float *__restrict__ v, const float *__restrict__ dout,
                                                                      const float *__restrict__ stats, const float *__restrict__ D,
                                                                      float *__restrict__ dk, float *__restrict__ dv, int H, int Lq,
                                                                      int Lk, float rT, MaskArgs mask, int strict, int nkb,
                                                                      int total_blocks, int order, int token_major, int hd) {
    extern __shared__ __align__(16) float lds[];
    // (the arguments in one trip to memory instead of several, one behind the other, before the first row is requested)
    asm volatile("" ::"s"(q), "s"(k), "s"(v), "s"(dout), "s"(stats), "s"(D), "s"(dk), "s"(dv), "s"(H), "s"(Lq), "s"(Lk), "s"(rT),
                 "s"(strict), "s"(nkb), "s"(total_blocks), "s"(order), "s"(token_major), "s"(hd));
    int bh, unit;
    if (!work_item(nkb, total_blocks, order & 1, bh, unit, order >> 1)) return;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, ln = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int REGION = 2 * TILE_FLOATS + 96;   // q tile, dout tile, the tile's (m, 1/l, D)
    float *Qs = lds + wave * REGION, *Gs = Qs + TILE_FLOATS, *Ss = Gs + TILE_FLOATS;

    constexpr bool CAUSAL = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool LENS = (KIND == DL4S_MASK_KEY_LENGTHS || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    constexpr bool DENSE = (KIND == DL4S_MASK_DENSE_F32);

    const int kb = unit;                 // under a causal mask the first key block meets the most queries
    const int kw0 = kb * 32;
    const int key = kw0 + ln;
    const int keyc = key < Lk ? key : Lk - 1;
    int len = Lk;
    if (LENS) len = mask.lengths[b];
    const int rs = token_major ? H * hd : hd;
    const long long q_base = token_major ? ((long long)b * Lq * H + hh) * hd : (long long)bh * Lq * hd;
    const long long kv_base = token_major ? ((long long)b * Lk * H + hh) * hd : (long long)bh * Lk * hd;

    const int nqt = (Lq + 31) / 32;
    int t_begin = 0;
    const unsigned char *skip_cls0 = nullptr;
    if (!strict && !(LENS && len <= 0)) {
        if (CAUSAL) t_begin = kw0 / 32;
        if (LENS && kw0 >= len) t_begin = nqt;
        if (DENSE && mask.cls) {
            skip_cls0 = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh;
            t_begin = dense_query_begin(mask, skip_cls0, min(kw0, Lk - 1) >> 5, nqt, (Lk + 31) >> 5);
        }
    }

    float kr[32], vr[32];
    {
        const float *kp = k + kv_base + (long long)keyc * rs + half * 32;
        const float *vp = v + kv_base + (long long)keyc * rs + half * 32;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f}, c = {0.f, 0.f, 0.f, 0.f};
            if (half * 32 + 4 * j < hd) {
                a = *reinterpret_cast<const f32x4 *>(kp + 4 * j);
                c = *reinterpret_cast<const f32x4 *>(vp + 4 * j);
            }
            kr[4 * j + 0] = a.x; kr[4 * j + 1] = a.y; kr[4 * j + 2] = a.z; kr[4 * j + 3] = a.w;
            vr[4 * j + 0] = c.x; vr[4 * j + 1] = c.y; vr[4 * j + 2] = c.z; vr[4 * j + 3] = c.w;
        }
    }

    const int ld_row = lane >> 4, ld_col = (lane & 15) * 4;
    const int q_bytes = (int)(((long long)(Lq - 1) * rs + hd) * 4);
    const __amdgpu_buffer_rsrc_t qrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(q + q_base), 0, q_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t grsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(dout + q_base), 0, q_bytes, 0x00020000);
    const unsigned ld_off = ld_col < hd ? (unsigned)(ld_row * rs + ld_col) * 4u : 0x80000000u;
    const unsigned row4_bytes = 4u * rs * 4u, tile_bytes = (unsigned)BN * rs * 4u;
    // a query tile in two halves of 16 rows, so that the staging registers stay few
    f32x4 qst[4], gst[4];
    float s_ml = 0.f, s_d = 0.f;   // lanes 0..31: reference maximum and D of the tile's query ln; lanes 32..63: 1 / row sum
    auto load_half = [&](int t, int h) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int o = (int)(ld_off + t * tile_bytes + (4 * h + i) * row4_bytes);
            qst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(qrsrc, o, 0, 0));
            gst[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(grsrc, o, 0, 0));
        }
        if (h == 0) {
            const int row = t * 32 + ln;
            const long long at = (long long)bh * Lq + row;
            s_ml = 0.f; s_d = 0.f;
            if (row < Lq) {
                s_ml = stats[2 * at + half];
                if (half == 0) s_d = D[at];
            }
        }
    };
    auto store_half = [&](int h) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int off = ((4 * h + i) * 4 + ld_row) * LSTR + ld_col;
            f32x4 sc;
            sc.x = (qst[i].x * rT) * LOG2E; sc.y = (qst[i].y * rT) * LOG2E;
            sc.z = (qst[i].z * rT) * LOG2E; sc.w = (qst[i].w * rT) * LOG2E;
            *reinterpret_cast<f32x4 *>(Qs + off) = sc;
            *reinterpret_cast<f32x4 *>(Gs + off) = gst[i];
        }
        if (h == 0) {
            Ss[half * 32 + ln] = s_ml;           // [0..31] m, [32..63] 1 / l
            if (half == 0) Ss[64 + ln] = s_d;    // [64..95] D
        }
    };

    f32x16 k0a, k1a, v0a, v1a;
#pragma unroll
    for (int i = 0; i < 16; ++i) { k0a[i] = 0.f; k1a[i] = 0.f; v0a[i] = 0.f; v1a[i] = 0.f; }
    const int row_lds = ln * LSTR + half * 32;
    const int col_lds = (4 * half) * LSTR + 2 * ln;
    const unsigned char *cls_col = nullptr;
    if (DENSE && mask.cls) cls_col = mask.cls + (long long)b * mask.cls_sb + hh * mask.cls_sh + (long long)(min(kw0, Lk - 1) >> 5) * mask.cls_sk;
    const float *mcol = DENSE ? mask.dense + b * mask.sb + hh * mask.sh + keyc * mask.sk : nullptr;

    // query tile t belongs to wavefront t % 4 whatever t_begin is, so that skipping tiles does not change which partial
    // sum a tile goes into (the same bits with and without skipping)
    for (int t = t_begin + ((wave - t_begin) & 3); t < nqt; t += 4) {
        load_half(t, 0);
        store_half(0);
        load_half(t, 1);
        store_half(1);
        const int qt0 = t * 32;
        int cls = 2;
        if (DENSE && cls_col) cls = cls_col[(long long)t * mask.cls_sq] & 3;
        if (DENSE && cls == 1 && skip_cls0 && dense_block_open(skip_cls0 + (long long)t * mask.cls_sq, mask.cls_sk, t, (Lk + 31) >> 5)) continue;
        f32x16 p = tile_product(Qs + row_lds, kr);
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
        const float *st = Ss + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 m4 = *reinterpret_cast<const f32x4 *>(st + 8 * g);
            const f32x4 r4 = *reinterpret_cast<const f32x4 *>(st + 32 + 8 * g);
            p[4 * g + 0] = fast_exp2(p[4 * g + 0] - m4.x) * r4.x;
            p[4 * g + 1] = fast_exp2(p[4 * g + 1] - m4.y) * r4.y;
            p[4 * g + 2] = fast_exp2(p[4 * g + 2] - m4.z) * r4.z;
            p[4 * g + 3] = fast_exp2(p[4 * g + 3] - m4.w) * r4.w;
        }
        tile_accumulate_t(Gs + col_lds, p, v0a, v1a);
        const f32x16 dp = tile_product(Gs + row_lds, vr);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f32x4 d4 = *reinterpret_cast<const f32x4 *>(st + 64 + 8 * g);
            p[4 * g + 0] = p[4 * g + 0] * (dp[4 * g + 0] - d4.x);
            p[4 * g + 1] = p[4 * g + 1] * (dp[4 * g + 1] - d4.y);
            p[4 * g + 2] = p[4 * g + 2] * (dp[4 * g + 2] - d4.z);
            p[4 * g + 3] = p[4 * g + 3] * (dp[4 * g + 3] - d4.w);
        }
        tile_accumulate_t(Qs + col_lds, p, k0a, k1a);
    }

    // Add the four partial dK^T / dV^T blocks in wavefront order: every wavefront leaves its blocks in its own LDS region
    // (no barrier before the writes, as above), and behind the barrier wavefront w adds and stores the accumulator
    // registers 4w .. 4w + 3 (16 of the 64 columns of dK and of dV).
    float *mine = lds + wave * REGION;   // [64][64]: rows 4r .. 4r + 3 = k0a[r], k1a[r], v0a[r], v1a[r]
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        mine[(4 * r + 0) * 64 + lane] = k0a[r]; mine[(4 * r + 1) * 64 + lane] = k1a[r];
        mine[(4 * r + 2) * 64 + lane] = v0a[r]; mine[(4 * r + 3) * 64 + lane] = v1a[r];
    }
    __syncthreads();
    float sum[16];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const float *rows = lds + x * REGION + (16 * wave) * 64 + lane;
#pragma unroll
        for (int i = 0; i < 16; ++i) sum[i] = x == 0 ? rows[i * 64] : sum[i] + rows[i * 64];
    }
    if (key < Lk) {
        // sum[4i + {0,1,2,3}] = k0a, k1a, v0a, v1a of register 4w + i: columns 16w + 4(i/2)... in store_row_t's order
        const int ncols = hd - 8 * half - 16 * wave;
        float *pk = dk + kv_base + (long long)key * rs + 8 * half + 16 * wave, *pv = dv + kv_base + (long long)key * rs + 8 * half + 16 * wave;
        const f32x4 klo = {sum[0] * LN2, sum[1] * LN2, sum[4] * LN2, sum[5] * LN2}, khi = {sum[8] * LN2, sum[9] * LN2, sum[12] * LN2, sum[13] * LN2};
        const f32x4 vlo = {sum[2] * 1.0f, sum[3] * 1.0f, sum[6] * 1.0f, sum[7] * 1.0f}, vhi = {sum[10] * 1.0f, sum[11] * 1.0f, sum[14] * 1.0f, sum[15] * 1.0f};
        if (0 < ncols) { *reinterpret_cast<f32x4 *>(pv) = vlo; *reinterpret_cast<f32x4 *>(pk) = klo; }
        if (4 < ncols) { *reinterpret_cast<f32x4 *>(pv + 4) = vhi; *reinterpret_cast<f32x4 *>(pk + 4) = khi; }
    }
}

// ------------------------------------------------------------------------------------------------ other head dims
// Plain gradient kernels for head dims other than 64 (up to 256, key dim = value dim = d), the counterpart of the plain
// forward kernel: correctness paths for small models, one wavefront per query row (dq) and per key row (dk, dv).
// Weights are recomputed as exp(s - mx) * inv from the statistics the plain forward kernel leaves.
__global__ __launch_bounds__(64) void sdpa_bwd_rowdot_plain(const float *__restrict__ out, const float *__restrict__ dout,
                                                             float *__restrict__ D, int d) {
    const long long row = blockIdx.x;
    float acc = 0.f;
    for (int c = threadIdx.x; c < d; c += 64) acc += out[row * d + c] * dout[row * d + c];
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (threadIdx.x == 0) D[row] = acc;
}

__global__ __launch_bounds__(64) void sdpa_bwd_dq_plain(const float *__restrict__ q, const float *__restrict__ k,
                                                         const float *__restrict__ v, const float *__restrict__ dout,
                                                         const float *__restrict__ stats, const float *__restrict__ D,
                                                         float *__restrict__ dq, int H, int Lq, int Lk, int d, float rT,
                                                         MaskArgs mask) {
    __shared__ float qs[GEN_MAXD], go[GEN_MAXD], ds[64];
    const int row = blockIdx.x;   // over B*H*Lq
    const int qi = row % Lq, bh = row / Lq, b = bh / H, hh = bh % H, lane = threadIdx.x;
    for (int c = lane; c < d; c += 64) {
        qs[c] = q[(long long)row * d + c] * rT;
        go[c] = dout[(long long)row * d + c];
    }
    __syncthreads();
    const float *kp = k + (long long)bh * Lk * d, *vp = v + (long long)bh * Lk * d;
    int len = Lk;
    if (mask.kind == DL4S_MASK_KEY_LENGTHS || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS) len = mask.lengths[b];
    const float mx = stats[2 * (long long)row], inv = stats[2 * (long long)row + 1], Di = D[row];
    float acc[GEN_MAXD / 64];
    for (int i = 0; i < GEN_MAXD / 64; ++i) acc[i] = 0.f;
    for (int j0 = 0; j0 < Lk; j0 += 64) {
        const int j = j0 + lane;
        float g = 0.f;
        if (j < Lk) {
            const float p = expf(plain_score(qs, kp + (long long)j * d, d, mask, b, hh, qi, j, len) - mx) * inv;
            float dp = 0.f;
            for (int c = 0; c < d; ++c) dp += go[c] * vp[(long long)j * d + c];
            g = p * (dp - Di);
        }
        ds[lane] = g;
        __syncthreads();
        const int n = min(64, Lk - j0);
        for (int i = 0; i < GEN_MAXD / 64; ++i) {
            const int c = lane + 64 * i;
            if (c < d)
                for (int jj = 0; jj < n; ++jj) acc[i] += ds[jj] * kp[(long long)(j0 + jj) * d + c];
        }
        __syncthreads();
    }
    for (int i = 0; i < GEN_MAXD / 64; ++i) {
        const int c = lane + 64 * i;
        if (c < d) dq[(long long)row * d + c] = acc[i] * rT;
    }
}

__global__ __launch_bounds__(64) void sdpa_bwd_dkv_plain(const float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v, const float *__restrict__ dout,
                                                          const float *__restrict__ stats, const float *__restrict__ D,
                                                          float *__restrict__ dk, float *__restrict__ dv, int H, int Lq, int Lk,
                                                          int d, float rT, MaskArgs mask) {
    __shared__ float kj[GEN_MAXD], vj[GEN_MAXD], ps[64], ds[64];
    const int row = blockIdx.x;   // over B*H*Lk
    const int j = row % Lk, bh = row / Lk, b = bh / H, hh = bh % H, lane = threadIdx.x;
    for (int c = lane; c < d; c += 64) {
        kj[c] = k[(long long)row * d + c];
        vj[c] = v[(long long)row * d + c];
    }
    __syncthreads();
    const float *qp = q + (long long)bh * Lq * d, *gp = dout + (long long)bh * Lq * d;
    int len = Lk;
    if (mask.kind == DL4S_MASK_KEY_LENGTHS || mask.kind == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS) len = mask.lengths[b];
    float acck[GEN_MAXD / 64], accv[GEN_MAXD / 64];
    for (int i = 0; i < GEN_MAXD / 64; ++i) { acck[i] = 0.f; accv[i] = 0.f; }
    for (int i0 = 0; i0 < Lq; i0 += 64) {
        const int qi = i0 + lane;
        float p = 0.f, g = 0.f;
        if (qi < Lq) {
            // the score with the forward kernel's roundings: (q * rT) . k accumulated in order, then the mask
            float s = 0.f;
            for (int c = 0; c < d; ++c) s = __fadd_rn(s, __fmul_rn(qp[(long long)qi * d + c] * rT, kj[c]));
            s = plain_masked(s, mask, b, hh, qi, j, len);
            const long long r = (long long)bh * Lq + qi;
            p = expf(s - stats[2 * r]) * stats[2 * r + 1];
            float dp = 0.f;
            for (int c = 0; c < d; ++c) dp += gp[(long long)qi * d + c] * vj[c];
            g = p * (dp - D[r]);
        }
        ps[lane] = p;
        ds[lane] = g;
        __syncthreads();
        const int n = min(64, Lq - i0);
        for (int i = 0; i < GEN_MAXD / 64; ++i) {
            const int c = lane + 64 * i;
            if (c < d)
                for (int ii = 0; ii < n; ++ii) {
                    accv[i] += ps[ii] * gp[(long long)(i0 + ii) * d + c];
                    acck[i] += ds[ii] * (qp[(long long)(i0 + ii) * d + c] * rT);
                }
        }
        __syncthreads();
    }
    for (int i = 0; i < GEN_MAXD / 64; ++i) {
        const int c = lane + 64 * i;
        if (c < d) {
            dv[(long long)row * d + c] = accv[i];
            dk[(long long)row * d + c] = acck[i];
        }
    }
}

template <int KIND>
int launch_bwd(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *dout, const float *stats,
               const float *D, float *dq, float *dk, float *dv, int B, int H, int Lq, int Lk, float rT, const MaskArgs &m,
               int strict, int token_major, int hd, int no_split) {
    constexpr bool causal_kind = (KIND == DL4S_MASK_CAUSAL || KIND == DL4S_MASK_CAUSAL_OR_KEY_LENGTHS);
    if (hd <= 32) {     // narrow heads: tiles of 16 or 32 columns on the stored-dS route, when the launch can take it
        const int rn = hd <= 16 ? launch_bwd_narrow<KIND, 16>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, rT, m, strict, token_major,
                                                              hd, no_split, ds_scratch_max_bytes())
                                : launch_bwd_narrow<KIND, 32>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, rT, m, strict, token_major,
                                                              hd, no_split, ds_scratch_max_bytes());
        if (rn != 0) return rn < 0 ? rn : DL4S_HIP_OK;
    }
    const size_t lds_dq = 4 * TILE_FLOATS * sizeof(float);
    const size_t lds_dkv = (4 * TILE_FLOATS + 192) * sizeof(float);
    const size_t lds_dq_split = 8 * TILE_FLOATS * sizeof(float);
    const size_t lds_dkv_split = 4 * (2 * TILE_FLOATS + 96) * sizeof(float);
    if (dl4s::lds_limit_pending(ctx, dl4s::LDS_BWD, KIND)) {
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dq_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dkv_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dkv_f32_d64<KIND, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dq_split_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dq_split));
        DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_bwd_dkv_split_f32_d64<KIND>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_dkv_split));
        dl4s::lds_limit_done(ctx, dl4s::LDS_BWD, KIND);
    }
    const bool uneven = (causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict;
    const bool dq_small = !no_split && sdpa_bwd_small_launch(ctx, B, H, Lq, uneven, false) && Lk >= 2 * BN;
    const bool dkv_small = !no_split && sdpa_bwd_small_launch(ctx, B, H, Lk, uneven, false) && Lq >= 2 * BN;
    // Large launches: the dK/dV kernel stores dS, the dQ kernel only contracts it with K (five products for five).  The
    // scratch tensor [B*H][Lk][Lq] comes from the pool; when it cannot be had (too large, pool miss while a graph is being
    // recorded, out of memory) the two self-contained kernels below run instead.
    if (!dq_small && !dkv_small) {
        const long long Lqp = (Lq + 31) & ~31ll, Lkp = (Lk + 31) & ~31ll;
        const long long slab = Lqp * Lkp * 4;
        const int nqb = (Lq + BM - 1) / BM, nkb = (Lk + BM - 1) / BM;
        const long long total_q = (long long)nqb * B * H, total_k = (long long)nkb * B * H;
        void *dsv = nullptr;
        if (slab < (1ll << 31) && (long long)B * H * slab <= ds_scratch_max_bytes() && total_q < (1ll << 30) && total_k < (1ll << 30) &&
            dl4s_hip_alloc(ctx, (size_t)((long long)B * H * slab), &dsv) == DL4S_HIP_OK) {
            float *ds = static_cast<float *>(dsv);
            int lpt = (uneven && nkb >= 2) ? 1 : 0;
            // (reversed rounds as well up to five workgroups per CU, two and a half times what is resident at once: B4 H16 L2048
            // 792 -> 764 us, B8 H16 L1024 438 -> 415 us, B1 H16 L8192 3.00 -> 2.85 ms; at eight per CU it loses 1.5 %)
            if (lpt && total_k <= 5ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
            hipLaunchKernelGGL((sdpa_bwd_dkv_f32_d64<KIND, true>), dim3((unsigned)((total_k + 7) / 8 * 8)), dim3(256), lds_dkv, ctx->stream, q,
                               k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb, (int)total_k, lpt, token_major, hd, ds);
            int rc = dl4s::launch_status("sdpa_bwd_dkv_f32_d64");
            if (rc == DL4S_HIP_OK) {
                lpt = (uneven && nqb >= 2) ? 1 : 0;
                if (lpt && total_q <= 5ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
                hipLaunchKernelGGL(sdpa_bwd_dq_from_ds_f32_d64<KIND>, dim3((unsigned)((total_q + 7) / 8 * 8)), dim3(256),
                                   2 * TILE_FLOATS * sizeof(float), ctx->stream, k, ds, dq, H, Lq, Lk, rT, m, strict, nqb, (int)total_q,
                                   lpt, token_major, hd);
                rc = dl4s::launch_status("sdpa_bwd_dq_from_ds_f32_d64");
            }
            const int rcf = dl4s_hip_free(ctx, dsv);   // stream-ordered
            return rc != DL4S_HIP_OK ? rc : rcf;
        }
    }
    // Small launches (the forward pass's rule, from the extents only): one 32-row block per workgroup, the tiles along the
    // other axis split over its four wavefronts.
    if (dq_small) {
        const int nqb32 = (Lq + 31) / 32;
        const long long total = (long long)nqb32 * B * H;
        int order = (uneven && nqb32 >= 2) ? 1 : 0;
        if (order && total <= 2ll * ctx->cu_count) order |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL(sdpa_bwd_dq_split_f32_d64<KIND>, dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dq_split, ctx->stream,
                           q, k, v, dout, stats, D, dq, H, Lq, Lk, rT, m, strict, nqb32, (int)total, order, token_major, hd);
        const int rc = dl4s::launch_status("sdpa_bwd_dq_split_f32_d64");
        if (rc != DL4S_HIP_OK) return rc;
    } else {
        const int nqb = (Lq + BM - 1) / BM;
        const long long total = (long long)nqb * B * H;
        DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa backward: %lld workgroups exceed the grid limit", total);
        // longest first; in a launch that fits the chip at once (two workgroups per CU) also every second round of the CUs
        // reversed, which pairs long items with short ones on a CU
        int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nqb >= 2) ? 1 : 0;
        if (lpt && total <= 2ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL(sdpa_bwd_dq_f32_d64<KIND>, dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dq, ctx->stream, q, k,
                           v, dout, stats, D, dq, H, Lq, Lk, rT, m, strict, nqb, (int)total, lpt, token_major, hd);
        const int rc = dl4s::launch_status("sdpa_bwd_dq_f32_d64");
        if (rc != DL4S_HIP_OK) return rc;
    }
    if (dkv_small) {
        const int nkb32 = (Lk + 31) / 32;
        const long long total = (long long)nkb32 * B * H;
        int order = (uneven && nkb32 >= 2) ? 1 : 0;
        if (order && total <= 2ll * ctx->cu_count) order |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL(sdpa_bwd_dkv_split_f32_d64<KIND>, dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dkv_split, ctx->stream,
                           q, k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb32, (int)total, order, token_major, hd);
        return dl4s::launch_status("sdpa_bwd_dkv_split_f32_d64");
    }
    {
        const int nkb = (Lk + BM - 1) / BM;
        const long long total = (long long)nkb * B * H;
        DL4S_REQUIRE(total < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa backward: %lld workgroups exceed the grid limit", total);
        int lpt = ((causal_kind || (KIND == DL4S_MASK_DENSE_F32 && m.cls && m.sq)) && !strict && nkb >= 2) ? 1 : 0;
        if (lpt && total <= 2ll * ctx->cu_count) lpt |= (ctx->cu_count / 8) << 1;
        hipLaunchKernelGGL(sdpa_bwd_dkv_f32_d64<KIND>, dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), lds_dkv, ctx->stream, q,
                           k, v, dout, stats, D, dk, dv, H, Lq, Lk, rT, m, strict, nkb, (int)total, lpt, token_major, hd);
        return dl4s::launch_status("sdpa_bwd_dkv_f32_d64");
    }
}

}  // namespace

#include "sdpa_backward_wide.h"


extern "C" int dl4s_hip_sdpa_bwd_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *out,
                                     const float *stats, const float *dout, float *dq, float *dk, float *dv, int64_t B,
                                     int64_t H, int64_t Lq, int64_t Lk, int64_t d, float inv_temperature,
                                     const dl4s_mask_desc *mask, uint32_t flags) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0 && Lq >= 0 && Lk >= 0 && d >= 0, DL4S_HIP_EINVALID_ARG, "sdpa backward: negative extent");
    DL4S_REQUIRE(d > 0 && d <= GEN_MAXD, DL4S_HIP_EUNSUPPORTED, "sdpa backward: head dim %lld is not implemented (1..%d)",
                 (long long)d, GEN_MAXD);
    DL4S_REQUIRE((flags & ~(uint32_t)(DL4S_SDPA_STRICT | DL4S_SDPA_TOKEN_MAJOR | DL4S_SDPA_NO_KEY_SPLIT)) == 0, DL4S_HIP_EINVALID_ARG,
                 "sdpa backward: unknown flag bits 0x%x", flags);
    if (B * H == 0 || (Lq == 0 && Lk == 0)) return DL4S_HIP_OK;
    DL4S_REQUIRE(Lk > 0, DL4S_HIP_ESHAPE, "sdpa backward: keyCount is 0");
    DL4S_REQUIRE(k && v && dk && dv, DL4S_HIP_EINVALID_ARG, "sdpa backward: NULL tensor pointer");
    const int token_major = (flags & DL4S_SDPA_TOKEN_MAJOR) ? 1 : 0;
    if (Lq == 0) {   // no queries: the keys and values receive no gradient
        if (token_major) return dl4s::set_error(DL4S_HIP_EUNSUPPORTED, "sdpa backward: empty query axis in the token-major layout");
        const int rc = dl4s_hip_fill_f32(ctx, 0.f, dk, B * H * Lk * d);
        return rc != DL4S_HIP_OK ? rc : dl4s_hip_fill_f32(ctx, 0.f, dv, B * H * Lk * d);
    }
    DL4S_REQUIRE(q && out && stats && dout && dq, DL4S_HIP_EINVALID_ARG, "sdpa backward: NULL tensor pointer");
    DL4S_REQUIRE(B * H * (Lq > Lk ? Lq : Lk) * d < (1ll << 40) && Lq < (1ll << 30) && Lk < (1ll << 30), DL4S_HIP_EUNSUPPORTED,
                 "sdpa backward: extents too large");
    // head dims that are multiples of 4 up to 64 run on the MFMA kernels (tiles padded with zero columns) when every row
    // starts on a 16-byte boundary
    // The route follows the forward pass's rule (head dim, alignment of q, k, v, out): the two kinds of kernels keep the
    // row statistics in different forms (base-2 and natural exponent), so the gradient call must land where the forward
    // call landed.  On the MFMA route the gradient tensors have to be aligned as well.
    const bool fwd_aligned = ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
                               reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const bool grads_aligned = ((reinterpret_cast<uintptr_t>(dout) | reinterpret_cast<uintptr_t>(dq) | reinterpret_cast<uintptr_t>(dk) |
                                 reinterpret_cast<uintptr_t>(dv)) & 15) == 0;
    const bool mfma_path = d > 0 && d <= HD && d % 4 == 0 && fwd_aligned;
    const bool mfma128_path = d > HD && d <= HD2 && d % 4 == 0 && fwd_aligned;
    // head dims above 128: the forward call ran the 192- / 256-wide kernels
    const bool wide_as_is = d > HD2 && d <= 256 && d % 4 == 0 && fwd_aligned;    // no copies, whichever kernel it was
    const bool wide_path = wide_as_is && sdpa_wide_route(H, Lk, d, token_major);
    // the forward pass ran on zero-padded copies (sdpa_padded_route): so does this call, gradients included
    if (!token_major && sdpa_padded_route(mfma_path || mfma128_path || wide_as_is, B, H, Lq, Lk, d, d)) {
        const int64_t dp = (d + 3) / 4 * 4, qrows = B * H * Lq, krows = B * H * Lk;
        const int64_t rows_of[8] = {qrows, krows, krows, qrows, qrows, qrows, krows, krows};   // q k v out dout dq dk dv
        void *bufs[8] = {nullptr};
        for (int i = 0; i < 8; ++i)
            if (dl4s_hip_alloc(ctx, (size_t)(rows_of[i] * dp) * sizeof(float), &bufs[i]) != DL4S_HIP_OK) {
                for (int j = 0; j < i; ++j) (void)dl4s_hip_free(ctx, bufs[j]);
                return DL4S_HIP_EOOM;
            }
        float *p[8];
        for (int i = 0; i < 8; ++i) p[i] = static_cast<float *>(bufs[i]);
        const float *src[5] = {q, k, v, out, dout};
        for (int i = 0; i < 5; ++i) launch_copy_rows(ctx, src[i], p[i], rows_of[i], d, dp);
        int rc = dl4s::launch_status("copy_rows_f32");
        if (rc == DL4S_HIP_OK)
            rc = dl4s_hip_sdpa_bwd_f32(ctx, p[0], p[1], p[2], p[3], stats, p[4], p[5], p[6], p[7], B, H, Lq, Lk, dp, inv_temperature, mask, flags);
        if (rc == DL4S_HIP_OK) {
            float *dst[3] = {dq, dk, dv};
            for (int i = 0; i < 3; ++i) launch_copy_rows(ctx, p[5 + i], dst[i], rows_of[5 + i], dp, d);
            rc = dl4s::launch_status("copy_rows_f32");
        }
        for (int i = 0; i < 8; ++i) (void)dl4s_hip_free(ctx, bufs[i]);
        return rc;
    }
    DL4S_REQUIRE(!(mfma_path || mfma128_path || wide_path) || grads_aligned, DL4S_HIP_EUNSUPPORTED,
                 "sdpa backward: dout, dq, dk and dv must be 16-byte aligned when q, k, v and out are (the forward pass ran on "
                 "the MFMA kernels and left its row statistics in their form)");
    DL4S_REQUIRE(!mfma128_path || (Lk > Lq ? Lk : Lq) * (token_major ? H : 1) * d * 4 < (d == HD2 ? (1ll << 31) : (1ll << 30)),
                 DL4S_HIP_EUNSUPPORTED,
                 "sdpa backward: the rows of one (batch, head) pair span more than 2 GiB (1 GiB for padded head dims)");
    DL4S_REQUIRE(!mfma_path || (Lk > Lq ? Lk : Lq) * (token_major ? H : 1) * d * 4 < (d == HD ? (1ll << 31) : (1ll << 30)),
                 DL4S_HIP_EUNSUPPORTED,
                 "sdpa backward: the rows of one (batch, head) pair span more than 2 GiB (1 GiB for head dims below 64)");
    if (wide_path) {
        DL4S_REQUIRE(!token_major, DL4S_HIP_EUNSUPPORTED, "sdpa backward: the token-major layout needs a head dim of at most 128");
        return sdpa_backward_wide(ctx, q, k, v, out, stats, dout, dq, dk, dv, B, H, Lq, Lk, d, inv_temperature, mask,
                                  (flags & DL4S_SDPA_STRICT) ? 1 : 0, ds_scratch_max_bytes());
    }
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    MaskArgs m{};
    int rc = build_mask_args(ctx, mask, B, H, Lq, Lk, mfma_path || mfma128_path, m);
    if (rc != DL4S_HIP_OK) return rc;
    const int strict = (flags & DL4S_SDPA_STRICT) ? 1 : 0;
    const int no_split = (flags & DL4S_SDPA_NO_KEY_SPLIT) ? 1 : 0;
    void *Dv = nullptr;
    rc = dl4s_hip_alloc(ctx, (size_t)(B * H * Lq) * sizeof(float), &Dv);
    if (rc != DL4S_HIP_OK) return rc;
    float *D = static_cast<float *>(Dv);
    const long long rows = B * H * Lq;
    if (mfma128_path) {
        hipLaunchKernelGGL(sdpa_bwd_rowdot128, dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, ctx->stream, out, dout, D, (int)H, (int)Lq,
                           rows, token_major, (int)d);
        rc = dl4s::launch_status("sdpa_bwd_rowdot128");
        if (rc == DL4S_HIP_OK) {
            // head dims up to 96 on 96-wide tiles (three quarters of the MFMAs; up to 80 on their 80-column form, like the
            // forward call that left the statistics), the others on 128-wide ones
#define DL4S_BWD_WIDE(KIND_) \
    rc = d <= 80 ? launch_bwd128<KIND_, 80>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, ds_scratch_max_bytes(), no_split) \
       : d <= 96 ? launch_bwd128<KIND_, 96>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, ds_scratch_max_bytes(), no_split) \
                 : launch_bwd128<KIND_, 128>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, ds_scratch_max_bytes(), no_split)
            switch (m.kind) {
                case DL4S_MASK_NONE: DL4S_BWD_WIDE(DL4S_MASK_NONE); break;
                case DL4S_MASK_DENSE_F32: DL4S_BWD_WIDE(DL4S_MASK_DENSE_F32); break;
                case DL4S_MASK_CAUSAL: DL4S_BWD_WIDE(DL4S_MASK_CAUSAL); break;
                case DL4S_MASK_KEY_LENGTHS: DL4S_BWD_WIDE(DL4S_MASK_KEY_LENGTHS); break;
                default: DL4S_BWD_WIDE(DL4S_MASK_CAUSAL_OR_KEY_LENGTHS); break;
            }
#undef DL4S_BWD_WIDE
        }
        const int rcf = dl4s_hip_free(ctx, Dv);
        return rc != DL4S_HIP_OK ? rc : rcf;
    }
    if (!mfma_path) {   // plain kernels
        rc = DL4S_HIP_OK;
        if (token_major) rc = dl4s::set_error(DL4S_HIP_EUNSUPPORTED, "sdpa backward: the token-major layout needs a head dim that is a multiple of 4, at most 128, and 16-byte aligned tensors");
        else if (rows >= (1ll << 31) || B * H * Lk >= (1ll << 31)) rc = dl4s::set_error(DL4S_HIP_EUNSUPPORTED, "sdpa backward: too many rows for the plain kernels");
        if (rc == DL4S_HIP_OK) {
            hipLaunchKernelGGL(sdpa_bwd_rowdot_plain, dim3((unsigned)rows), dim3(64), 0, ctx->stream, out, dout, D, (int)d);
            hipLaunchKernelGGL(sdpa_bwd_dq_plain, dim3((unsigned)rows), dim3(64), 0, ctx->stream, q, k, v, dout, stats, D, dq, (int)H,
                               (int)Lq, (int)Lk, (int)d, inv_temperature, m);
            hipLaunchKernelGGL(sdpa_bwd_dkv_plain, dim3((unsigned)(B * H * Lk)), dim3(64), 0, ctx->stream, q, k, v, dout, stats, D, dk,
                               dv, (int)H, (int)Lq, (int)Lk, (int)d, inv_temperature, m);
            rc = dl4s::launch_status("sdpa_bwd_plain");
        }
        const int rcf = dl4s_hip_free(ctx, Dv);
        return rc != DL4S_HIP_OK ? rc : rcf;
    }
    hipLaunchKernelGGL(sdpa_bwd_rowdot, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, ctx->stream, out, dout, D, (int)H, (int)Lq,
                       rows, token_major, (int)d);
    rc = dl4s::launch_status("sdpa_bwd_rowdot");
    if (rc == DL4S_HIP_OK) {
        switch (m.kind) {
            case DL4S_MASK_NONE: rc = launch_bwd<DL4S_MASK_NONE>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, no_split); break;
            case DL4S_MASK_DENSE_F32: rc = launch_bwd<DL4S_MASK_DENSE_F32>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, no_split); break;
            case DL4S_MASK_CAUSAL: rc = launch_bwd<DL4S_MASK_CAUSAL>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, no_split); break;
            case DL4S_MASK_KEY_LENGTHS: rc = launch_bwd<DL4S_MASK_KEY_LENGTHS>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, no_split); break;
            default: rc = launch_bwd<DL4S_MASK_CAUSAL_OR_KEY_LENGTHS>(ctx, q, k, v, dout, stats, D, dq, dk, dv, B, H, Lq, Lk, inv_temperature, m, strict, token_major, (int)d, no_split); break;
        }
    }
    const int rc2 = dl4s_hip_free(ctx, Dv);   // stream-ordered: later users of the block queue behind these kernels
    return rc != DL4S_HIP_OK ? rc : rc2;
}

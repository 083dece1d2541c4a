// fp32 GEMM on v_mfma_f32_32x32x2_f32 for gfx950:  C = alpha * op(A) . op(B) + beta * C, row-major, optional strided
// batch, optional epilogue act(. + bias[n]) + residual[m][n] (the fused Dense forms).  A workgroup (4 wavefronts, 2x2)
// computes a 128x128 (or 64x64) tile of C; the next K step is prefetched into registers while the current one is
// multiplied.  Two kernels:
//   gemm_f32_mfma      any (row stride, column stride) operands, i.e. every transpose combination: scalar loads, LDS
//                      tiles stored k-major ([k][m] and [k][n]) so that the MFMA operand reads (lane l wants row l % 32
//                      at k = l / 32) are consecutive 32-bit words; the thread-to-element mapping of the loader is
//                      chosen so that the unit-stride direction runs along the lanes
//   gemm_f32_mfma_fast every transpose combination of aligned operands with extents that are multiples of 4 (the layers'
//                      products and their gradients): 128-bit buffer loads, see below
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GBM = 128, GBN = 128, GBK = 16;
constexpr int GLS = GBM + 4;  // LDS row stride in floats

struct GemmArgs {
    const float *A, *B;
    float *C;
    int M, N, K;
    long long a_rs, a_cs;  // element strides of op(A)[m][k]
    long long b_rs, b_cs;  // element strides of op(B)[k][n]
    long long a_bs, b_bs, c_bs;  // batch strides
    // grouped launches (groups > 0): blockIdx.z selects one of up to 4 products of the same shape whose operands lie at
    // these element offsets from A, B, C
    int groups;
    long long a_off[4], b_off[4], c_off[4];
    long long lda, ldb;          // row strides of A and B as stored (the fast kernels)
    float alpha, beta;
    int tiles_n;
    // epilogue of the fused Dense forms: C = act(alpha * A.B + bias[n]) + residual[m][n]
    const float *bias, *residual;
    int act;   // 0 none, 1 gaussianErrorLinear
    // LayerNorm statistics from the epilogue (the fused Dense forms on the tiled kernels): when ln_part is set, every
    // workgroup also leaves the sum and the sum of squares of the values it stored.  The rows of one normalised item
    // span ln_tiles_m row tiles; item i's pairs are ln_part[(i * ln_tiles_m * tiles_n + (tile_m % ln_tiles_m) * tiles_n +
    // tile_n) * 2 ..], the layout ln_apply_f32 sums in a fixed order.
    float *ln_part;
    int ln_tiles_m;
    // Products with a causal triangle (the tiled fast kernels, callers inside the library; rows and columns count from the
    // same origin): 1 = only the output tiles that hold an element with column <= row are computed, the others are
    // left untouched; 2 = the contraction index starts at the output tile's first row (everything before it is known to be
    // zero in A); 3 = the contraction index ends with the output tile's last row (everything after it is zero in A).
    int tri;
};

// x * (0.5 * tanh(0.5 * (1.702 * x)) + 0.5), every operation rounded, as Tensor/Operators/Unary.swift:184-186, :245-247
__device__ __forceinline__ float gelu_sigmoid(float v) {
    const float a = __fmul_rn(v, 1.702f);
    const float t = tanhf(__fmul_rn(a, 0.5f));
    return __fmul_rn(v, __fadd_rn(__fmul_rn(0.5f, t), 0.5f));
}

__device__ __forceinline__ float epilogue(const GemmArgs &g, float val, long long gm, int gn) {
    if (g.bias) val = __fadd_rn(val, g.bias[gn]);
    if (g.act == 1) val = gelu_sigmoid(val);
    if (g.residual) val = __fadd_rn(val, g.residual[gm * g.N + gn]);
    return val;
}

__global__ __launch_bounds__(256, 2) void gemm_f32_mfma(GemmArgs g) {
    __shared__ float As[2][GBK][GLS];
    __shared__ float Bs[2][GBK][GLS];
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int half = lane >> 5, ln = lane & 31;
    const int wm = wave >> 1, wn = wave & 1;
    const int tile_m = blockIdx.x / g.tiles_n, tile_n = blockIdx.x % g.tiles_n;
    const int m0 = tile_m * GBM, n0 = tile_n * GBN;
    const float *A = g.A + (g.groups ? g.a_off[blockIdx.z] : (long long)blockIdx.z * g.a_bs);
    const float *B = g.B + (g.groups ? g.b_off[blockIdx.z] : (long long)blockIdx.z * g.b_bs);
    float *C = g.C + (g.groups ? g.c_off[blockIdx.z] : (long long)blockIdx.z * g.c_bs);

    // loader mappings: unit stride along k -> 16 lanes walk k; otherwise 128 threads walk m (or n)
    const bool a_kfast = (g.a_cs == 1);
    const bool b_kfast = (g.b_rs == 1);
    float ast[8], bst[8];
    auto load = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int kk, mm;
            if (a_kfast) { kk = tid & 15; mm = (tid >> 4) + 16 * i; } else { mm = tid & 127; kk = (tid >> 7) + 2 * i; }
            const int gm = m0 + mm, gk = kt * GBK + kk;
            ast[i] = (gm < g.M && gk < g.K) ? A[gm * g.a_rs + gk * g.a_cs] : 0.f;
            int kb, nn;
            if (b_kfast) { kb = tid & 15; nn = (tid >> 4) + 16 * i; } else { nn = tid & 127; kb = (tid >> 7) + 2 * i; }
            const int gn = n0 + nn, gkb = kt * GBK + kb;
            bst[i] = (gn < g.N && gkb < g.K) ? B[gkb * g.b_rs + gn * g.b_cs] : 0.f;
        }
    };
    auto store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int kk, mm;
            if (a_kfast) { kk = tid & 15; mm = (tid >> 4) + 16 * i; } else { mm = tid & 127; kk = (tid >> 7) + 2 * i; }
            As[buf][kk][mm] = ast[i];
            int kb, nn;
            if (b_kfast) { kb = tid & 15; nn = (tid >> 4) + 16 * i; } else { nn = tid & 127; kb = (tid >> 7) + 2 * i; }
            Bs[buf][kb][nn] = bst[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int ktiles = (g.K + GBK - 1) / GBK;
    if (ktiles > 0) { load(0); store(0); }
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
        const int buf = kt & 1;
        const bool more = kt + 1 < ktiles;
        if (more) load(kt + 1);
#pragma unroll
        for (int ks = 0; ks < GBK / 2; ++ks) {
            const int kk = 2 * ks + half;
            const float a0 = As[buf][kk][wm * 64 + ln];
            const float a1 = As[buf][kk][wm * 64 + 32 + ln];
            const float b0 = Bs[buf][kk][wn * 64 + ln];
            const float b1 = Bs[buf][kk][wn * 64 + 32 + ln];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        if (more) store(buf ^ 1);
        __syncthreads();
    }

    // accumulator register r of a 32x32 tile: row 8*(r/4) + 4*half + r%4, column ln
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int gn = n0 + wn * 64 + j * 32 + ln;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int gm = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (gm < g.M && gn < g.N) {
                    float *cp = C + (long long)gm * g.N + gn;
                    float val = g.alpha * acc[i][j][r];
                    if (g.beta != 0.f) val = val + g.beta * (*cp);
                    *cp = epilogue(g, val, gm, gn);
                }
            }
        }
}

// Fast kernels: 128-bit buffer loads, K and the unit-stride extents multiples of 4, 16-byte aligned operands.  Same
// 2x2 wavefront layout as above.  An operand is staged in one of two ways, chosen by how it lies in memory:
//   rows x K, K contiguous (A, or B when transposeSecond)   kept [row][k] in LDS on a row stride of KT + 4 floats, so that
//                                                           128-bit operand reads of 8 rows fall on distinct banks
//                                                           and one LDS read feeds four MFMA steps
//   K x rows, rows contiguous (B, or A when transposeFirst) kept [k][row] in LDS, read one word per MFMA step
// Both go through buffer loads with the whole byte offset in the (range-checked) vector operand: rows past the extent,
// K rows past K and -- through an offset beyond any descriptor -- columns past the extent read as zeros, so a K step
// costs one add per load and no predication.  MFMA step s of a 16-deep half of a K tile takes k = 8*half + s from both
// operands (any bijection of k works as long as A and B agree).
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned OUTSIDE = 0x80000000u;   // an offset beyond every descriptor (the host keeps them below 2^31 bytes)

// One operand of the fast kernels.  XI = MFMA tiles per wavefront along this operand's extent (tile extent T = 64*XI);
// KROWS = true for the K x rows memory layout; KT = depth of a K tile (16 or 32).  A K tile of 32 is contracted as two
// halves of 16 one after the other, so that an output element sees its products in the same order whatever KT is.
// SLOTS = register sets for tiles in flight: with two, the tile after the next is requested while the next one waits in
// registers for its turn in LDS, so a load has two K steps to arrive.
template <int XI, bool KROWS, int KT, int SLOTS = 1>
struct FastOperand {
    static constexpr int T = 64 * XI;
    static constexpr int LS = KT + 4;            // row stride of a [row][k] tile (floats): 128-bit reads of 8 rows on distinct banks
    static constexpr int LDS_FLOATS = KROWS ? 2 * KT * (T + 4) : 2 * T * LS;
    static constexpr int NV = XI * KT / 16;      // 128-bit pieces per thread and K tile
    static constexpr int Q = T / 4, PASS_ROWS = 256 / Q;      // K x rows: pieces per K row, K rows covered per pass
    static constexpr int QK = KT / 4, RP = 256 / QK;          // rows x K: pieces per row, rows covered per pass
    float *lds;
    __amdgpu_buffer_rsrc_t rsrc;
    unsigned off[NV];
    unsigned step;          // byte step of one K tile
    f32x4 st[SLOTS][NV];
    int kq;                 // rows x K: the thread's k quad
    bool ragged_k;
    int K;

    // base: the operand's matrix (batch applied); extent rows, row stride rs (elements), first row / column r0 of the tile
    __device__ __forceinline__ void init(float *lds_, const float *base, int extent, long long rs, int r0, int K_, int tid) {
        lds = lds_;
        K = K_;
        ragged_k = (K % KT) != 0;
        if (KROWS) {
            const int krow = tid / Q, rq = (tid % Q) * 4;
            rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(base + r0), 0, (int)((((long long)K - 1) * rs + (extent - r0)) * 4), 0x00020000);
#pragma unroll
            for (int i = 0; i < NV; ++i) off[i] = (r0 + rq < extent) ? (unsigned)((krow + PASS_ROWS * i) * (int)rs + rq) * 4u : OUTSIDE;
            step = (unsigned)KT * (unsigned)rs * 4u;
            kq = 0;
        } else {
            const int row = tid / QK;
            kq = (tid % QK) * 4;
            const long long rem = ((long long)(extent - r0 - 1) * rs + K) * 4;
            rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(base + (long long)r0 * rs), 0, (int)(rem < 0x7fffffffll ? rem : 0x7fffffffll), 0x00020000);
#pragma unroll
            for (int i = 0; i < NV; ++i) off[i] = (r0 + row + RP * i < extent) ? (unsigned)((row + RP * i) * (int)rs + kq) * 4u : OUTSIDE;
            step = (unsigned)KT * 4u;
        }
    }
    template <int SLOT = 0>
    __device__ __forceinline__ void load(int kt) {
        // rows x K on the last K step of a ragged K: quads at or past K lie inside the next row, so they are sent outside
        const bool past = !KROWS && ragged_k && (kt * KT + kq >= K);
#pragma unroll
        for (int i = 0; i < NV; ++i)
            st[SLOT][i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(past ? OUTSIDE : off[i] + kt * step), 0, 0));
    }
    template <int SLOT = 0>
    __device__ __forceinline__ void store(int buf, int tid) {
        if (KROWS) {
            const int krow = tid / Q, rq = (tid % Q) * 4;
#pragma unroll
            for (int i = 0; i < NV; ++i) *reinterpret_cast<f32x4 *>(lds + (buf * KT + krow + PASS_ROWS * i) * (T + 4) + rq) = st[SLOT][i];
        } else {
            const int row = tid / QK;
#pragma unroll
            for (int i = 0; i < NV; ++i) *reinterpret_cast<f32x4 *>(lds + (buf * T + row + RP * i) * LS + kq) = st[SLOT][i];
        }
    }
    // rows x K: the lane's fragment of tile x for half h2 of the K tile (k = 16*h2 + 8*half .. + 7)
    __device__ __forceinline__ void fragment(int buf, int row, int half, int h2, f32x4 (&f)[2]) const {
        f[0] = *reinterpret_cast<const f32x4 *>(lds + (buf * T + row) * LS + 16 * h2 + 8 * half);
        f[1] = *reinterpret_cast<const f32x4 *>(lds + (buf * T + row) * LS + 16 * h2 + 8 * half + 4);
    }
    // K x rows: the lane's value for MFMA step s8 of half h2
    __device__ __forceinline__ float word(int buf, int row, int half, int h2, int s8) const {
        return lds[(buf * KT + 16 * h2 + 8 * half + s8) * (T + 4) + row];
    }
};

// MI x NI = MFMA tiles per wavefront (2x2: 128x128 workgroup tile for large products, 1x1: 64x64 so that small
// products still put a workgroup on every CU).  TA / TB: the operand is stored transposed (transposeFirst / Second).
// KT: K tile depth.  The 64x64 form runs one to three wavefronts per SIMD, where a K tile of 16 (8 MFMAs = 512 cycles
// between barriers) does not cover the latency of the next tile's loads; it takes K tiles of 32.
// (128 x 128 tiles with 32-deep K tiles hold 70 KiB of LDS: two workgroups per CU, which is all their launches have)
// HV: how the contraction is summed.  0 = tile after tile from zero.  1 and 2 (products the launcher's shape rule picks:
// few output tiles, K a multiple of 128) = the first and the second half of the K tiles each summed from zero
// and the two sums added at the end - by one group of four wavefronts that sets the first sum aside when it reaches the
// middle (1), or by two groups of four wavefronts that work on the halves side by side, each with its own LDS tiles (2:
// a launch of one workgroup per CU or less, which would otherwise run one wavefront per SIMD).  Same additions in the same
// order, same bits; which of the two runs depends on how many workgroups the launch has, which the result cannot see.
template <int MI, int NI, bool EPI, bool TA, bool TB, int KT, int HV = 0>
__global__ __launch_bounds__(HV == 2 ? 512 : 256, HV == 2 ? 1 : ((MI == 2 && KT == 32) ? 2 : 3)) void gemm_f32_mfma_fast(GemmArgs g) {
    static_assert(HV == 0 || (MI == 1 && NI == 1), "the halved contraction exists for the 64 x 64 form");
    constexpr int TM = 64 * MI, TN = 64 * NI;       // workgroup tile
    // The 64 x 64 form runs one to three wavefronts per SIMD and a K step of 16 MFMAs (0.4 us) is shorter than a load's way
    // through L2: it keeps two tiles in flight ([2048,512]x[512,512] 15.1 -> 14.0 us, with the LayerNorm sums 21.0 -> 19.7 us,
    // three such products in one launch 29.9 -> 29.2 us).  Same order of additions, same bits.
    constexpr int SLOTS = (MI == 1 && NI == 1 && KT == 32) ? 2 : 1;
    using OpA = FastOperand<MI, TA, KT, SLOTS>;      // A is M x K in memory unless transposed
    using OpB = FastOperand<NI, !TB, KT, SLOTS>;     // B is K x N in memory unless transposed
    extern __shared__ __align__(16) float gemm_lds[];
    const int grp = HV == 2 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;     // the wavefront's group
    float *As = gemm_lds + grp * (OpA::LDS_FLOATS + OpB::LDS_FLOATS), *Bs = As + OpA::LDS_FLOATS;
    // Every argument on the way to the first tile's loads is asked for at once (fetched where the code first needs them,
    // they arrive in six trips, one behind the other - a microsecond of a 15 us launch); the offsets of a grouped launch
    // are picked from registers for the same reason.
    asm volatile("" ::"s"(g.A), "s"(g.B), "s"(g.C), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.a_bs), "s"(g.b_bs), "s"(g.c_bs),
                 "s"(g.groups), "s"(g.lda), "s"(g.ldb), "s"(g.tiles_n), "s"(g.tri), "s"(g.a_off[0]), "s"(g.a_off[1]),
                 "s"(g.a_off[2]), "s"(g.a_off[3]), "s"(g.b_off[0]), "s"(g.b_off[1]), "s"(g.b_off[2]), "s"(g.b_off[3]),
                 "s"(g.c_off[0]), "s"(g.c_off[1]), "s"(g.c_off[2]), "s"(g.c_off[3]));
    const int tid = HV == 2 ? (int)(threadIdx.x & 255) : (int)threadIdx.x;      // the thread within its group
    const int wave = tid >> 6, lane = tid & 63;
    const int half = lane >> 5, ln = lane & 31;
    const int wm = wave >> 1, wn = wave & 1;
    int tile_m = blockIdx.x / g.tiles_n, tile_n = blockIdx.x % g.tiles_n, zb = blockIdx.z;
    if (g.tri == 1) {
        // The grid holds only the tiles that reach the diagonal (column tile <= row tile; TM == TN), row after row: rows
        // 0 .. t0 - 1 have 1, 2, .. t0 tiles (t0 = the smaller tile count), the rows after them all tiles_n.
        const int tiles_m = (g.M + TM - 1) / TM, t0 = min(tiles_m, g.tiles_n), tri_count = t0 * (t0 + 1) / 2;
        const int idx = blockIdx.x;
        if (idx < tri_count) {
            int m = (int)((__fsqrt_rn(8.0f * (float)idx + 1.0f) - 1.0f) * 0.5f);
            while (m * (m + 1) / 2 > idx) --m;
            while ((m + 1) * (m + 2) / 2 <= idx) ++m;
            tile_m = m;
            tile_n = idx - m * (m + 1) / 2;
        } else {
            tile_m = t0 + (idx - tri_count) / g.tiles_n;
            tile_n = (idx - tri_count) % g.tiles_n;
        }
    } else if (g.tri >= 2) {
        // The contraction length depends on the row tile.  Workgroups start in the order of their linear index (and go to
        // the chip's eight dies by that index modulo 8): column tile fastest, then the batch, the row tiles slowest and
        // from the longest contraction to the shortest - the dies get equal shares and the launch ends on its lightest work.
        const long long lin = (long long)blockIdx.z * gridDim.x + blockIdx.x;
        const int tiles_m = (g.M + TM - 1) / TM;
        tile_n = (int)(lin % g.tiles_n);
        zb = (int)((lin / g.tiles_n) % gridDim.z);
        const int rank = (int)(lin / ((long long)g.tiles_n * gridDim.z));
        tile_m = g.tri == 3 ? tiles_m - 1 - rank : rank;
    }
    const int m0 = tile_m * TM, n0 = tile_n * TN;
    auto pick = [&](const long long (&off)[4]) { return zb == 0 ? off[0] : zb == 1 ? off[1] : zb == 2 ? off[2] : off[3]; };
    const long long c_at = g.groups ? pick(g.c_off) : (long long)zb * g.c_bs;
    float *C = g.C + c_at;

    OpA opa;
    OpB opb;
    opa.init(As, g.A + (g.groups ? pick(g.a_off) : (long long)zb * g.a_bs), g.M, g.lda, m0, g.K, tid);
    opb.init(Bs, g.B + (g.groups ? pick(g.b_off) : (long long)zb * g.b_bs), g.N, g.ldb, n0, g.K, tid);

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int ktiles_all = (g.K + KT - 1) / KT;
    const int kh = ktiles_all / 2;      // HV != 0: where the second half of the contraction starts
    int kt_first = g.tri == 2 ? min(m0 / KT, ktiles_all) : 0;      // (a tile past the end reads as zeros)
    int ktiles = g.tri == 3 ? min(ktiles_all, (m0 + TM + KT - 1) / KT) : ktiles_all;
    if (HV == 2) {      // (no triangle forms here: both groups walk kh tiles and meet at the same barriers)
        if (grp == 0) ktiles = kh;
        else kt_first = kh;
    }
    f32x16 first_half[MI][NI];      // HV == 1: the sum over the first half, set aside at the middle
    if (HV == 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) first_half[0][0][r] = 0.f;
    }
    opa.template load<0>(kt_first);
    opb.template load<0>(kt_first);
    // The 64 x 64 form with an epilogue asks for its bias and residual values now, behind the first tile: requested in the
    // epilogue, they would add a trip to memory (the residual is the layer's input, long out of the caches) to a launch
    // that has nothing else left to do.  16 + 16 registers, which this form can spare.  So does the 128 x 128 form on K tiles
    // of 32 (64 + 8 registers; it runs two workgroups per CU and may use 256): its workgroups all end together, and the
    // residual then no longer shares the memory system with the burst of their stores.
    constexpr bool PRE = EPI && ((MI == 1 && NI == 1) || (MI == 2 && NI == 2 && KT == 32));
    f32x4 pre_bias[PRE ? NI : 1][4], pre_res[PRE ? MI : 1][PRE ? NI : 1][4];
    if (PRE) {
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int gn = n0 + wn * 32 * NI + j * 32 + 8 * q4 + 4 * half;
                pre_bias[j][q4] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (gn < g.N && grp == 0 && g.bias) pre_bias[j][q4] = *reinterpret_cast<const f32x4 *>(g.bias + gn);
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    const int gm = m0 + wm * 32 * MI + i * 32 + ln;
                    pre_res[i][j][q4] = f32x4{0.f, 0.f, 0.f, 0.f};
                    if (gm < g.M && gn < g.N && grp == 0 && g.residual)
                        pre_res[i][j][q4] = *reinterpret_cast<const f32x4 *>(g.residual + c_at + (long long)gm * g.N + gn);
                }
            }
    }
    if (SLOTS == 2) {
        // the second tile is requested with the first and both are waited for (they arrive together): entering the loop
        // with loads pending in another order than the loop's own made the compiler wait, at the head of every second
        // step, for loads that step does not need yet
        opa.template load<SLOTS - 1>(kt_first + 1);
        opb.template load<SLOTS - 1>(kt_first + 1);
        __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
    }
    opa.template store<0>(0, tid);
    opb.template store<0>(0, tid);
    // (with two register sets the loads and the LDS stores of a step are unconditional: a tile past the end reads as zeros
    // or as values nobody uses, and on straight-line code the compiler's wait before the stores covers exactly the older
    // set's loads - with the loads under a condition it waited for the newest ones too)
    __syncthreads();
    // one K step; the LDS buffer index is a compile-time constant (the loop below is unrolled by two) so that every LDS
    // address is a per-thread base plus a literal
    auto k_step = [&](const int kt, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        const bool more = kt + 1 < ktiles;
        if (SLOTS == 2) {      // tile kt + 1 is in the other register set already; set `buf` (tile kt, stored a step ago) is free
            opa.template load<(SLOTS == 2 ? buf : 0)>(kt + 2);
            opb.template load<(SLOTS == 2 ? buf : 0)>(kt + 2);
            __builtin_amdgcn_sched_barrier(0);      // the requests go out before the step's MFMAs, not after them
        } else if (more) { opa.template load<0>(kt + 1); opb.template load<0>(kt + 1); }
#pragma unroll
        for (int h2 = 0; h2 < KT / 16; ++h2) {
            f32x4 af[MI][2], bf[NI][2];
            if (!TA) {
#pragma unroll
                for (int i = 0; i < MI; ++i) opa.fragment(buf, wm * 32 * MI + i * 32 + ln, half, h2, af[i]);
            }
            if (TB) {
#pragma unroll
                for (int j = 0; j < NI; ++j) opb.fragment(buf, wn * 32 * NI + j * 32 + ln, half, h2, bf[j]);
            }
#pragma unroll
            for (int s8 = 0; s8 < 8; ++s8) {
                float av[MI], bv[NI];
#pragma unroll
                for (int i = 0; i < MI; ++i) av[i] = TA ? opa.word(buf, wm * 32 * MI + i * 32 + ln, half, h2, s8) : af[i][s8 >> 2][s8 & 3];
#pragma unroll
                for (int j = 0; j < NI; ++j) bv[j] = TB ? bf[j][s8 >> 2][s8 & 3] : opb.word(buf, wn * 32 * NI + j * 32 + ln, half, h2, s8);
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        // operands swapped: the accumulator is the TRANSPOSED tile (lane = row m, registers = columns n), so
                        // that a lane holds four consecutive columns and the epilogue moves 128 bits per access
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j], av[i], acc[i][j], 0, 0, 0);
            }
        }
        if (more || SLOTS == 2) { opa.template store<(SLOTS == 2 ? (buf ^ 1) : 0)>(buf ^ 1, tid); opb.template store<(SLOTS == 2 ? (buf ^ 1) : 0)>(buf ^ 1, tid); }
        __syncthreads();
    };
    if (HV == 1) {
        // Two loops with the first sum set aside between them (the launcher's rule makes kh even and keeps the triangle
        // forms away).  Set aside under a condition inside the step, the accumulator went through 32 selects per step,
        // each of which waits for the matrix pipe to drain: three such products in one launch 29.2 -> 32.0 us.
        int kt = kt_first;
        for (; kt + 1 < kh; kt += 2) {
            k_step(kt, std::integral_constant<int, 0>{});
            k_step(kt + 1, std::integral_constant<int, 1>{});
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) { first_half[0][0][r] = acc[0][0][r]; acc[0][0][r] = 0.f; }
        for (; kt + 1 < ktiles; kt += 2) {
            k_step(kt, std::integral_constant<int, 0>{});
            k_step(kt + 1, std::integral_constant<int, 1>{});
        }
    } else if (SLOTS == 2) {
        // The odd last step stands outside the loop: with an exit between the two steps of the body the compiler sees a way
        // from the first step back to the loop's head, and makes every first step wait for the loads the second one
        // issued - which is what the second register set is there to avoid.  (The 128 x 128 form keeps the plain loop:
        // peeled, [8192,1024]x[1024,1024] ran 135 instead of 132 us.)
        int kt = kt_first;
        for (; kt + 1 < ktiles; kt += 2) {
            k_step(kt, std::integral_constant<int, 0>{});
            k_step(kt + 1, std::integral_constant<int, 1>{});
        }
        if (kt < ktiles) k_step(kt, std::integral_constant<int, 0>{});
    } else {
        for (int kt = kt_first; kt < ktiles; kt += 2) {
            k_step(kt, std::integral_constant<int, 0>{});
            if (kt + 1 < ktiles) k_step(kt + 1, std::integral_constant<int, 1>{});
        }
    }

    if (HV == 1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][0][r] = first_half[0][0][r] + acc[0][0][r];
    }
    if (HV == 2) {      // the K loop ended on a barrier: the tiles are dead.  Group 1 hands its sum over, group 0 finishes.
        float *sums = gemm_lds + (wave * 16) * 64 + lane;
        if (grp == 1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sums[r * 64] = acc[0][0][r];
        }
        __syncthreads();
        if (grp == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][0][r] = acc[0][0][r] + sums[r * 64];
        }
    }
    // accumulator register r of a transposed 32x32 tile: row m = lane % 32, column n = 8*(r/4) + 4*half + r%4
    float ln_s = 0.f, ln_ss = 0.f;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int gm = m0 + wm * 32 * MI + i * 32 + ln;
        if (gm >= g.M || grp != 0) continue;
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int gn = n0 + wn * 32 * NI + j * 32 + 8 * q4 + 4 * half;
                if (gn >= g.N) continue;      // N is a multiple of 4: a quad is inside or outside as a whole
                float *cp = C + (long long)gm * g.N + gn;
                f32x4 val;
                val.x = g.alpha * acc[i][j][4 * q4 + 0]; val.y = g.alpha * acc[i][j][4 * q4 + 1];
                val.z = g.alpha * acc[i][j][4 * q4 + 2]; val.w = g.alpha * acc[i][j][4 * q4 + 3];
                if (g.beta != 0.f) {
                    const f32x4 old = *reinterpret_cast<const f32x4 *>(cp);
                    val.x = val.x + g.beta * old.x; val.y = val.y + g.beta * old.y;
                    val.z = val.z + g.beta * old.z; val.w = val.w + g.beta * old.w;
                }
                if (EPI) {
                    if (g.bias) {
                        const f32x4 bq = PRE ? pre_bias[PRE ? j : 0][q4] : *reinterpret_cast<const f32x4 *>(g.bias + gn);
                        val.x = __fadd_rn(val.x, bq.x); val.y = __fadd_rn(val.y, bq.y);
                        val.z = __fadd_rn(val.z, bq.z); val.w = __fadd_rn(val.w, bq.w);
                    }
                    if (g.act == 1) {
                        val.x = gelu_sigmoid(val.x); val.y = gelu_sigmoid(val.y);
                        val.z = gelu_sigmoid(val.z); val.w = gelu_sigmoid(val.w);
                    }
                    if (g.residual) {
                        const f32x4 rq = PRE ? pre_res[PRE ? i : 0][PRE ? j : 0][q4] : *reinterpret_cast<const f32x4 *>(g.residual + c_at + (long long)gm * g.N + gn);
                        val.x = __fadd_rn(val.x, rq.x); val.y = __fadd_rn(val.y, rq.y);
                        val.z = __fadd_rn(val.z, rq.z); val.w = __fadd_rn(val.w, rq.w);
                    }
                    if (g.ln_part) {
                        ln_s += (val.x + val.y) + (val.z + val.w);
                        ln_ss += (__fmul_rn(val.x, val.x) + __fmul_rn(val.y, val.y)) + (__fmul_rn(val.z, val.z) + __fmul_rn(val.w, val.w));
                    }
                }
                *reinterpret_cast<f32x4 *>(cp) = val;
            }
    }
    if (EPI) {
        if (g.ln_part) {   // the workgroup's pair: the lanes of a wavefront, then the four wavefronts in order
            ln_s = dl4s::wave_sum(ln_s);
            ln_ss = dl4s::wave_sum(ln_ss);
            // the K loop ended on a barrier: the tiles are dead (HV == 2: behind the 4096 floats of group 1's sum, which a
            // slower wavefront of group 0 may still be reading)
            float *pairs = gemm_lds + (HV == 2 ? 4096 : 0);
            if (lane == 0 && grp == 0) { pairs[2 * wave] = ln_s; pairs[2 * wave + 1] = ln_ss; }
            __syncthreads();
            if (tid == 0 && grp == 0) {
                const int item = tile_m / g.ln_tiles_m;
                const long long at = ((long long)item * g.ln_tiles_m + tile_m % g.ln_tiles_m) * g.tiles_n + tile_n;
                g.ln_part[2 * at] = ((pairs[0] + pairs[2]) + pairs[4]) + pairs[6];
                g.ln_part[2 * at + 1] = ((pairs[1] + pairs[3]) + pairs[5]) + pairs[7];
            }
        }
    }
}

// ---- Skinny products: few rows (a handful of tokens) against a whole weight matrix, e.g. the decoder's projections
// during greedy decoding (NN/Models/Transformer/Transformer.swift:118-137 re-runs the decoder on the prefix for every
// generated token).  The tiled kernels above would put such a product on a handful of workgroups of four wavefronts
// that each walk all of K, one latency-bound step after the other.  Here a workgroup of SKW wavefronts owns a
// 32 x 32 output block: each wavefront contracts one SKW-th of K straight from global memory (no staging: every
// element of B is used once), the partial blocks are added up in LDS in wavefront order, and the block is finished
// with alpha, beta and the fused Dense epilogue.  For very long K the contraction is also cut into S slices over
// workgroups, which write part[z][s][M][N]; a second small kernel then adds the slices in order and finishes.  No
// atomics anywhere: the same bits on every run.
// op(A) is rows x K with K contiguous; B is K x N (TB = false) or N x K (TB = true).  K % 4 == 0.
constexpr int SKW = 16;
template <bool TB>
__global__ __launch_bounds__(64 * SKW) void gemm_f32_skinny(GemmArgs g, float *__restrict__ part, int kslice, int nbn, int S) {
    __shared__ float red[SKW][32][32];
    // (every argument on the way to the first loads is asked for in one trip, the offsets of a grouped launch picked from
    // registers: see gemm_f32_mfma_fast)
    asm volatile("" ::"s"(g.A), "s"(g.B), "s"(g.C), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.a_bs), "s"(g.b_bs), "s"(g.c_bs),
                 "s"(g.groups), "s"(g.lda), "s"(g.ldb), "s"(g.a_off[0]), "s"(g.a_off[1]), "s"(g.a_off[2]), "s"(g.a_off[3]),
                 "s"(g.b_off[0]), "s"(g.b_off[1]), "s"(g.b_off[2]), "s"(g.b_off[3]), "s"(part), "s"(kslice), "s"(nbn), "s"(S));
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, ln = lane & 31;
    const int cb = blockIdx.x % nbn, rb = blockIdx.x / nbn, s = blockIdx.y, z = blockIdx.z;
    auto pick = [&](const long long (&off)[4]) { return z == 0 ? off[0] : z == 1 ? off[1] : z == 2 ? off[2] : off[3]; };
    const float *A = g.A + (g.groups ? pick(g.a_off) : (long long)z * g.a_bs);
    const float *B = g.B + (g.groups ? pick(g.b_off) : (long long)z * g.b_bs);
    const int m = rb * 32 + ln, n = cb * 32 + ln;
    const int share = kslice / SKW;   // a multiple of 8
    const int k_begin = s * kslice + wave * share;
    const int k_end = min(g.K, k_begin + share);
    const float *arow = A + (long long)min(m, g.M - 1) * g.lda;
    const int nc = min(n, g.N - 1);   // rows >= M and columns >= N compute on clamped addresses and are never stored
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    // One block = 8 of K: lanes 0..31 contract k = kb .. kb+3, lanes 32..63 k = kb+4 .. kb+7 (the order inside the
    // contraction is free as long as both operands use it).  Loads are unconditional - out-of-range rows, columns and
    // blocks read a valid address and are zeroed or dropped afterwards - and run one batch of SKU blocks ahead of the
    // MFMAs, so that a wavefront has up to 2 * SKU blocks in flight instead of waiting for each (a kernel starts on a cold
    // L2: every first touch pays the full memory latency, and little else limits these products).
    constexpr int SKU = 4;
    const int nblk = (k_end - k_begin + 7) / 8;
    if (nblk > 0) {
        auto fetch = [&](const int blk, f32x4 &a, f32x4 &b) {
            const int kb = k_begin + 8 * min(blk, nblk - 1);
            int k0 = kb + 4 * half;
            if (k0 >= k_end) k0 = kb;
            a = *reinterpret_cast<const f32x4 *>(arow + k0);
            if (TB) {
                b = *reinterpret_cast<const f32x4 *>(B + (long long)nc * g.ldb + k0);
            } else {
                const float *bp = B + (long long)k0 * g.ldb + nc;
                b.x = bp[0]; b.y = bp[g.ldb]; b.z = bp[2 * g.ldb]; b.w = bp[3 * g.ldb];
            }
        };
        auto contract = [&](const int base, const f32x4 (&a)[SKU], const f32x4 (&b)[SKU]) {
#pragma unroll
            for (int u = 0; u < SKU; ++u) {
                // blocks past the end contribute nothing (both operands zeroed: the clamped loads hold real data)
                const bool ok = base + u < nblk && k_begin + 8 * (base + u) + 4 * half < k_end;
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                const f32x4 av = ok ? a[u] : zero, bv = ok ? b[u] : zero;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, acc, 0, 0, 0);
            }
        };
        // two register sets taken in turn: the loads of one are in flight while the other is contracted
        f32x4 a0[SKU], b0[SKU], a1[SKU], b1[SKU];
#pragma unroll
        for (int u = 0; u < SKU; ++u) fetch(u, a0[u], b0[u]);
        for (int base = 0; base < nblk; base += 2 * SKU) {
            if (base + SKU < nblk) {
#pragma unroll
                for (int u = 0; u < SKU; ++u) fetch(base + SKU + u, a1[u], b1[u]);
            }
            contract(base, a0, b0);
            if (base + 2 * SKU < nblk) {
#pragma unroll
                for (int u = 0; u < SKU; ++u) fetch(base + 2 * SKU + u, a0[u], b0[u]);
            }
            if (base + SKU < nblk) contract(base + SKU, a1, b1);
        }
    }
    // accumulator register r: row 8*(r/4) + 4*half + r%4, column ln
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][8 * (r >> 2) + 4 * half + (r & 3)][ln] = acc[r];
    __syncthreads();
    const long long c_at = g.groups ? g.c_off[z] : (long long)z * g.c_bs;
    float *pz = part ? part + ((long long)z * S + s) * g.M * g.N : nullptr;
#pragma unroll
    for (int i = 0; i < 1024 / (64 * SKW); ++i) {
        const int e = tid + 64 * SKW * i, row = e >> 5, col = e & 31;
        const int gm = rb * 32 + row, gn = cb * 32 + col;
        if (gm < g.M && gn < g.N) {
            float sum = red[0][row][col];
#pragma unroll
            for (int w = 1; w < SKW; ++w) sum += red[w][row][col];
            const long long at = (long long)gm * g.N + gn;
            if (pz) {
                pz[at] = sum;
            } else {
                float *cp = g.C + c_at + at;
                float val = g.alpha * sum;
                if (g.beta != 0.f) val = val + g.beta * (*cp);
                if (g.bias) val = __fadd_rn(val, g.bias[gn]);
                if (g.act == 1) val = gelu_sigmoid(val);
                if (g.residual) val = __fadd_rn(val, g.residual[c_at + at]);
                *cp = val;
            }
        }
    }
}

// The same for products of at most 16 rows (a single token of cached decoding, the first steps of a prefix re-run): a
// workgroup owns a 16 x 16 output block and contracts with v_mfma_f32_16x16x4_f32.  A 32 x 32 block costs K/2 MFMAs of 64
// cycles whatever the row count - 4096 cycles per SIMD at K = 512, 1.7 us of the 5 us such a launch takes - and leaves
// N/32 workgroups; here the block costs K/4 MFMAs of 32 cycles (1024 cycles per SIMD) on N/16 workgroups.
// One block = 16 of K: the 16-lane group q of a wavefront contracts k = kb + 4q .. kb + 4q + 3.
template <bool TB>
__global__ __launch_bounds__(64 * SKW) void gemm_f32_skinny16(GemmArgs g, float *__restrict__ part, int kslice, int nbn, int S) {
    __shared__ float red[SKW][16][16];
    // (every argument on the way to the first loads is asked for in one trip, the offsets of a grouped launch picked from
    // registers: see gemm_f32_mfma_fast)
    asm volatile("" ::"s"(g.A), "s"(g.B), "s"(g.C), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.a_bs), "s"(g.b_bs), "s"(g.c_bs),
                 "s"(g.groups), "s"(g.lda), "s"(g.ldb), "s"(g.a_off[0]), "s"(g.a_off[1]), "s"(g.a_off[2]), "s"(g.a_off[3]),
                 "s"(g.b_off[0]), "s"(g.b_off[1]), "s"(g.b_off[2]), "s"(g.b_off[3]), "s"(part), "s"(kslice), "s"(nbn), "s"(S));
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, q = lane >> 4, ln = lane & 15;
    const int cb = blockIdx.x % nbn, rb = blockIdx.x / nbn, s = blockIdx.y, z = blockIdx.z;
    auto pick = [&](const long long (&off)[4]) { return z == 0 ? off[0] : z == 1 ? off[1] : z == 2 ? off[2] : off[3]; };
    const float *A = g.A + (g.groups ? pick(g.a_off) : (long long)z * g.a_bs);
    const float *B = g.B + (g.groups ? pick(g.b_off) : (long long)z * g.b_bs);
    const int m = rb * 16 + ln, n = cb * 16 + ln;
    const int share = kslice / SKW;   // a multiple of 16
    const int k_begin = s * kslice + wave * share;
    const int k_end = min(g.K, k_begin + share);
    const float *arow = A + (long long)min(m, g.M - 1) * g.lda;
    const int nc = min(n, g.N - 1);   // rows >= M and columns >= N compute on clamped addresses and are never stored
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    constexpr int SKU = 2;
    const int nblk = (k_end - k_begin + 15) / 16;
    if (nblk > 0) {
        auto fetch = [&](const int blk, f32x4 &a, f32x4 &b) {
            const int kb = k_begin + 16 * min(blk, nblk - 1);
            int k0 = kb + 4 * q;
            if (k0 >= k_end) k0 = kb;
            a = *reinterpret_cast<const f32x4 *>(arow + k0);
            if (TB) {
                b = *reinterpret_cast<const f32x4 *>(B + (long long)nc * g.ldb + k0);
            } else {
                const float *bp = B + (long long)k0 * g.ldb + nc;
                b.x = bp[0]; b.y = bp[g.ldb]; b.z = bp[2 * g.ldb]; b.w = bp[3 * g.ldb];
            }
        };
        auto contract = [&](const int base, const f32x4 (&a)[SKU], const f32x4 (&b)[SKU]) {
#pragma unroll
            for (int u = 0; u < SKU; ++u) {
                // blocks past the end contribute nothing (both operands zeroed: the clamped loads hold real data)
                const bool ok = base + u < nblk && k_begin + 16 * (base + u) + 4 * q < k_end;
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                const f32x4 av = ok ? a[u] : zero, bv = ok ? b[u] : zero;
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, bv.x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, bv.y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, bv.z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, bv.w, acc, 0, 0, 0);
            }
        };
        f32x4 a0[SKU], b0[SKU], a1[SKU], b1[SKU];
#pragma unroll
        for (int u = 0; u < SKU; ++u) fetch(u, a0[u], b0[u]);
        for (int base = 0; base < nblk; base += 2 * SKU) {
            if (base + SKU < nblk) {
#pragma unroll
                for (int u = 0; u < SKU; ++u) fetch(base + SKU + u, a1[u], b1[u]);
            }
            contract(base, a0, b0);
            if (base + 2 * SKU < nblk) {
#pragma unroll
                for (int u = 0; u < SKU; ++u) fetch(base + 2 * SKU + u, a0[u], b0[u]);
            }
            if (base + SKU < nblk) contract(base + SKU, a1, b1);
        }
    }
    // accumulator register r: row 4*q + r, column ln
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * q + r][ln] = acc[r];
    __syncthreads();
    if (tid < 256) {
        const int row = tid >> 4, col = tid & 15;
        const int gm = rb * 16 + row, gn = cb * 16 + col;
        if (gm < g.M && gn < g.N) {
            float sum = red[0][row][col];
#pragma unroll
            for (int w = 1; w < SKW; ++w) sum += red[w][row][col];
            const long long c_at = g.groups ? g.c_off[z] : (long long)z * g.c_bs;
            const long long at = (long long)gm * g.N + gn;
            if (part) {
                part[((long long)z * S + s) * g.M * g.N + at] = sum;
            } else {
                float *cp = g.C + c_at + at;
                float val = g.alpha * sum;
                if (g.beta != 0.f) val = val + g.beta * (*cp);
                if (g.bias) val = __fadd_rn(val, g.bias[gn]);
                if (g.act == 1) val = gelu_sigmoid(val);
                if (g.residual) val = __fadd_rn(val, g.residual[c_at + at]);
                *cp = val;
            }
        }
    }
}


__global__ __launch_bounds__(256) void gemm_f32_skinny_finish(GemmArgs g, const float *__restrict__ part, int S) {
    const long long mn = (long long)g.M * g.N;
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    const int z = blockIdx.z;
    if (e >= mn) return;
    const float *pz = part + (long long)z * S * mn + e;
    float sum = 0.f;   // slices in order, eight loads in flight at a time
    for (int s0 = 0; s0 < S; s0 += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = pz[(long long)min(s0 + i, S - 1) * mn];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < S) sum = (s0 + i == 0) ? v[i] : sum + v[i];
    }
    const long long c_at = g.groups ? g.c_off[z] : (long long)z * g.c_bs;
    float *cp = g.C + c_at + e;
    float val = g.alpha * sum;
    if (g.beta != 0.f) val = val + g.beta * (*cp);
    const long long gm = e / g.N;
    const int gn = (int)(e - gm * g.N);
    if (g.bias) val = __fadd_rn(val, g.bias[gn]);
    if (g.act == 1) val = gelu_sigmoid(val);
    if (g.residual) val = __fadd_rn(val, g.residual[c_at + e]);
    *cp = val;
}

constexpr int GEMM_LN_NOT_FUSED = 1;   // gemm_launch with ln_part: nothing was launched, the caller takes the two-call route
constexpr int LN_MAX_PAIRS = 256;      // partial pairs per item that dl4s::layernorm_apply sums (one per thread)

int gemm_launch(dl4s_hip_ctx *ctx, const float *lhs, int64_t lr, int64_t lc, int64_t lbs, const float *rhs, int64_t rr,
                int64_t rc, int64_t rbs, float *result, int64_t cbs, int64_t batch, float alpha, float beta, int ta, int tb,
                const float *bias = nullptr, const float *residual = nullptr, int act = 0, const float *const *group_lhs = nullptr,
                const float *const *group_rhs = nullptr, float *const *group_result = nullptr, float *ln_part = nullptr,
                int64_t ln_item_rows = 0, int *ln_nblk = nullptr, bool tiled_only = false, int tri = 0) {
    // group_*: `batch` (at most 4) products of one shape with unrelated operand addresses, in one launch
    // ln_part: also leave LayerNorm partial sums over items of ln_item_rows rows (see GemmArgs); *ln_nblk receives the
    // number of pairs per item.  A product that does not run on the tiled kernels with whole tiles per item, or would
    // leave more pairs than ln_apply_f32 sums, is not launched at all: GEMM_LN_NOT_FUSED.
    DL4S_REQUIRE(lr >= 0 && lc >= 0 && rr >= 0 && rc >= 0 && batch >= 0, DL4S_HIP_EINVALID_ARG, "gemm: negative extent");
    const int64_t M = ta ? lc : lr, K = ta ? lr : lc;
    const int64_t K2 = tb ? rc : rr, N = tb ? rr : rc;
    DL4S_REQUIRE(K == K2, DL4S_HIP_ESHAPE, "gemm: inner dimensions differ (%lld vs %lld)", (long long)K, (long long)K2);
    if (M * N * batch == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(result && (K == 0 || (lhs && rhs)), DL4S_HIP_EINVALID_ARG, "gemm: NULL pointer");
    DL4S_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && batch <= 65535, DL4S_HIP_EUNSUPPORTED,
                 "gemm: extent too large");
    GemmArgs g{};
    g.A = lhs; g.B = rhs; g.C = result;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.a_rs = ta ? 1 : lc; g.a_cs = ta ? lc : 1;
    g.b_rs = tb ? 1 : rc; g.b_cs = tb ? rc : 1;
    g.a_bs = lbs; g.b_bs = rbs; g.c_bs = cbs;
    bool group_aligned = true;
    if (group_lhs) {
        g.groups = (int)batch;
        for (int i = 0; i < g.groups; ++i) {
            g.a_off[i] = group_lhs[i] - lhs;
            g.b_off[i] = group_rhs[i] - rhs;
            g.c_off[i] = group_result[i] - result;
            group_aligned = group_aligned && ((g.a_off[i] | g.b_off[i] | g.c_off[i]) & 3) == 0;
        }
    }
    g.lda = lc; g.ldb = rc;
    g.alpha = alpha; g.beta = beta;
    g.bias = bias; g.residual = residual; g.act = act;
    const bool epi = bias || residual || act || ln_part;   // the LayerNorm sums are part of the epilogue kernels
    const auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    // The fast kernels: every unit-stride extent a multiple of 4 (128-bit accesses), 16-byte aligned operands, and 32-bit
    // byte offsets below 2^31 (an operand stored rows x K is addressed within a tile's 128 rows, one stored K x rows as a whole).
    const auto rows_by_k_ok = [&](int64_t ld) { return K % 4 == 0 && ld < (1ll << 21); };
    const auto k_by_rows_ok = [&](int64_t extent, int64_t ld) { return extent % 4 == 0 && K * ld * 4 < (1ll << 31); };
    const bool fast = K > 0 && N % 4 == 0 && (ta ? k_by_rows_ok(M, lc) : rows_by_k_ok(lc)) && (tb ? rows_by_k_ok(rc) : k_by_rows_ok(N, rc)) &&
                      aligned16(lhs) && aligned16(rhs) && lbs % 4 == 0 && rbs % 4 == 0 && aligned16(result) && cbs % 4 == 0 &&
                      aligned16(bias) && aligned16(residual) && !(epi && (ta || tb)) && group_aligned;
    // Skinny products (see gemm_f32_skinny): up to 128 rows and too few 64 x 64 tiles to give every CU one, or any shape
    // with at most two 32 x 32 output blocks per CU (e.g. the weights . values product of one (batch, head) pair,
    // [512,512] . [512,64], which the reference issues pair by pair, Tensor/Operators/Matrix.swift:106-116): the tiled
    // kernels would run such a product one wavefront per SIMD or less.  Measured against the 64 x 64 tiles:
    // [512,512].[512,512] 6.6 against 14.5 us, [1024,512].[512,512] 11.1 against 14.7 us; from [2048,512].[512,512]
    // (1024 blocks) on the tiles win (16.6 against 21.0 us).  The rule looks at one product's shape only, so a product gets the same bits alone, in a batch, in a
    // group and with the fused Dense epilogue.
    const auto rows_by_k_any = [&](int64_t ld) { return K % 4 == 0 && ld % 4 == 0; };
    const bool few_rows = M <= 128 && ((M + 63) / 64) * ((N + 63) / 64) < ctx->cu_count;
    const bool few_blocks = ((M + 31) / 32) * ((N + 31) / 32) <= 2 * ctx->cu_count;
    // tiled_only: a caller inside the library with a batch that fills the GPU by itself (the skinny rule looks at one
    // product's shape, which says nothing about such a launch)
    const bool skinny = !tiled_only && !ta && K >= 64 && (few_rows || few_blocks) && rows_by_k_any(lc) &&
                        (tb ? rows_by_k_any(rc) : true) && aligned16(lhs) && (!tb || aligned16(rhs)) && lbs % 4 == 0 &&
                        (!tb || rbs % 4 == 0) && group_aligned && M * N * batch < (1ll << 31) && K * (tb ? 1 : rc) < (1ll << 31);
    if (ln_part && (skinny || !fast)) return GEMM_LN_NOT_FUSED;
    // (callers check their operands first; nothing has been launched when this fails)
    DL4S_REQUIRE(!tri || (fast && !skinny), DL4S_HIP_EUNSUPPORTED, "gemm: a triangular product on operands the tiled fast kernels do not take");
    g.tri = tri;
    if (skinny) {
        // 16 x 16 output blocks (gemm_f32_skinny16) for up to 16 rows, and beyond for an unsliced K while that grid stays
        // within two workgroups per CU ([32,512].[512,512] 5.7 -> 3.7 us, [128,512].[512,512] 5.8 -> 4.0 us,
        // [64,1024].[1024,1024] 10.6 -> 6.4 us); else 32 x 32 blocks ([32,512].[8000,512]^T: 8.5 us, against 11.3 us on a
        // thousand 16 x 16 blocks that read the weights twice; [96,2048].[2048,512] in slices: 9.5 against 12.8 us)
        const bool rows16 = M <= 16 || (K <= 1024 && ((M + 15) / 16) * ((N + 15) / 16) <= 2 * ctx->cu_count);
        const int blk = rows16 ? 16 : 32;
        const int nbn = (int)((N + blk - 1) / blk), nbm = (int)((M + blk - 1) / blk);
        // One slice up to K = 1024; beyond, slices of 512 (one batch of loads per wavefront), since a single workgroup per
        // column block pulls a long K through one CU: M16 N512 K2048 8.9 us against 15.3 us unsliced, K4096 8.9 against
        // 26.9.  The slicing depends on K alone, so a product gets the same summation order alone, batched and grouped.
        const int unit = (rows16 ? 16 : 8) * SKW;
        // (not more slices than it takes to give every CU two workgroups: with many column blocks the launch is wide
        // enough already, and a workgroup that lives for a single batch of loads spends its time starting and finishing)
        const long long want = (2ll * ctx->cu_count + (long long)nbn * nbm - 1) / ((long long)nbn * nbm);
        const long long S = K <= 1024 ? 1 : std::max(1ll, std::min((long long)((K + 511) / 512), want));
        const int kslice = (int)((((K + S - 1) / S) + unit - 1) / unit * unit);
        const dim3 pgrid((unsigned)(nbn * nbm), (unsigned)S, (unsigned)batch);
        const auto launch = [&](float *partials) {
            const int variant = (rows16 ? 2 : 0) | (tb ? 1 : 0);
#define DL4S_SKINNY(KERNEL) hipLaunchKernelGGL(KERNEL, pgrid, dim3(64 * SKW), 0, ctx->stream, g, partials, kslice, nbn, (int)S)
            switch (variant) {
                case 0: DL4S_SKINNY(gemm_f32_skinny<false>); break;
                case 1: DL4S_SKINNY(gemm_f32_skinny<true>); break;
                case 2: DL4S_SKINNY(gemm_f32_skinny16<false>); break;
                default: DL4S_SKINNY(gemm_f32_skinny16<true>); break;
            }
#undef DL4S_SKINNY
        };
        if (S == 1) {
            launch(nullptr);
            return dl4s::launch_status("gemm_f32_skinny");
        }
        std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
        const int rc_s = dl4s::ensure_scratch(ctx, (size_t)(batch * S * M * N) * sizeof(float));
        if (rc_s != DL4S_HIP_OK) return rc_s;
        float *part = static_cast<float *>(ctx->scratch);
        launch(part);
        hipLaunchKernelGGL(gemm_f32_skinny_finish, dim3((unsigned)((M * N + 255) / 256), 1, (unsigned)batch), dim3(256), 0, ctx->stream, g,
                           part, (int)S);
        return dl4s::launch_status("gemm_f32_skinny");
    }
    long long tm = (M + GBM - 1) / GBM, tn = (N + GBN - 1) / GBN;
    // Products of at most one 64 x 64 tile per CU with a long contraction (K a multiple of 128 from 256 on: two halves of
    // an even number of 32-deep tiles): alone, such a product runs one wavefront per SIMD, so its K tiles are summed in
    // two halves that two groups of wavefronts can work on side by side ([2048,512].[512,512]: 13.7 -> 13.0 us, with the
    // LayerNorm sums and the normalising pass 18.3 -> 17.4 us).  The rule looks at one product's shape only and fixes the
    // order of the additions; a batch or a group of such products that fills the GPU anyway runs the one-group form of
    // the same order.  (Callers inside the library with their own batches keep the plain order.)
    const long long t64 = ((M + 63) / 64) * ((N + 63) / 64);
    const bool halves = fast && !tiled_only && !tri && t64 <= ctx->cu_count && K >= 256 && K % 128 == 0;
    const int hv = !halves ? 0 : (t64 * batch <= ctx->cu_count ? 2 : 1);
    // small products: 64x64 tiles, so that there are at least about two workgroups per CU
    const bool small = fast && (halves || tm * tn * batch < 2ll * ctx->cu_count);
    if (small) { tm = (M + 63) / 64; tn = (N + 63) / 64; }
    g.tiles_n = (int)tn;
    if (ln_part) {
        const int64_t TM = small ? 64 : GBM;
        if (ln_item_rows <= 0 || ln_item_rows % TM != 0 || M % ln_item_rows != 0 || batch != 1 || (ln_item_rows / TM) * tn > LN_MAX_PAIRS)
            return GEMM_LN_NOT_FUSED;
        g.ln_part = ln_part;
        g.ln_tiles_m = (int)(ln_item_rows / TM);
        *ln_nblk = (int)((ln_item_rows / TM) * tn);
    }
    DL4S_REQUIRE(tm * tn < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "gemm: too many tiles");
    // (tri == 1: only the tiles that reach the diagonal, see the kernel)
    const long long t0 = std::min(tm, tn);
    const dim3 grid((unsigned)(tri == 1 ? t0 * (t0 + 1) / 2 + (tm - t0) * tn : tm * tn), 1, (unsigned)batch);
    // 128 x 128 tiles on a launch of at most two workgroups per CU: K tiles of 32 (half the barriers; contracted as two
    // halves of 16, so the bits do not depend on the depth)
    const bool deep = fast && !small && tm * tn * batch <= 2ll * ctx->cu_count;
#define DL4S_GEMM_FAST_KT(MI_, EPI_, TA_, TB_, KT_, HV_)                                                                              \
    do {                                                                                                                              \
        constexpr size_t lds_bytes = (HV_ == 2 ? 2 : 1) * (FastOperand<MI_, TA_, KT_>::LDS_FLOATS + FastOperand<MI_, !TB_, KT_>::LDS_FLOATS) * sizeof(float); \
        if (lds_bytes > 65536) {                                                                                                      \
            constexpr int which = (EPI_ ? 4 : 0) + (TA_ ? 2 : 0) + (TB_ ? 1 : 0);                                                     \
            constexpr int family = HV_ == 2 ? dl4s::LDS_GEMM_HALVES : dl4s::LDS_GEMM_DEEP;                                            \
            if (dl4s::lds_limit_pending(ctx, family, which)) {                                                                        \
                DL4S_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_f32_mfma_fast<MI_, MI_, EPI_, TA_, TB_, KT_, HV_>), \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));                        \
                dl4s::lds_limit_done(ctx, family, which);                                                                             \
            }                                                                                                                         \
        }                                                                                                                             \
        hipLaunchKernelGGL((gemm_f32_mfma_fast<MI_, MI_, EPI_, TA_, TB_, KT_, HV_>), grid, dim3(HV_ == 2 ? 512 : 256), lds_bytes,     \
                           ctx->stream, g);                                                                                           \
    } while (0)
#define DL4S_GEMM_FAST(MI_, EPI_, TA_, TB_)                                                   \
    do {                                                                                      \
        if (MI_ == 1 && hv == 2) DL4S_GEMM_FAST_KT(1, EPI_, TA_, TB_, 32, 2);                 \
        else if (MI_ == 1 && hv == 1) DL4S_GEMM_FAST_KT(1, EPI_, TA_, TB_, 32, 1);            \
        else if (MI_ == 1 || deep) DL4S_GEMM_FAST_KT(MI_, EPI_, TA_, TB_, 32, 0);             \
        else DL4S_GEMM_FAST_KT(MI_, EPI_, TA_, TB_, 16, 0);                                   \
    } while (0)
    if (fast) {
        const int variant = (small ? 0 : 8) + (epi ? 4 : 0) + (ta ? 2 : 0) + (tb ? 1 : 0);
        switch (variant) {
            case 0: DL4S_GEMM_FAST(1, false, false, false); break;
            case 1: DL4S_GEMM_FAST(1, false, false, true); break;
            case 2: DL4S_GEMM_FAST(1, false, true, false); break;
            case 3: DL4S_GEMM_FAST(1, false, true, true); break;
            case 4: DL4S_GEMM_FAST(1, true, false, false); break;
            case 8: DL4S_GEMM_FAST(2, false, false, false); break;
            case 9: DL4S_GEMM_FAST(2, false, false, true); break;
            case 10: DL4S_GEMM_FAST(2, false, true, false); break;
            case 11: DL4S_GEMM_FAST(2, false, true, true); break;
            default: DL4S_GEMM_FAST(2, true, false, false); break;   // 12: epilogue forms are never transposed
        }
    }
#undef DL4S_GEMM_FAST
#undef DL4S_GEMM_FAST_KT
    else hipLaunchKernelGGL(gemm_f32_mfma, grid, dim3(256), 0, ctx->stream, g);
    return dl4s::launch_status("gemm_f32_mfma");
}

}  // namespace

namespace dl4s {

int gemm_batched_tiled(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols, int64_t lhs_stride, const float *rhs,
                       int64_t rhs_rows, int64_t rhs_cols, int64_t rhs_stride, float *result, int64_t result_stride, int64_t batch,
                       float alpha, float beta, int transpose_first, int transpose_second, int triangle) {
    return gemm_launch(ctx, lhs, lhs_rows, lhs_cols, lhs_stride, rhs, rhs_rows, rhs_cols, rhs_stride, result, result_stride, batch, alpha,
                       beta, transpose_first, transpose_second, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, 0, nullptr, true,
                       triangle);
}

}  // namespace dl4s

extern "C" {

int dl4s_hip_gemm_f32(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols, const float *rhs,
                      int64_t rhs_rows, int64_t rhs_cols, float *result, float alpha, float beta, int transpose_first,
                      int transpose_second) {
    DL4S_CHECK_CTX(ctx);
    return gemm_launch(ctx, lhs, lhs_rows, lhs_cols, 0, rhs, rhs_rows, rhs_cols, 0, result, 0, 1, alpha, beta,
                       transpose_first, transpose_second);
}

int dl4s_hip_gemm_batched_f32(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols, int64_t lhs_stride,
                              const float *rhs, int64_t rhs_rows, int64_t rhs_cols, int64_t rhs_stride, float *result,
                              int64_t result_stride, int64_t batch, float alpha, float beta, int transpose_first,
                              int transpose_second) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(lhs_stride >= 0 && rhs_stride >= 0 && result_stride >= 0, DL4S_HIP_EINVALID_ARG, "gemm: negative batch stride");
    return gemm_launch(ctx, lhs, lhs_rows, lhs_cols, lhs_stride, rhs, rhs_rows, rhs_cols, rhs_stride, result, result_stride,
                       batch, alpha, beta, transpose_first, transpose_second);
}

int dl4s_hip_gemm_grouped_f32(dl4s_hip_ctx *ctx, int count, const float *const *lhs, int64_t lhs_rows, int64_t lhs_cols,
                              const float *const *rhs, int64_t rhs_rows, int64_t rhs_cols, float *const *result, float alpha,
                              float beta, int transpose_first, int transpose_second) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(count >= 0 && count <= 4, DL4S_HIP_EINVALID_ARG, "gemm: a group holds at most 4 products, got %d", count);
    if (count == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(lhs && rhs && result, DL4S_HIP_EINVALID_ARG, "gemm: NULL pointer array");
    for (int i = 0; i < count; ++i)
        DL4S_REQUIRE(result[i] && lhs[i] && rhs[i], DL4S_HIP_EINVALID_ARG, "gemm: NULL pointer in group entry %d", i);
    return gemm_launch(ctx, lhs[0], lhs_rows, lhs_cols, 0, rhs[0], rhs_rows, rhs_cols, 0, result[0], 0, count, alpha, beta,
                       transpose_first, transpose_second, nullptr, nullptr, 0, lhs, rhs, result);
}

int dl4s_hip_dense_fused_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t in_features, const float *weights,
                             int64_t out_features, const float *bias, int activation, const float *residual, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(activation == DL4S_ACT_NONE || activation == DL4S_ACT_GELU, DL4S_HIP_EINVALID_ARG,
                 "dense: unknown activation %d", activation);
    return gemm_launch(ctx, x, rows, in_features, 0, weights, in_features, out_features, 0, result, 0, 1, 1.0f, 0.0f, 0, 0, bias,
                       residual, activation);
}

// LayerNorm(act(x . weights + bias) + residual) over items of item_rows rows (NN/Layer/LayerNorm.swift:62-77 applied to
// the sum MultiHeadAttention.swift:120-124 forms): the product's epilogue leaves the per-tile sums, so the
// normalisation is one more pass instead of two.
int dl4s_hip_dense_layernorm_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t in_features, const float *weights,
                                 int64_t out_features, const float *bias, int activation, const float *residual,
                                 int64_t item_rows, const float *scale, const float *shift, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(activation == DL4S_ACT_NONE || activation == DL4S_ACT_GELU, DL4S_HIP_EINVALID_ARG,
                 "dense: unknown activation %d", activation);
    DL4S_REQUIRE(rows >= 0 && item_rows > 0 && rows % item_rows == 0, DL4S_HIP_ESHAPE,
                 "dense + layernorm: %lld rows are not whole items of %lld rows", (long long)rows, (long long)item_rows);
    DL4S_REQUIRE(scale && shift, DL4S_HIP_EINVALID_ARG, "dense + layernorm: NULL pointer");
    const int64_t items = rows / item_rows;
    const auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (rows * out_features > 0 && items <= 65535 && out_features % 4 == 0 && a16(scale) && a16(shift) && a16(result)) {
        std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
        int rc = dl4s::ensure_scratch(ctx, (size_t)items * LN_MAX_PAIRS * 2 * sizeof(float));
        if (rc != DL4S_HIP_OK) return rc;
        int nblk = 0;
        float *part = static_cast<float *>(ctx->scratch);
        rc = gemm_launch(ctx, x, rows, in_features, 0, weights, in_features, out_features, 0, result, 0, 1, 1.0f, 0.0f, 0, 0, bias, residual,
                         activation, nullptr, nullptr, nullptr, part, item_rows, &nblk);
        if (rc == DL4S_HIP_OK) return dl4s::layernorm_apply(ctx, result, scale, shift, result, part, items, item_rows * out_features, out_features, nblk);
        if (rc != GEMM_LN_NOT_FUSED) return rc;
    }
    const int rc = gemm_launch(ctx, x, rows, in_features, 0, weights, in_features, out_features, 0, result, 0, 1, 1.0f, 0.0f, 0, 0, bias,
                               residual, activation);
    if (rc != DL4S_HIP_OK) return rc;
    return dl4s_hip_layernorm_f32(ctx, result, nullptr, scale, shift, result, items, item_rows, out_features);
}

}  // extern "C"

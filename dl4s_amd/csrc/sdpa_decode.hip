// Single-query attention over a key/value cache (one decode step), split over the keys.
//
// The cache is [B,H,Tcap,d] fp32.  At d = 64 a 16-lane group reads one 256-byte key (or value) row with one
// 128-bit load per lane, so every load instruction of a wavefront covers four whole rows (1 KiB,
// contiguous), and a wavefront keeps the 8 K loads and 8 V loads of a 32-key block in flight together.
// The dot product is reduced inside the 16-lane group with DPP adds.  Rows of 32 and 128 floats use groups of 8 and
// 32 lanes in the same way (64 and 16 keys per iteration), rows of 96 floats groups of 8 lanes that read three pieces each
// (32 keys per iteration); other head dims run the next wider form with idle lanes, and a
// head dim that is no multiple of 4 (rows off the 16-byte grid) reads 64 or 32 bits per load.  With 16 wavefronts resident per CU
// that is ample memory-level parallelism to keep HBM busy.
//
// Work split: grid = (nsplit, B*H).  When B*H alone fills the GPU (the decode benchmark: 256 pairs on 256
// CUs) nsplit is 1, a 16-wavefront workgroup streams the whole cache row range of its pair and writes the
// output itself: ONE launch per step.  Otherwise the key range is split, every workgroup leaves
// (max, sum, 64 partial outputs) in a scratch record and a small second kernel merges the records of each
// pair with the usual softmax rescaling.  (A single-launch merge by the last workgroup to finish needs
// agent-scope release/acquire fences, i.e. an L2 write-back and invalidate per workgroup on gfx950, and ran
// an order of magnitude slower than the two launches.)
#include "common.h"

// Partial records of dl4s_hip_sdpa_decode_noalloc_f32: a fixed block in the code object's own device memory (one copy per
// GPU, held until the process ends), so that entry point never asks the driver for memory.  Host code must not pass this
// name to a kernel: it uses the device address hipGetSymbolAddress returns (dl4s::decode_static_scratch_init).
constexpr size_t NOALLOC_SCRATCH_FLOATS = size_t(1) << 20;   // 4 MiB
static __device__ __align__(256) float scratch[NOALLOC_SCRATCH_FLOATS];
// Held while the two launches of a split decode on the fixed block are enqueued, so that host threads cannot interleave
// them.  That orders calls of ONE context (one stream).  Calls of different contexts on one GPU run on different
// streams: g_static_scratch_user remembers the context that used the GPU's block last, and a call on another context
// makes its stream wait for that context's event first (events are created with the context: no allocation here).
// Replays of a recorded graph are outside this bookkeeping: their owner keeps them apart from other contexts' calls.
static std::mutex g_static_scratch_mu;
constexpr int MAX_DEVICES = 64;
static dl4s_hip_ctx *g_static_scratch_user[MAX_DEVICES];

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int MAXD = 256;                     // widest cache row the kernels take
constexpr float LOG2E = 1.44269504088896340736f;
// floats per partial record: o[0 .. D-1], m, l, pad (D = the row width the kernel instance covers: 32, 64 or 128)
constexpr int pstr(int D) { return D + 4; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
// Sum over the LPR (4, 8, 16 or 32) lanes that share a cache row; every one of them ends up with the total.
template <int LPR>
__device__ __forceinline__ float row_sum(float x) {
    x += dpp<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp<0x4E>(x);   // quad_perm [2,3,0,1]
    if (LPR >= 8) x += dpp<0x141>(x);  // row_half_mirror
    if (LPR >= 16) x += dpp<0x140>(x);  // row_mirror
    if (LPR >= 32) x += __shfl_xor(x, 16, 64);
    return x;
}

// Keys per lane and loop iteration of the decode kernel for rows read in `seg` pieces: as many as keep the two batches of
// loads (K, then V) of an iteration in registers at 128 per lane, the budget of 16 wavefronts per CU.  Three- and five-piece
// rows had 4 and 2 and spilled 18 and 15 registers inside the loop: with 3 and 1, B16 H16 T4096 went from 136 to 117 us at
// head dim 96 (5.9 -> 6.9 TB/s), 256 -> 232 us at 192, 145 -> 120 us at 80 and 217 -> 196 us at 160.
__host__ __device__ constexpr int keys_per_lane(int seg) { return seg == 1 ? 8 : seg == 2 ? 4 : seg == 3 ? 3 : 1; }

// LPR lanes read one cache row of up to 4 * LPR floats with one 128-bit load per lane (lanes at or beyond d / 4 hold
// zeros), so a load instruction of a wavefront covers G = 64 / LPR whole rows; a wavefront iteration covers KB = 8 * G
// keys with 8 K loads and 8 V loads per lane in flight (16 KiB per wavefront whatever the row width).
// NW wavefronts per workgroup; the wavefronts of a workgroup take KB-key blocks of the workgroup's key range
// [split*chunk, split*chunk + chunk) round-robin.  Inside a wavefront each LPR-lane group keeps its own running
// (max, sum, 4 output columns per lane), so the loop has no cross-lane traffic beyond the dot-product reduction;
// groups, wavefronts and (through the scratch records) workgroups are merged once at the end.
// FULL: the rows are exactly 4 * LPR floats long (no lane is idle, no load is predicated).
// DEVPOS: the row to append comes from device memory (*pos_dev) and T = row + 1, for callers that replay one recorded
// step at successive positions; a value outside [0, Tcap) leaves caches and output untouched.
// lengths (optional, one per batch element): keys at or beyond lengths[b] are blocked the way the reference blocks them,
// score - 1e9 (NN/Models/Transformer/ScaledDotProductAttention.swift:55-57 with the mask of makeEncoderMasks).  With at
// least one key left their weights are exactly zero and they are not visited at all; a length of zero or less blocks every
// key, the penalty is applied to all of them and the row comes out uniform, as in the reference.
// SEG: the row is read as SEG consecutive segments of 4 * LPR floats by the same LPR lanes (SEG loads per row and lane, fewer
// keys per lane and iteration, see keys_per_lane).  SEG = 3 with LPR = 8 (16) serves rows of 96 (192) floats with every lane
// busy, where the one-piece form would leave a quarter of the lanes idle; SEG = 5 with LPR = 4 (8) rows of 80 (160) floats;
// SEG = 2 with LPR = 32 serves rows of 129 to 256 floats.
template <bool APPEND, int NW, int LPR, bool FULL, bool DEVPOS = false, int SEG = 1>
__global__ __launch_bounds__(NW * 64) void sdpa_decode_splitk_f32(const float *__restrict__ q, float *kcache,
                                                                   float *vcache, const float *__restrict__ k_new,
                                                                   const float *__restrict__ v_new,
                                                                   float *__restrict__ out, float *part, int T, int Tcap,
                                                                   int pos, float rT, int nsplit, int chunk, int d, int H,
                                                                   const int *__restrict__ lengths,
                                                                   const int *__restrict__ pos_dev = nullptr, int vec = 4) {
    constexpr int SW = 4 * LPR, D = SW * SEG, G = 64 / LPR, NK = keys_per_lane(SEG), KB = NK * G, PSTR = pstr(D);
    __shared__ float sm_o[NW][D];
    __shared__ float sm_m[NW], sm_l[NW];
    if (DEVPOS) {
        pos = *pos_dev;
        if (pos < 0 || pos >= Tcap) return;   // uniform over the grid
        T = pos + 1;
    }
    const int split = blockIdx.x;
    const int bh = blockIdx.y;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane / LPR, c = lane % LPR;
    // FULL: d = D, every lane has its pieces of the row; else pieces beyond the row hold zeros
    // vec < 4: rows that are no whole number of 16-byte pieces, or operands that are not 16-byte aligned - a lane reads its
    // (up to) four columns as two 64-bit halves (even row length, 8-byte aligned operands) or one float at a time; the
    // wavefront's loads still cover whole contiguous rows.
    const bool vec4 = FULL || vec == 4;
    // p: the lane's piece of segment sg of a row (row base + SW * sg + 4 * c)
    auto load4 = [&](const float *p, const int sg) -> f32x4 {
        const int ncol = FULL ? 4 : d - SW * sg - 4 * c;
        f32x4 r = {0.f, 0.f, 0.f, 0.f};
        if (vec4) {
            if (ncol > 0) r = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
        } else if (vec == 2) {      // even row length: ncol is 2 or at least 4 wherever it is positive
            typedef float f32x2 __attribute__((ext_vector_type(2)));
            if (ncol > 0) { const f32x2 t = __builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(p)); r.x = t.x; r.y = t.y; }
            if (ncol > 2) { const f32x2 t = __builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(p + 2)); r.z = t.x; r.w = t.y; }
        } else {
            if (ncol > 0) r.x = __builtin_nontemporal_load(p);
            if (ncol > 1) r.y = __builtin_nontemporal_load(p + 1);
            if (ncol > 2) r.z = __builtin_nontemporal_load(p + 2);
            if (ncol > 3) r.w = __builtin_nontemporal_load(p + 3);
        }
        return r;
    };
    auto store4 = [&](float *p, const f32x4 r, const int sg) {
        const int ncol = FULL ? 4 : d - SW * sg - 4 * c;
        if (vec4) {
            if (ncol > 0) *reinterpret_cast<f32x4 *>(p) = r;
        } else if (vec == 2) {
            typedef float f32x2 __attribute__((ext_vector_type(2)));
            if (ncol > 0) *reinterpret_cast<f32x2 *>(p) = f32x2{r.x, r.y};
            if (ncol > 2) *reinterpret_cast<f32x2 *>(p + 2) = f32x2{r.z, r.w};
        } else {
            if (ncol > 0) p[0] = r.x;
            if (ncol > 1) p[1] = r.y;
            if (ncol > 2) p[2] = r.z;
            if (ncol > 3) p[3] = r.w;
        }
    };

    bool all_blocked = false;                 // a length of zero: every key takes the penalty
    if (lengths) {
        const int len = lengths[bh / H];
        if (len <= 0) all_blocked = true;
        else if (len < T) T = len;
    }

    f32x4 qv[SEG];
#pragma unroll
    for (int sg = 0; sg < SEG; ++sg) {
        qv[sg] = load4(q + (long long)bh * d + SW * sg + 4 * c, sg);
        qv[sg].x *= rT; qv[sg].y *= rT; qv[sg].z *= rT; qv[sg].w *= rT;
    }

    const long long base = (long long)bh * Tcap * d + 4 * c;
    const int c0 = split * chunk;
    const int c1 = min(T, c0 + chunk);
    // Row `pos` is the row being appended in this step: it is read from k_new / v_new (the cache does not
    // hold it yet) by selecting the ADDRESS per lane, so that all loads stay unconditional; one group of lanes
    // of the workgroup whose range holds the row writes it into the cache from its own copy.  (With lengths the
    // row may lie beyond the keys that are visited: the first workgroup of the pair writes it then.)
    const float *kn_row = nullptr, *vn_row = nullptr;
    if (APPEND) {
        kn_row = k_new + (long long)bh * d + 4 * c;
        vn_row = v_new + (long long)bh * d + 4 * c;
        const bool mine = (pos >= c0 && pos < c1) || (pos >= T && split == 0);
        if (mine && wave == 0 && g == 0) {
#pragma unroll
            for (int sg = 0; sg < SEG; ++sg) {
                store4(kcache + base + (long long)pos * d + SW * sg, load4(kn_row + SW * sg, sg), sg);
                store4(vcache + base + (long long)pos * d + SW * sg, load4(vn_row + SW * sg, sg), sg);
            }
        }
    }

    float m_run = -INFINITY, l_run = 0.f;
    f32x4 acc[SEG];
#pragma unroll
    for (int sg = 0; sg < SEG; ++sg) acc[sg] = f32x4{0.f, 0.f, 0.f, 0.f};
    // The wavefronts take the KB-key blocks of [c0, c1) round-robin, starting at a block that depends on the
    // (batch, head) pair: all workgroups run in lockstep, and without the rotation they would all be at the same
    // offset of their cache rows at the same time, which for some row strides (Tcap) lands on few HBM channels.
    const int nblk = (c1 - c0 + KB - 1) / KB;
    const int rot = nblk > 0 ? (int)(((unsigned)bh * 37u) % (unsigned)nblk) : 0;
    for (int bi = wave; bi < nblk; bi += NW) {
        int bb = bi + rot;
        if (bb >= nblk) bb -= nblk;
        const int kb = c0 + bb * KB;
        f32x4 kk[NK][SEG], vv[NK][SEG];
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int key = kb + G * i + g;
            const int kc = key < T ? key : T - 1;
            const float *kp = kcache + base + (long long)kc * d;
            if (APPEND) kp = (kc == pos) ? kn_row : kp;
#pragma unroll
            for (int sg = 0; sg < SEG; ++sg) kk[i][sg] = load4(kp + SW * sg, sg);
        }
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int key = kb + G * i + g;
            const int kc = key < T ? key : T - 1;
            const float *vp = vcache + base + (long long)kc * d;
            if (APPEND) vp = (kc == pos) ? vn_row : vp;
#pragma unroll
            for (int sg = 0; sg < SEG; ++sg) vv[i][sg] = load4(vp + SW * sg, sg);
        }
        if (kb + KB > c1) {     // the range's last block: lanes past its end re-read row T-1 and must add nothing, not 0 * Inf
#pragma unroll
            for (int i = 0; i < NK; ++i)
                if (kb + G * i + g >= c1) {
#pragma unroll
                    for (int sg = 0; sg < SEG; ++sg) vv[i][sg] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
        }
        float s[NK];
        float bm = -INFINITY;
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            float dot = qv[0].x * kk[i][0].x;
            dot += qv[0].y * kk[i][0].y;
            dot += qv[0].z * kk[i][0].z;
            dot += qv[0].w * kk[i][0].w;
#pragma unroll
            for (int sg = 1; sg < SEG; ++sg) {
                dot += qv[sg].x * kk[i][sg].x;
                dot += qv[sg].y * kk[i][sg].y;
                dot += qv[sg].z * kk[i][sg].z;
                dot += qv[sg].w * kk[i][sg].w;
            }
            dot = row_sum<LPR>(dot);
            if (all_blocked) dot = __fsub_rn(dot, 1e9f);
            if (kb + G * i + g >= c1) dot = -INFINITY;
            s[i] = dot;
            bm = fmaxf(bm, dot);
        }
        const float m_new = fmaxf(m_run, bm);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2((m_run - m_use) * LOG2E);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int sg = 0; sg < SEG; ++sg) { acc[sg].x *= alpha; acc[sg].y *= alpha; acc[sg].z *= alpha; acc[sg].w *= alpha; }
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const float p = fast_exp2((s[i] - m_use) * LOG2E);
            l_run += p;
#pragma unroll
            for (int sg = 0; sg < SEG; ++sg) {
                acc[sg].x += p * vv[i][sg].x; acc[sg].y += p * vv[i][sg].y; acc[sg].z += p * vv[i][sg].z; acc[sg].w += p * vv[i][sg].w;
            }
        }
    }
    // merge the G groups of the wavefront
    float mw = m_run;
#pragma unroll
    for (int o = LPR; o <= 32; o <<= 1) mw = fmaxf(mw, __shfl_xor(mw, o, 64));
    {
        const float mu = (mw == -INFINITY) ? 0.f : mw;
        const float f = fast_exp2((m_run - mu) * LOG2E);
        l_run *= f;
#pragma unroll
        for (int sg = 0; sg < SEG; ++sg) { acc[sg].x *= f; acc[sg].y *= f; acc[sg].z *= f; acc[sg].w *= f; }
    }
#pragma unroll
    for (int o = LPR; o <= 32; o <<= 1) {
        l_run += __shfl_xor(l_run, o, 64);
#pragma unroll
        for (int sg = 0; sg < SEG; ++sg) {
            acc[sg].x += __shfl_xor(acc[sg].x, o, 64); acc[sg].y += __shfl_xor(acc[sg].y, o, 64);
            acc[sg].z += __shfl_xor(acc[sg].z, o, 64); acc[sg].w += __shfl_xor(acc[sg].w, o, 64);
        }
    }
    if (g == 0) {
#pragma unroll
        for (int sg = 0; sg < SEG; ++sg) *reinterpret_cast<f32x4 *>(&sm_o[wave][SW * sg + 4 * c]) = acc[sg];
    }
    if (lane == 0) { sm_m[wave] = mw; sm_l[wave] = l_run; }
    __syncthreads();

    if (tid < D) {
        float M = sm_m[0];
#pragma unroll
        for (int w = 1; w < NW; ++w) M = fmaxf(M, sm_m[w]);
        const float Mu = (M == -INFINITY) ? 0.f : M;
        float L = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = fast_exp2((sm_m[w] - Mu) * LOG2E);
            L += sm_l[w] * f;
            O += sm_o[w][tid] * f;
        }
        if (nsplit == 1) {
            if (tid < d) out[(long long)bh * d + tid] = O * (1.0f / L);
        } else {
            float *rec = part + ((long long)bh * nsplit + split) * PSTR;
            rec[tid] = O;
            if (tid == 0) { rec[D] = M; rec[D + 1] = L; }
        }
    }
}

// Merges the partial records of one (batch, head): one thread per output column.
__global__ __launch_bounds__(MAXD) void sdpa_decode_merge_f32(const float *__restrict__ part, float *__restrict__ out,
                                                               int nsplit, int D, int d) {
    const int bh = blockIdx.x, tid = threadIdx.x;
    const int PSTR = pstr(D);
    const float *recs = part + (long long)bh * nsplit * PSTR;
    float M = -INFINITY;
    for (int sidx = 0; sidx < nsplit; ++sidx) M = fmaxf(M, recs[sidx * PSTR + D]);
    const float Mu = (M == -INFINITY) ? 0.f : M;
    float L = 0.f, O = 0.f;
    for (int sidx = 0; sidx < nsplit; ++sidx) {
        const float f = fast_exp2((recs[sidx * PSTR + D] - Mu) * LOG2E);
        L += recs[sidx * PSTR + D + 1] * f;
        if (tid < D) O += recs[sidx * PSTR + tid] * f;
    }
    if (tid < d) out[(long long)bh * d + tid] = O * (1.0f / L);
}

__global__ void kv_append_f32(float *kcache, float *vcache, const float *__restrict__ k_new,
                              const float *__restrict__ v_new, int pos, int Tcap, int d, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // over B*H*d
    if (i >= n) return;
    const long long bh = i / d;
    const int c = (int)(i % d);
    const long long dst = (bh * Tcap + pos) * d + c;
    kcache[dst] = k_new[i];
    vcache[dst] = v_new[i];
}

// Row widths the kernel is instantiated for: 32, 64, 128 floats (8, 16, 32 lanes per row, one 128-bit piece per lane), 96 and
// 192 floats (8 and 16 lanes per row, three pieces per lane), 80 and 160 floats (4 and 8 lanes per row, five pieces per lane)
// and 256 floats (32 lanes per row, two pieces per lane).
// (the three- and five-piece forms for exactly 96 / 192 and 80 / 160 floats and 128-bit pieces: with part-filled or narrower pieces its three loads per lane
// cost more than the idle lanes of the 128-float form - B16 H16 over 4096 rows: d = 96 163 -> 137 us, d = 80 160 -> 175 us)
inline int row_segments(int64_t d, int vec) {
    if (vec == 4 && (d == 96 || d == 192)) return 3;
    if (vec == 4 && (d == 80 || d == 160)) return 5;
    return d > 128 ? 2 : 1;
}
inline int lanes_per_row(int64_t d, int vec) {
    const int seg = row_segments(d, vec);
    return seg == 3 ? (int)d / 12 : (seg == 5 ? (int)d / 20 : (d <= 32 ? 8 : (d <= 64 ? 16 : 32)));
}
inline int row_width(int64_t d, int vec) { return 4 * lanes_per_row(d, vec) * row_segments(d, vec); }
inline int keys_per_iteration(int64_t d, int vec) { return keys_per_lane(row_segments(d, vec)) * (64 / lanes_per_row(d, vec)); }

// 4 when every cache row starts on a 16-byte boundary (the row length a multiple of 4 floats, every operand aligned): a lane
// reads its piece of a row with one 128-bit load.  2 for an even row length and 8-byte aligned operands (two 64-bit loads),
// 1 otherwise (one float at a time).
inline int row_vector_width(int64_t d, const void *q, const void *kcache, const void *vcache, const void *k_new, const void *v_new) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kcache) | reinterpret_cast<uintptr_t>(vcache) |
                           reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new);
    return (d % 4 == 0 && (bits & 15) == 0) ? 4 : ((d % 2 == 0 && (bits & 7) == 0) ? 2 : 1);
}

template <bool APPEND, int NW, int LPR, bool DEVPOS, int SEG = 1>
void decode_launch_kernel(dl4s_hip_ctx *ctx, dim3 grid, const float *q, float *kcache, float *vcache, const float *k_new,
                          const float *v_new, float *out, float *part, int T, int Tcap, int pos, float rT, int nsplit, int chunk,
                          int d, int H, const int *lengths, const int *pos_dev, int vec) {
    if (SEG == 3 || SEG == 5 || (d == 4 * LPR * SEG && vec == 4))      // the three- and five-piece forms are only chosen for full rows
        hipLaunchKernelGGL((sdpa_decode_splitk_f32<APPEND, NW, LPR, true, DEVPOS, SEG>), grid, dim3(NW * 64), 0, ctx->stream, q, kcache, vcache,
                           k_new, v_new, out, part, T, Tcap, pos, rT, nsplit, chunk, d, H, lengths, pos_dev, 4);
    else if constexpr (SEG != 3 && SEG != 5)
        hipLaunchKernelGGL((sdpa_decode_splitk_f32<APPEND, NW, LPR, false, DEVPOS, SEG>), grid, dim3(NW * 64), 0, ctx->stream, q, kcache, vcache,
                           k_new, v_new, out, part, T, Tcap, pos, rT, nsplit, chunk, d, H, lengths, pos_dev, vec);
}

template <bool APPEND, bool DEVPOS>
void decode_launch_width(dl4s_hip_ctx *ctx, int nw, dim3 grid, const float *q, float *kcache, float *vcache, const float *k_new,
                         const float *v_new, float *out, float *part, int T, int Tcap, int pos, float rT, int nsplit, int chunk,
                         int d, int H, const int *lengths, const int *pos_dev, int vec) {
#define DL4S_DECODE_ARGS ctx, grid, q, kcache, vcache, k_new, v_new, out, part, T, Tcap, pos, rT, nsplit, chunk, d, H, lengths, pos_dev, vec
    if (row_segments(d, vec) == 3 && d == 96) {
        if (nw == 16) decode_launch_kernel<APPEND, 16, 8, DEVPOS, 3>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 8, DEVPOS, 3>(DL4S_DECODE_ARGS);
    } else if (row_segments(d, vec) == 3) {
        if (nw == 16) decode_launch_kernel<APPEND, 16, 16, DEVPOS, 3>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 16, DEVPOS, 3>(DL4S_DECODE_ARGS);
    } else if (row_segments(d, vec) == 5 && d == 80) {
        if (nw == 16) decode_launch_kernel<APPEND, 16, 4, DEVPOS, 5>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 4, DEVPOS, 5>(DL4S_DECODE_ARGS);
    } else if (row_segments(d, vec) == 5) {
        if (nw == 16) decode_launch_kernel<APPEND, 16, 8, DEVPOS, 5>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 8, DEVPOS, 5>(DL4S_DECODE_ARGS);
    } else if (row_segments(d, vec) == 2) {
        if (nw == 16) decode_launch_kernel<APPEND, 16, 32, DEVPOS, 2>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 32, DEVPOS, 2>(DL4S_DECODE_ARGS);
    } else switch (lanes_per_row(d, vec)) {
        case 8: if (nw == 16) decode_launch_kernel<APPEND, 16, 8, DEVPOS>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 8, DEVPOS>(DL4S_DECODE_ARGS); break;
        case 16: if (nw == 16) decode_launch_kernel<APPEND, 16, 16, DEVPOS>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 16, DEVPOS>(DL4S_DECODE_ARGS); break;
        default: if (nw == 16) decode_launch_kernel<APPEND, 16, 32, DEVPOS>(DL4S_DECODE_ARGS); else decode_launch_kernel<APPEND, 4, 32, DEVPOS>(DL4S_DECODE_ARGS); break;
    }
#undef DL4S_DECODE_ARGS
}

int decode_launch(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache, const float *k_new,
                  const float *v_new, float *out, int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t pos,
                  int64_t d, float rT, bool append, const int32_t *lengths = nullptr, bool fixed_scratch = false) {
    const int64_t BH = B * H;
    if (BH == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(q && kcache && vcache && out, DL4S_HIP_EINVALID_ARG, "sdpa_decode: NULL tensor pointer");
    DL4S_REQUIRE(d >= 1 && d <= MAXD, DL4S_HIP_EUNSUPPORTED, "sdpa_decode: head dim %lld (1 to %d are implemented)", (long long)d, MAXD);
    const int vec = row_vector_width(d, q, kcache, vcache, k_new, v_new);
    DL4S_REQUIRE(T >= 1 && T <= Tcap, DL4S_HIP_ESHAPE, "sdpa_decode: T=%lld must be in [1, Tcap=%lld]", (long long)T,
                 (long long)Tcap);
    DL4S_REQUIRE(BH <= 65535 && Tcap < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa_decode: B*H=%lld above 65535", (long long)BH);
    const int KB = keys_per_iteration(d, vec);   // keys per wavefront iteration
    const int PSTR = pstr(row_width(d, vec));
    // Aim at 16 resident wavefronts on every CU.  Caches above 128 rows use 16-wavefront workgroups (between 512 and 2048
    // rows they had four: B16 H16 d64 over 600 rows 17.1 -> 13.0 us, 1536 rows 35.2 -> 30.2 us, B4 H16 d128 over 1536 rows
    // 27.2 -> 20.2 us - fewer, larger workgroups, and with 256 pairs no split and no merge launch at all); the key range is
    // split over several workgroups only when batch*heads alone does not fill the GPU.  Up to 512 rows one workgroup per
    // pair does it all: a second launch for the merge costs more than the split saves (B1 H8: 256 rows 6.4 -> 4.5 us,
    // 512 rows 6.5 -> 4.8 us).  The split follows T alone; with key lengths a workgroup whose share lies beyond its batch
    // element's length leaves an empty record.
    const bool short_cache = T <= 512;
    const int nw = T > 128 ? 16 : 4;
    const long long want_wg = ((long long)ctx->cu_count * 16 + nw - 1) / nw;
    long long max_split = short_cache ? 1 : (T + (long long)nw * KB - 1) / ((long long)nw * KB);
    long long ns = (want_wg + BH - 1) / BH;
    if (ns > max_split) ns = max_split;
    if (ns < 1) ns = 1;
    int chunk = (int)((T + ns - 1) / ns);
    chunk = (chunk + KB - 1) / KB * KB;
    const int nsplit = (int)((T + chunk - 1) / chunk);
    float *part = nullptr;
    std::unique_lock<std::mutex> scratch_lock(fixed_scratch ? g_static_scratch_mu : ctx->scratch_mu, std::defer_lock);
    if (nsplit > 1) {
        const size_t need = (size_t)BH * nsplit * PSTR;
        scratch_lock.lock();
        if (fixed_scratch) {
            DL4S_REQUIRE(ctx->static_scratch, DL4S_HIP_EHIP, "sdpa_decode_noalloc: the fixed scratch block has no device address");
            DL4S_REQUIRE(need <= NOALLOC_SCRATCH_FLOATS, DL4S_HIP_EUNSUPPORTED,
                         "sdpa_decode_noalloc: B*H=%lld pairs split %d ways need %zu bytes of partial records, the fixed block "
                         "holds %zu: use dl4s_hip_sdpa_decode_f32", (long long)BH, nsplit, need * sizeof(float),
                         NOALLOC_SCRATCH_FLOATS * sizeof(float));
            part = ctx->static_scratch;
            dl4s_hip_ctx *last = ctx->device < MAX_DEVICES ? g_static_scratch_user[ctx->device] : nullptr;
            if (last && last != ctx && !ctx->capturing) DL4S_HIP_TRY(hipStreamWaitEvent(ctx->stream, last->static_scratch_done, 0));
        } else {
            int rc = dl4s::ensure_scratch(ctx, need * sizeof(float));
            if (rc) return rc;
            part = reinterpret_cast<float *>(ctx->scratch);
        }
    }
    dim3 grid(nsplit, (unsigned)BH);
    if (append)
        decode_launch_width<true, false>(ctx, nw, grid, q, kcache, vcache, k_new, v_new, out, part, (int)T, (int)Tcap, (int)pos, rT, nsplit,
                                         chunk, (int)d, (int)H, lengths, nullptr, vec);
    else
        decode_launch_width<false, false>(ctx, nw, grid, q, kcache, vcache, k_new, v_new, out, part, (int)T, (int)Tcap, -1, rT, nsplit, chunk,
                                          (int)d, (int)H, lengths, nullptr, vec);
    int st = dl4s::launch_status("sdpa_decode_splitk_f32");
    if (st || nsplit == 1) return st;
    hipLaunchKernelGGL(sdpa_decode_merge_f32, dim3((unsigned)BH), dim3(MAXD), 0, ctx->stream, part, out, nsplit, row_width(d, vec), (int)d);
    st = dl4s::launch_status("sdpa_decode_merge_f32");
    if (st == DL4S_HIP_OK && fixed_scratch && !ctx->capturing && ctx->device < MAX_DEVICES) {
        DL4S_HIP_TRY(hipEventRecord(ctx->static_scratch_done, ctx->stream));
        g_static_scratch_user[ctx->device] = ctx;
    }
    return st;
}

}  // namespace

namespace dl4s {

// Device address of the fixed scratch block on the context's GPU (each GPU holds its own copy at its own address).
// Called by dl4s_hip_create with that GPU current.
int decode_static_scratch_init(dl4s_hip_ctx *ctx) {
    void *p = nullptr;
    DL4S_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    ctx->static_scratch = reinterpret_cast<float *>(p);
    DL4S_HIP_TRY(hipEventCreateWithFlags(&ctx->static_scratch_done, hipEventDisableTiming));
    return DL4S_HIP_OK;
}

// Called by dl4s_hip_destroy after the context's stream has drained.
void decode_static_scratch_release(dl4s_hip_ctx *ctx) {
    std::lock_guard<std::mutex> lock(g_static_scratch_mu);
    if (ctx->device < MAX_DEVICES && g_static_scratch_user[ctx->device] == ctx) g_static_scratch_user[ctx->device] = nullptr;
    if (ctx->static_scratch_done) (void)hipEventDestroy(ctx->static_scratch_done);
    ctx->static_scratch_done = nullptr;
}

}  // namespace dl4s

extern "C" {

int dl4s_hip_sdpa_decode_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache, float *out,
                             int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d, float inv_temperature) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode: negative extent");
    return decode_launch(ctx, q, const_cast<float *>(kcache), const_cast<float *>(vcache), nullptr, nullptr, out, B, H, T,
                         Tcap, -1, d, inv_temperature, false);
}

int dl4s_hip_sdpa_decode_lengths_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache, float *out,
                                     int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d, float inv_temperature,
                                     const int32_t *lengths) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode_lengths: negative extent");
    return decode_launch(ctx, q, const_cast<float *>(kcache), const_cast<float *>(vcache), nullptr, nullptr, out, B, H, T,
                         Tcap, -1, d, inv_temperature, false, lengths);
}

int dl4s_hip_sdpa_decode_noalloc_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache, float *out,
                                     int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d, float inv_temperature) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode_noalloc: negative extent");
    return decode_launch(ctx, q, const_cast<float *>(kcache), const_cast<float *>(vcache), nullptr, nullptr, out, B, H, T,
                         Tcap, -1, d, inv_temperature, false, nullptr, true);
}

int dl4s_hip_kv_append_f32(dl4s_hip_ctx *ctx, float *kcache, float *vcache, const float *k_new, const float *v_new,
                           int64_t B, int64_t H, int64_t pos, int64_t Tcap, int64_t d) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0 && d >= 0, DL4S_HIP_EINVALID_ARG, "kv_append: negative extent");
    const long long n = B * H * d;
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(kcache && vcache && k_new && v_new, DL4S_HIP_EINVALID_ARG, "kv_append: NULL tensor pointer");
    DL4S_REQUIRE(pos >= 0 && pos < Tcap, DL4S_HIP_ESHAPE, "kv_append: row %lld outside the cache capacity %lld",
                 (long long)pos, (long long)Tcap);
    hipLaunchKernelGGL(kv_append_f32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, kcache, vcache, k_new,
                       v_new, (int)pos, (int)Tcap, (int)d, n);
    return dl4s::launch_status("kv_append_f32");
}

int dl4s_hip_sdpa_decode_step_f32(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache, const float *k_new,
                                  const float *v_new, float *out, int64_t B, int64_t H, int64_t pos, int64_t Tcap,
                                  int64_t d, float inv_temperature) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode_step: negative extent");
    DL4S_REQUIRE(k_new && v_new, DL4S_HIP_EINVALID_ARG, "sdpa_decode_step: NULL new-row pointer");
    DL4S_REQUIRE(pos >= 0 && pos < Tcap, DL4S_HIP_ESHAPE, "sdpa_decode_step: row %lld outside the cache capacity %lld",
                 (long long)pos, (long long)Tcap);
    return decode_launch(ctx, q, kcache, vcache, k_new, v_new, out, B, H, pos + 1, Tcap, pos, d, inv_temperature, true);
}

int dl4s_hip_sdpa_decode_step_at_f32(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache, const float *k_new,
                                     const float *v_new, float *out, int64_t B, int64_t H, const int32_t *pos_dev, int64_t Tcap,
                                     int64_t d, float inv_temperature) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode_step_at: negative extent");
    const int64_t BH = B * H;
    if (BH == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(q && kcache && vcache && out && k_new && v_new && pos_dev, DL4S_HIP_EINVALID_ARG, "sdpa_decode_step_at: NULL pointer");
    DL4S_REQUIRE(d >= 1 && d <= MAXD, DL4S_HIP_EUNSUPPORTED,
                 "sdpa_decode_step_at: head dim %lld (1 to %d are implemented)", (long long)d, MAXD);
    const int vec = row_vector_width(d, q, kcache, vcache, k_new, v_new);
    DL4S_REQUIRE(Tcap >= 1 && Tcap < (1ll << 30) && BH <= 65535, DL4S_HIP_EUNSUPPORTED,
                 "sdpa_decode_step_at: capacity %lld or B*H=%lld out of range", (long long)Tcap, (long long)BH);
    // the row count is not known on the host: one workgroup per pair walks whatever rows there are (16 wavefronts, 4 for a
    // cache of up to 128 rows, where one block per wavefront covers it)
    const int KB = keys_per_iteration(d, vec);
    const int chunk = (int)((Tcap + KB - 1) / KB * KB);
    decode_launch_width<true, true>(ctx, Tcap > 128 ? 16 : 4, dim3(1, (unsigned)BH), q, kcache, vcache, k_new, v_new, out, nullptr, 0,
                                    (int)Tcap, 0, inv_temperature, 1, chunk, (int)d, (int)H, nullptr, pos_dev, vec);
    return dl4s::launch_status("sdpa_decode_splitk_f32");
}

}  // extern "C"

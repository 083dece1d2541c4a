// Engine primitives the attention layers call around the fused kernels: same-shape and broadcast
// binaries, unary maps, reductions, permuteAxes, band, stack, LayerNorm and bias+GELU.  All are
// HBM-bound streaming kernels: one pass, coalesced, grid-stride.
#include "common.h"

namespace {

constexpr int TPB = 256;

inline unsigned grid_for(long long n, int per_thread = 4) {
    long long b = (n + (long long)TPB * per_thread - 1) / ((long long)TPB * per_thread);
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return (unsigned)b;
}

enum { U_NEG, U_EXP, U_SQRT, U_RELU, U_TANH, U_LOG, U_SIN, U_COS };

// IEEE-exact fp32 square root (the device sqrtf is 1 ulp): the correctly rounded fp64 root rounds to the
// correctly rounded fp32 root because 53 >= 2*24 + 2.
__device__ __forceinline__ float sqrt_rn(float v) { return (float)sqrt((double)v); }


template <int OP>
__global__ void unary_f32(const float *__restrict__ x, float *__restrict__ y, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        float v = x[i], r;
        if (OP == U_NEG) r = -v;
        else if (OP == U_EXP) r = expf(v);
        else if (OP == U_SQRT) r = sqrt_rn(v);
        else if (OP == U_RELU) r = v > 0.f ? v : 0.f;
        else if (OP == U_LOG) r = logf(v);
        else if (OP == U_SIN) r = sinf(v);
        else if (OP == U_COS) r = cosf(v);
        else r = tanhf(v);
        y[i] = r;
    }
}

template <int OP>
__global__ void binary_f32(const float *a, const float *b, float *y, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        float r;
        if (OP == DL4S_OP_ADD) r = __fadd_rn(a[i], b[i]);
        else if (OP == DL4S_OP_SUB) r = __fsub_rn(a[i], b[i]);
        else if (OP == DL4S_OP_MUL) r = __fmul_rn(a[i], b[i]);
        else r = __fdiv_rn(a[i], b[i]);
        y[i] = r;
    }
}

__global__ void fill_f32(float v, float *y, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) y[i] = v;
}

struct Bcast {
    int dim;
    long long oshape[DL4S_HIP_MAX_DIM];
    long long ls[DL4S_HIP_MAX_DIM], rs[DL4S_HIP_MAX_DIM];  // element strides, 0 on broadcast axes
};

// mode: 0 element by element, 1 lhs is a scalar per slice, 2 rhs is a scalar per slice (Engine/CPU/CPUEngine.swift:117-176)
template <int OP>
__global__ void broadcast_f32(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ y, Bcast bc,
                              int mode, long long n) {
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long long)gridDim.x * blockDim.x) {
        long long rem = e, li = 0, ri = 0;
#pragma unroll 1
        for (int i = bc.dim - 1; i >= 0; --i) {
            const long long idx = rem % bc.oshape[i];
            rem /= bc.oshape[i];
            li += idx * bc.ls[i];
            ri += idx * bc.rs[i];
        }
        const float x = a[li], z = b[ri];
        float r;
        if (OP == DL4S_OP_ADD) r = __fadd_rn(x, z);
        else if (OP == DL4S_OP_MUL) r = __fmul_rn(x, z);
        else if (OP == DL4S_OP_SUB) {
            if (mode == 2) r = __fadd_rn(x, -z);             // x + (-s)
            else if (mode == 1) r = -__fadd_rn(z, -x);       // -(x + (-s))
            else r = __fsub_rn(x, z);
        } else {
            if (mode == 2) r = __fmul_rn(x, __fdiv_rn(1.0f, z));  // x * (1/s)
            else r = __fdiv_rn(x, z);
        }
        y[e] = r;
    }
}

// ---- reductions: one workgroup per output element, strided gather of the reduced elements
struct Reduce {
    int kdim, rdim;
    long long kshape[DL4S_HIP_MAX_DIM], kstride[DL4S_HIP_MAX_DIM];  // kept axes: extents and source strides
    long long rshape[DL4S_HIP_MAX_DIM], rstride[DL4S_HIP_MAX_DIM];  // reduced axes
    long long rcount;
};

// One workgroup per (output element, part): blockIdx.x = output, blockIdx.y = part of the reduced range
// [part * chunk, min(rcount, (part + 1) * chunk)); the result goes to y[output * gridDim.y + part].
template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void reduce_f32(const float *__restrict__ x, float *__restrict__ y, Reduce rd, long long chunk) {
    __shared__ float sm[TPB / 64];
    long long o = blockIdx.x, base = 0;
    for (int i = rd.kdim - 1; i >= 0; --i) {
        base += (o % rd.kshape[i]) * rd.kstride[i];
        o /= rd.kshape[i];
    }
    const long long j0 = (long long)blockIdx.y * chunk, j1 = min(rd.rcount, j0 + chunk);
    float acc = IS_MAX ? -INFINITY : 0.f;
    if (rd.rdim == 1) {     // one (merged) reduced axis: no index arithmetic beyond a multiply
        const long long rs = rd.rstride[0];
        for (long long j = j0 + threadIdx.x; j < j1; j += TPB) {
            const float v = x[base + j * rs];
            if (IS_MAX) acc = fmaxf(acc, v);   // NaN never selected, like the reference's "v > max" scan
            else acc += v;
        }
    } else {
        for (long long j = j0 + threadIdx.x; j < j1; j += TPB) {
            long long rem = j, off = base;
            for (int i = rd.rdim - 1; i >= 0; --i) {
                off += (rem % rd.rshape[i]) * rd.rstride[i];
                rem /= rd.rshape[i];
            }
            const float v = x[off];
            if (IS_MAX) acc = fmaxf(acc, v);
            else acc += v;
        }
    }
    for (int s = 32; s > 0; s >>= 1) {
        const float t = __shfl_xor(acc, s, 64);
        acc = IS_MAX ? fmaxf(acc, t) : acc + t;
    }
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = sm[0];
        for (int w = 1; w < TPB / 64; ++w) r = IS_MAX ? fmaxf(r, sm[w]) : r + sm[w];
        y[(long long)blockIdx.x * gridDim.y + blockIdx.y] = r;
    }
}

// Rows of a matrix reduced along their (contiguous) length, one wavefront per row: the reductions of a softmax over
// materialised scores ([B*H*L] rows of L keys) and of a per-token LayerNorm.  A workgroup per row leaves most of its
// threads with one or two elements and a block-wide merge for 2 KB of data (config 2's row maximum: 16 us for 34 MB).
template <bool IS_MAX>
__global__ __launch_bounds__(TPB) void reduce_rows_f32(const float *__restrict__ x, float *__restrict__ y, long long rows, int len) {
    const long long row = (long long)blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float *p = x + row * len;
    float acc = IS_MAX ? -INFINITY : 0.f;
    for (int j = lane; j < len; j += 64) {
        const float v = p[j];
        if (IS_MAX) acc = fmaxf(acc, v);
        else acc += v;
    }
    for (int s = 32; s > 0; s >>= 1) {
        const float t = __shfl_xor(acc, s, 64);
        acc = IS_MAX ? fmaxf(acc, t) : acc + t;
    }
    if (lane == 0) y[row] = acc;
}

struct Permute {
    int dim;
    long long sshape[DL4S_HIP_MAX_DIM];
    long long dstride[DL4S_HIP_MAX_DIM];  // destination stride for source axis i
};

__global__ void permute_f32(const float *__restrict__ x, float *__restrict__ y, Permute p, long long n) {
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long long)gridDim.x * blockDim.x) {
        long long rem = e, d = 0;
#pragma unroll 1
        for (int i = p.dim - 1; i >= 0; --i) {
            d += (rem % p.sshape[i]) * p.dstride[i];
            rem /= p.sshape[i];
        }
        y[d] = x[e];
    }
}

// Copy between a box of a row-major tensor and a contiguous buffer (the slice forms of get / set(slice:)).  The box is
// described after merging axes: `run` contiguous floats per piece, and the pieces' offsets in the tensor from up to
// DL4S_HIP_MAX_DIM outer axes (count, stride in floats).  READ: tensor -> buffer; else buffer -> tensor.
struct SliceBox {
    int dim;                                 // outer axes
    long long count[DL4S_HIP_MAX_DIM];
    long long stride[DL4S_HIP_MAX_DIM];
    long long run;                           // contiguous floats per piece
    long long base;                          // offset of the box's first element in the tensor
};
typedef float slice_f32x4 __attribute__((ext_vector_type(4)));
template <bool READ, int VEC>
__global__ void slice_copy_f32(const float *__restrict__ src, float *__restrict__ dst, SliceBox bx, long long n) {
    // n counts units of VEC floats; run is a multiple of VEC
    const long long run_units = bx.run / VEC;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long long)gridDim.x * blockDim.x) {
        long long piece = e / run_units;
        const long long within = (e - piece * run_units) * VEC;
        long long off = bx.base + within;
#pragma unroll 1
        for (int i = bx.dim - 1; i >= 0; --i) {
            off += (piece % bx.count[i]) * bx.stride[i];
            piece /= bx.count[i];
        }
        const long long lin = e * VEC;
        if (VEC == 4) {
            if (READ) *reinterpret_cast<slice_f32x4 *>(dst + lin) = *reinterpret_cast<const slice_f32x4 *>(src + off);
            else *reinterpret_cast<slice_f32x4 *>(dst + off) = *reinterpret_cast<const slice_f32x4 *>(src + lin);
        } else {
            if (READ) dst[lin] = src[off];
            else dst[off] = src[lin];
        }
    }
}

__global__ void band_f32(const float *__restrict__ x, float *__restrict__ y, long long rows, long long cols, long long below,
                         long long above) {
    const long long n = rows * cols;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long long)gridDim.x * blockDim.x) {
        const long long i = e / cols, j = e % cols;
        long long start = i - below; if (start < 0) start = 0; if (start > cols) start = cols;
        long long end = i + above + 1; if (end > cols) end = cols; if (end < start) end = start;
        if (j >= start && j < end) y[e] = x[e];
    }
}

// ---- LayerNorm over rows*D elements per batch item (NN/Layer/LayerNorm.swift:62-77)
template <int NT = TPB>
__device__ __forceinline__ void block_sum2(float &a, float &b, float *sm) {
    a = dl4s::wave_sum(a);
    b = dl4s::wave_sum(b);
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) { sm[2 * w] = a; sm[2 * w + 1] = b; }
    __syncthreads();
    a = 0.f; b = 0.f;
    for (int i = 0; i < NT / 64; ++i) { a += sm[2 * i]; b += sm[2 * i + 1]; }
}

// LayerNorm kernels.  VEC: rows, D and the pointers allow 128-bit accesses (n % 4 == 0, D % 4 == 0, 16-byte alignment);
// the arithmetic per element is the same either way.
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 ln_load4(const float *xp, const float *rp, long long i) {
    f32x4 v = *reinterpret_cast<const f32x4 *>(xp + i);
    if (rp) {
        const f32x4 r = *reinterpret_cast<const f32x4 *>(rp + i);
        v.x = __fadd_rn(v.x, r.x); v.y = __fadd_rn(v.y, r.y); v.z = __fadd_rn(v.z, r.z); v.w = __fadd_rn(v.w, r.w);
    }
    return v;
}

__device__ __forceinline__ f32x4 ln_norm4(f32x4 v, float mean, float rden, const f32x4 sc, const f32x4 sh) {
    f32x4 y;
    y.x = __fadd_rn(__fmul_rn(__fmul_rn(__fadd_rn(v.x, -mean), rden), sc.x), sh.x);
    y.y = __fadd_rn(__fmul_rn(__fmul_rn(__fadd_rn(v.y, -mean), rden), sc.y), sh.y);
    y.z = __fadd_rn(__fmul_rn(__fmul_rn(__fadd_rn(v.z, -mean), rden), sc.z), sh.z);
    y.w = __fadd_rn(__fmul_rn(__fmul_rn(__fadd_rn(v.w, -mean), rden), sc.w), sh.w);
    return y;
}

__device__ __forceinline__ f32x4 ln_norm4(f32x4 v, float mean, float rden, const float *scale, const float *shift, long long d) {
    return ln_norm4(v, mean, rden, *reinterpret_cast<const f32x4 *>(scale + d), *reinterpret_cast<const f32x4 *>(shift + d));
}

template <bool VEC>
__global__ __launch_bounds__(TPB) void ln_partial_f32(const float *__restrict__ x, const float *__restrict__ res,
                                                       float *__restrict__ part, long long n, int nblk) {
    __shared__ float sm[2 * TPB / 64];
    const long long b = blockIdx.y;
    const float *xp = x + b * n;
    const float *rp = res ? res + b * n : nullptr;
    float s = 0.f, ss = 0.f;
    if (VEC) {
        for (long long i = ((long long)blockIdx.x * TPB + threadIdx.x) * 4; i < n; i += (long long)nblk * TPB * 4) {
            const f32x4 v = ln_load4(xp, rp, i);
            s += (v.x + v.y) + (v.z + v.w);
            ss += (__fmul_rn(v.x, v.x) + __fmul_rn(v.y, v.y)) + (__fmul_rn(v.z, v.z) + __fmul_rn(v.w, v.w));
        }
    } else {
        for (long long i = (long long)blockIdx.x * TPB + threadIdx.x; i < n; i += (long long)nblk * TPB) {
            float v = xp[i];
            if (rp) v = __fadd_rn(v, rp[i]);
            s += v;
            ss += __fmul_rn(v, v);
        }
    }
    block_sum2(s, ss, sm);
    if (threadIdx.x == 0) { part[(b * nblk + blockIdx.x) * 2] = s; part[(b * nblk + blockIdx.x) * 2 + 1] = ss; }
}

template <bool VEC>
__global__ __launch_bounds__(TPB) void ln_apply_f32(const float *__restrict__ x, const float *__restrict__ res,
                                                     const float *__restrict__ scale, const float *__restrict__ shift,
                                                     float *__restrict__ y, const float *__restrict__ part, long long n,
                                                     long long D, int nblk) {
    __shared__ float sm[2 * TPB / 64];
    const long long b = blockIdx.y;
    const float *xp = x + b * n;
    const float *rp = res ? res + b * n : nullptr;
    float *yp = y + b * n;
    // Everything the block waits for is requested at once, the partial sums first: the pairs, the thread's first two
    // pieces (the launcher sizes the grid for two per thread) and their scale / shift values travel together while the
    // column indices are computed, instead of one trip to memory before the reduction and two behind it.
    // (The arguments likewise: fetched where the code first needs them, they arrive in five trips, one behind the other.)
    asm volatile("" ::"s"(x), "s"(res), "s"(scale), "s"(shift), "s"(y), "s"(part), "s"(n), "s"(D), "s"(nblk));
    // nblk <= TPB: one partial pair per thread, summed in a fixed order - up to 64 pairs by every wavefront for itself
    // (no exchange between the wavefronts, no barrier), more through LDS
    const int pair = nblk <= 64 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
    float s = 0.f, ss = 0.f;
    if (pair < nblk) {
        s = part[(b * nblk + pair) * 2];
        ss = part[(b * nblk + pair) * 2 + 1];
    }
    const long long step = (long long)gridDim.x * TPB * 4;
    long long i = ((long long)blockIdx.x * TPB + threadIdx.x) * 4;
    f32x4 pre[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (VEC) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
            if (i + u * step < n) pre[u] = ln_load4(xp, rp, i + u * step);
    }
    // the column of element i advances by a constant per iteration: no division in the loop (and 32-bit ones before it
    // wherever the item has fewer than 2^31 elements)
    long long d, dstep;
    if (n + step < (1ll << 31)) { d = (unsigned)i % (unsigned)D; dstep = (unsigned)step % (unsigned)D; }
    else { d = i % D; dstep = step % D; }
    f32x4 sc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, sh[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (VEC) {
        long long du = d;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (i + u * step < n) {
                sc[u] = *reinterpret_cast<const f32x4 *>(scale + du);
                sh[u] = *reinterpret_cast<const f32x4 *>(shift + du);
            }
            du += dstep;
            if (du >= D) du -= D;
        }
    }
    if (nblk <= 64) { s = dl4s::wave_sum(s); ss = dl4s::wave_sum(ss); }
    else block_sum2(s, ss, sm);
    const float rN = __fdiv_rn(1.0f, (float)n);
    const float mean = __fmul_rn(s, rN);
    const float var = __fsub_rn(__fmul_rn(ss, rN), __fmul_rn(mean, mean));
    const float rden = __fdiv_rn(1.0f, __fadd_rn(sqrt_rn(var), 1e-5f));
    if (VEC) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (i < n) *reinterpret_cast<f32x4 *>(yp + i) = ln_norm4(pre[u], mean, rden, sc[u], sh[u]);
            i += step;
            d += dstep;
            if (d >= D) d -= D;
        }
        for (; i < n; i += step) {
            *reinterpret_cast<f32x4 *>(yp + i) = ln_norm4(ln_load4(xp, rp, i), mean, rden, scale, shift, d);
            d += dstep;
            if (d >= D) d -= D;
        }
    } else {
        for (long long i = (long long)blockIdx.x * TPB + threadIdx.x; i < n; i += (long long)gridDim.x * TPB) {
            float v = xp[i];
            if (rp) v = __fadd_rn(v, rp[i]);
            const float c = __fadd_rn(v, -mean);
            const float nrm = __fmul_rn(c, rden);
            const long long d = i % D;
            yp[i] = __fadd_rn(__fmul_rn(nrm, scale[d]), shift[d]);
        }
    }
}

// ---- LayerNorm whose two sums are added in the reference's order (Engine/CPU/CPUEngine.swift:306-378 with the generic
// Float.sum, Engine/CPU/Numeric/CPUFloat.swift:239-261): every row of D elements is added left to right starting from
// zero, then the rows of an item are added to zero one after the other.  Such a sum has one rounding per element in a
// fixed sequence, so it cannot be spread over lanes: a lane owns a row.  A wavefront takes 64 rows and walks them in
// tiles of 64 columns, staged through LDS so that global memory is read 256 contiguous bytes per row (lane = column)
// while the additions run with lane = row (a row stride of 65 floats keeps the 64 lanes on 64 banks).
constexpr int LN_SEQ_ROWS = 64, LN_SEQ_COLS = 64, LN_SEQ_STRIDE = LN_SEQ_COLS + 1;

__global__ __launch_bounds__(64) void ln_row_sums_seq_f32(const float *__restrict__ x, const float *__restrict__ res,
                                                            float *__restrict__ part, long long R, long long D) {
    __shared__ float tile[LN_SEQ_ROWS * LN_SEQ_STRIDE];
    const int lane = threadIdx.x;
    const long long r0 = (long long)blockIdx.x * LN_SEQ_ROWS;
    const int nr = (int)(R - r0 < LN_SEQ_ROWS ? R - r0 : LN_SEQ_ROWS);
    float st[LN_SEQ_ROWS];
    auto load = [&](long long c0) {
        const long long c = c0 + lane;
#pragma unroll
        for (int i = 0; i < LN_SEQ_ROWS; ++i) {
            float v = 0.f;
            if (i < nr && c < D) {
                v = x[(r0 + i) * D + c];
                if (res) v = __fadd_rn(v, res[(r0 + i) * D + c]);
            }
            st[i] = v;
        }
    };
    float s = 0.f, ss = 0.f;
    load(0);
    for (long long c0 = 0; c0 < D; c0 += LN_SEQ_COLS) {
        __syncthreads();                  // the lanes are done with the tile before
#pragma unroll
        for (int i = 0; i < LN_SEQ_ROWS; ++i) tile[i * LN_SEQ_STRIDE + lane] = st[i];
        __syncthreads();
        if (c0 + LN_SEQ_COLS < D) load(c0 + LN_SEQ_COLS);       // in flight during the additions
        const float *row = tile + lane * LN_SEQ_STRIDE;
        if (D - c0 >= LN_SEQ_COLS) {
#pragma unroll
            for (int c = 0; c < LN_SEQ_COLS; ++c) {
                const float e = row[c];
                s = __fadd_rn(s, e);
                ss = __fadd_rn(ss, __fmul_rn(e, e));
            }
        } else {
            const int nc = (int)(D - c0);
            for (int c = 0; c < nc; ++c) {
                const float e = row[c];
                s = __fadd_rn(s, e);
                ss = __fadd_rn(ss, __fmul_rn(e, e));
            }
        }
    }
    if (lane < nr) { part[(r0 + lane) * 2] = s; part[(r0 + lane) * 2 + 1] = ss; }
}

// The same sums for rows that allow 128-bit accesses (D % 4 == 0, 16-byte aligned operands), with fewer rows per
// wavefront: the sums of a row are one chain of D dependent additions whoever runs it, so what a launch can win is
// the number of chains that run side by side - 2048 rows of 512 on wavefronts of 64 rows occupy 32 of the 1024 SIMDs
// (28.8 us), on wavefronts of 8 rows 256 of them.  A wavefront stages RW rows x 256 columns per step (all 64 lanes load
// and store, 16 bytes each; the next step's loads are in flight during the additions), then lanes 0 .. RW - 1 walk their
// rows left to right, four elements per LDS read.
template <int RW>
__global__ __launch_bounds__(64) void ln_row_sums_seq_vec_f32(const float *__restrict__ x, const float *__restrict__ res,
                                                                float *__restrict__ part, long long R, long long D) {
    constexpr int CT = 256, STRIDE = CT + 4;      // (a row stride of 260 floats: the RW lanes' 128-bit reads fall on distinct banks)
    __shared__ __align__(16) float tile[RW * STRIDE];
    const int lane = threadIdx.x;
    const long long r0 = (long long)blockIdx.x * RW;
    const int nr = (int)(R - r0 < RW ? R - r0 : RW);
    f32x4 st[RW];
    auto load = [&](long long c0) {
        const long long c = c0 + 4 * lane;
#pragma unroll
        for (int i = 0; i < RW; ++i) {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (i < nr && c < D) v = ln_load4(x, res, (r0 + i) * D + c);
            st[i] = v;
        }
    };
    float s = 0.f, ss = 0.f;
    load(0);
    for (long long c0 = 0; c0 < D; c0 += CT) {
        __syncthreads();                  // the lanes are done with the tile before
#pragma unroll
        for (int i = 0; i < RW; ++i) *reinterpret_cast<f32x4 *>(tile + i * STRIDE + 4 * lane) = st[i];
        __syncthreads();
        if (c0 + CT < D) load(c0 + CT);       // in flight during the additions
        if (lane < RW) {
            const float *row = tile + lane * STRIDE;
            const int nc = (int)(D - c0 < CT ? D - c0 : CT);
            auto add4 = [&](int c) {
                const f32x4 e = *reinterpret_cast<const f32x4 *>(row + c);
                s = __fadd_rn(s, e.x); ss = __fadd_rn(ss, __fmul_rn(e.x, e.x));
                s = __fadd_rn(s, e.y); ss = __fadd_rn(ss, __fmul_rn(e.y, e.y));
                s = __fadd_rn(s, e.z); ss = __fadd_rn(ss, __fmul_rn(e.z, e.z));
                s = __fadd_rn(s, e.w); ss = __fadd_rn(ss, __fmul_rn(e.w, e.w));
            };
            if (nc == CT) {
#pragma unroll
                for (int c = 0; c < CT; c += 4) add4(c);
            } else {
                for (int c = 0; c < nc; c += 4) add4(c);
            }
        }
    }
    if (lane < nr) { part[(r0 + lane) * 2] = s; part[(r0 + lane) * 2 + 1] = ss; }
}

// The rows of an item, one after the other: rowpart [items][rows][2] -> itempart [items][2].  One wavefront per item
// stages 512 rows' pairs at a time in LDS; lane 0 adds.
__global__ __launch_bounds__(64) void ln_item_sums_seq_f32(const float *__restrict__ rowpart, float *__restrict__ itempart, long long rows) {
    constexpr int CH = 512;
    __shared__ __align__(16) float sm[2 * CH];
    const int lane = threadIdx.x;
    const float *p = rowpart + (long long)blockIdx.x * rows * 2;
    float s = 0.f, ss = 0.f;
    for (long long r0 = 0; r0 < rows; r0 += CH) {
        const int cnt = (int)(rows - r0 < CH ? rows - r0 : CH);
        __syncthreads();
        for (int i = lane; i < 2 * cnt; i += 64) sm[i] = p[r0 * 2 + i];
        __syncthreads();
        if (lane == 0) {      // two rows' pairs per LDS read
            int i = 0;
#pragma unroll 8
            for (; i + 1 < cnt; i += 2) {
                const f32x4 e = *reinterpret_cast<const f32x4 *>(sm + 2 * i);
                s = __fadd_rn(s, e.x);
                ss = __fadd_rn(ss, e.y);
                s = __fadd_rn(s, e.z);
                ss = __fadd_rn(ss, e.w);
            }
            if (i < cnt) {
                s = __fadd_rn(s, sm[2 * i]);
                ss = __fadd_rn(ss, sm[2 * i + 1]);
            }
        }
    }
    if (lane == 0) { itempart[(long long)blockIdx.x * 2] = s; itempart[(long long)blockIdx.x * 2 + 1] = ss; }
}

// one workgroup (of NT threads: 256, or 1024 when a row is longer than 4096) per batch item, for short rows (per-token LayerNorm of the feed-forward block)
template <bool VEC, int NT>
__global__ __launch_bounds__(NT) void ln_small_f32(const float *__restrict__ x, const float *__restrict__ res,
                                                     const float *__restrict__ scale, const float *__restrict__ shift,
                                                     float *__restrict__ y, long long n, long long D) {
    __shared__ float sm[2 * NT / 64];
    const long long b = blockIdx.x;
    const float *xp = x + b * n;
    const float *rp = res ? res + b * n : nullptr;
    float *yp = y + b * n;
    float s = 0.f, ss = 0.f;
    if (VEC) {
        const bool one = n <= (long long)NT * 4;      // the whole row in one 128-bit access per thread: keep it in registers
        f32x4 keep = {0.f, 0.f, 0.f, 0.f};
        for (long long i = (long long)threadIdx.x * 4; i < n; i += (long long)NT * 4) {
            const f32x4 v = ln_load4(xp, rp, i);
            if (one) keep = v;
            s += (v.x + v.y) + (v.z + v.w);
            ss += (__fmul_rn(v.x, v.x) + __fmul_rn(v.y, v.y)) + (__fmul_rn(v.z, v.z) + __fmul_rn(v.w, v.w));
        }
        block_sum2<NT>(s, ss, sm);
        const float rN = __fdiv_rn(1.0f, (float)n);
        const float mean = __fmul_rn(s, rN);
        const float var = __fsub_rn(__fmul_rn(ss, rN), __fmul_rn(mean, mean));
        const float rden = __fdiv_rn(1.0f, __fadd_rn(sqrt_rn(var), 1e-5f));
        const long long step = (long long)NT * 4, dstep = step % D;
        long long i = (long long)threadIdx.x * 4, d = i % D;
        for (; i < n; i += step) {
            *reinterpret_cast<f32x4 *>(yp + i) = ln_norm4(one ? keep : ln_load4(xp, rp, i), mean, rden, scale, shift, d);
            d += dstep;
            if (d >= D) d -= D;
        }
    } else {
        for (long long i = threadIdx.x; i < n; i += NT) {
            float v = xp[i];
            if (rp) v = __fadd_rn(v, rp[i]);
            s += v;
            ss += __fmul_rn(v, v);
        }
        block_sum2<NT>(s, ss, sm);
        const float rN = __fdiv_rn(1.0f, (float)n);
        const float mean = __fmul_rn(s, rN);
        const float var = __fsub_rn(__fmul_rn(ss, rN), __fmul_rn(mean, mean));
        const float rden = __fdiv_rn(1.0f, __fadd_rn(sqrt_rn(var), 1e-5f));
        for (long long i = threadIdx.x; i < n; i += NT) {
            float v = xp[i];
            if (rp) v = __fadd_rn(v, rp[i]);
            const float nrm = __fmul_rn(__fadd_rn(v, -mean), rden);
            const long long d = i % D;
            yp[i] = __fadd_rn(__fmul_rn(nrm, scale[d]), shift[d]);
        }
    }
}

__global__ void bias_gelu_f32(const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ y, long long n,
                              long long D) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        float v = x[i];
        if (bias) v = __fadd_rn(v, bias[i % D]);
        const float a = __fmul_rn(v, 1.702f);
        const float t = tanhf(__fmul_rn(a, 0.5f));
        const float sg = __fadd_rn(__fmul_rn(0.5f, t), 0.5f);
        y[i] = __fmul_rn(v, sg);
    }
}

// The same for operands whose axes merge into at most three groups (outer, middle, inner), each group taken whole by
// both operands or broadcast whole by one of them - every broadcast of the attention path: scores - mask ([B,H,L,L] -
// [L,L]), x - max and x / sum ([.., L] against [.., 1]), LayerNorm's [B,L,D] against [B,1,1] and [D].  32-bit index
// arithmetic with two divisions per V elements (the general kernel spends two 64-bit divisions per axis and element:
// 2.4 TB/s on the mask subtraction of config 2), 128-bit accesses when the inner group allows.
// A_IN / B_IN: the operand runs along the inner group (else it is one value per inner row).  e2v = inner extent / V.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
template <int OP>
__device__ __forceinline__ float broadcast_op(const float x, const float z, const int mode) {
    if (OP == DL4S_OP_ADD) return __fadd_rn(x, z);
    if (OP == DL4S_OP_MUL) return __fmul_rn(x, z);
    if (OP == DL4S_OP_SUB) {
        if (mode == 2) return __fadd_rn(x, -z);             // x + (-s)
        if (mode == 1) return -__fadd_rn(z, -x);            // -(x + (-s))
        return __fsub_rn(x, z);
    }
    if (mode == 2) return __fmul_rn(x, __fdiv_rn(1.0f, z));  // x * (1/s)
    return __fdiv_rn(x, z);
}
template <int OP, int V, bool A_IN, bool B_IN>
__global__ void broadcast3_f32(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ y, unsigned e1,
                               unsigned e2v, unsigned sa0, unsigned sa1, unsigned sb0, unsigned sb1, int mode, unsigned nvec) {
    for (unsigned v = blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += gridDim.x * blockDim.x) {
        const unsigned i2 = v % e2v, t = v / e2v, i1 = t % e1, i0 = t / e1;
        const unsigned ao = i0 * sa0 + i1 * sa1 + (A_IN ? i2 * V : 0u), bo = i0 * sb0 + i1 * sb1 + (B_IN ? i2 * V : 0u);
        if (V == 4) {
            f32x4_t x, z, r;
            if (A_IN) x = *reinterpret_cast<const f32x4_t *>(a + ao);
            else { const float s = a[ao]; x = f32x4_t{s, s, s, s}; }
            if (B_IN) z = *reinterpret_cast<const f32x4_t *>(b + bo);
            else { const float s = b[bo]; z = f32x4_t{s, s, s, s}; }
            r.x = broadcast_op<OP>(x.x, z.x, mode); r.y = broadcast_op<OP>(x.y, z.y, mode);
            r.z = broadcast_op<OP>(x.z, z.z, mode); r.w = broadcast_op<OP>(x.w, z.w, mode);
            *reinterpret_cast<f32x4_t *>(y + (size_t)v * 4) = r;
        } else {
            y[v] = broadcast_op<OP>(a[ao], b[bo], mode);
        }
    }
}
template <int OP, int V>
void launch_broadcast3(hipStream_t stream, const int inner_type, const float *a, const float *b, float *y, unsigned e1, unsigned e2v,
                       unsigned sa0, unsigned sa1, unsigned sb0, unsigned sb1, int mode, unsigned nvec) {
    const dim3 g(grid_for((long long)nvec, 2)), blk(TPB);
    if (inner_type == 3) hipLaunchKernelGGL((broadcast3_f32<OP, V, true, true>), g, blk, 0, stream, a, b, y, e1, e2v, sa0, sa1, sb0, sb1, mode, nvec);
    else if (inner_type == 1) hipLaunchKernelGGL((broadcast3_f32<OP, V, true, false>), g, blk, 0, stream, a, b, y, e1, e2v, sa0, sa1, sb0, sb1, mode, nvec);
    else hipLaunchKernelGGL((broadcast3_f32<OP, V, false, true>), g, blk, 0, stream, a, b, y, e1, e2v, sa0, sa1, sb0, sb1, mode, nvec);
}
template <int OP>
int launch_unary(dl4s_hip_ctx *ctx, const float *x, float *y, int64_t n, const char *name) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(n >= 0, DL4S_HIP_EINVALID_ARG, "%s: negative count", name);
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(x && y, DL4S_HIP_EINVALID_ARG, "%s: NULL pointer", name);
    hipLaunchKernelGGL(unary_f32<OP>, dim3(grid_for(n)), dim3(TPB), 0, ctx->stream, x, y, (long long)n);
    return dl4s::launch_status(name);
}

template <int OP>
int launch_binary(dl4s_hip_ctx *ctx, const float *a, const float *b, float *y, int64_t n, const char *name) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(n >= 0, DL4S_HIP_EINVALID_ARG, "%s: negative count", name);
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(a && b && y, DL4S_HIP_EINVALID_ARG, "%s: NULL pointer", name);
    hipLaunchKernelGGL(binary_f32<OP>, dim3(grid_for(n)), dim3(TPB), 0, ctx->stream, a, b, y, (long long)n);
    return dl4s::launch_status(name);
}
// stack along axis 0: up to 64 equally sized source buffers per launch (their addresses travel as kernel arguments),
// blockIdx.y = buffer, the grid-stride loop copies 128 bits per thread where the addresses allow
struct StackSrc {
    const float *p[64];
};
__global__ void stack_f32(StackSrc src, float *__restrict__ dst, long long count, int vec) {
    const float *s = src.p[blockIdx.y];
    float *d = dst + (long long)blockIdx.y * count;
    const long long stride = (long long)gridDim.x * blockDim.x, i0 = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        const long long n4 = count >> 2;
        for (long long i = i0; i < n4; i += stride) reinterpret_cast<float4 *>(d)[i] = reinterpret_cast<const float4 *>(s)[i];
        for (long long i = (n4 << 2) + i0; i < count; i += stride) d[i] = s[i];
    } else {
        for (long long i = i0; i < count; i += stride) d[i] = s[i];
    }
}

// First index of the largest value, scanning like `if v > maxV` from (-inf, index 0): NaN is never selected, ties keep
// the earliest index (Engine/CPU/Numeric/CPUFloat.swift:294-318, generic branch).  One workgroup; out = {value, index}.
// out_token / counter (either may be NULL): the index as int32 and a counter advanced by one, both in device memory, for
// decoding loops that keep the chosen token and the position on the device
__global__ __launch_bounds__(1024) void argmax_f32(const float *__restrict__ x, long long n, float *out_value, long long *out_index,
                                                   int *out_token = nullptr, int *counter = nullptr) {
    __shared__ float sv[1024];
    __shared__ long long si[1024];
    float bv = -INFINITY;
    long long bi = 0;
    for (long long i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = x[i];
        if (v > bv) { bv = v; bi = i; }     // ascending i per thread: the first of equal values stays
    }
    sv[threadIdx.x] = bv;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int o = blockDim.x / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            const float v = sv[threadIdx.x + o];
            const long long i = si[threadIdx.x + o];
            // a candidate wins on a larger value, or on an equal value found earlier -- but never from the initial
            // state (-inf, 0) of a thread that selected nothing
            if (v > sv[threadIdx.x] || (v == sv[threadIdx.x] && v != -INFINITY && i < si[threadIdx.x])) {
                sv[threadIdx.x] = v;
                si[threadIdx.x] = i;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (out_value) *out_value = sv[0];
        if (out_index) *out_index = si[0];
        if (out_token) *out_token = (int)si[0];
        if (counter) *counter += 1;
    }
}

// One token whose id and position are in device memory: out[c] = table[token][c] * scale + pos[position][c].  A token
// outside [0, vocab) (the ignore index included) embeds as zeros; a position outside [0, pos_rows) adds nothing.
__global__ void embed_at_f32(const float *__restrict__ table, const int *__restrict__ token_dev, const float *__restrict__ pos,
                             const int *__restrict__ position_dev, float *__restrict__ out, long long vocab, long long D, long long pos_rows,
                             float scale, int has_scale) {
    const int tok = *token_dev;
    const int at = position_dev ? *position_dev : 0;
    for (long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x; c < D; c += (long long)gridDim.x * blockDim.x) {
        float v = (tok >= 0 && tok < vocab) ? table[(long long)tok * D + c] : 0.0f;
        if (has_scale) v = __fmul_rn(v, scale);
        if (pos && at >= 0 && at < pos_rows) v = __fadd_rn(v, pos[(long long)at * D + c]);
        out[c] = v;
    }
}

// Embedding lookup with the scale and positional term of Transformer.prepareInputs folded in:
// out[t][:] = (token[t] == ignore ? 0 : table[token[t]][:]) * scale + positions[t % L][:]
// A token outside [0, vocab) that is not the ignore index is a caller's mistake (the reference's subscript traps on it); the
// table is never read out of bounds for it: such a token embeds as a row of NaN, which no later step can hide.
__global__ void embed_positions_f32(const float *__restrict__ table, const int *__restrict__ tokens, const float *__restrict__ pos,
                                    float *__restrict__ out, long long ntok, long long L, long long D, long long vocab, int ignore,
                                    float scale, int has_scale) {
    const long long n = ntok * D;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const long long t = i / D, c = i % D;
        const int tok = tokens[t];
        float v = 0.0f;
        if (tok != ignore) v = (tok >= 0 && tok < vocab) ? table[(long long)tok * D + c] : __builtin_nanf("");
        if (has_scale) v = __fmul_rn(v, scale);
        if (pos) v = __fadd_rn(v, pos[(t % L) * D + c]);
        out[i] = v;
    }
}

// logSoftmax over the last axis, one workgroup per row: x - max, exp, sum, log, subtract
// (Tensor/Operators/Unary.swift:198-204).  The row sum is taken in index order by one thread per 256-element
// stripe and then across stripes, within the parity tolerance of the reference's sequential sum.
__global__ __launch_bounds__(256) void log_softmax_f32(const float *__restrict__ x, float *__restrict__ y, long long n) {
    __shared__ float red[256];
    const float *xr = x + (long long)blockIdx.x * n;
    float *yr = y + (long long)blockIdx.x * n;
    float mx = -INFINITY;
    for (long long i = threadIdx.x; i < n; i += 256) { const float v = xr[i]; if (v > mx) mx = v; }
    red[threadIdx.x] = mx;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) red[threadIdx.x] = red[threadIdx.x + o] > red[threadIdx.x] ? red[threadIdx.x + o] : red[threadIdx.x];
        __syncthreads();
    }
    mx = red[0];
    __syncthreads();
    float sum = 0.f;
    for (long long i = threadIdx.x; i < n; i += 256) sum += expf(__fadd_rn(xr[i], -mx));
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    const float lse = logf(red[0]);
    for (long long i = threadIdx.x; i < n; i += 256) yr[i] = __fsub_rn(__fadd_rn(xr[i], -mx), lse);
}

// Validates the box and merges axes: trailing axes taken whole join the contiguous run, the rest become outer axes.
int make_slice_box(const int64_t *shape, int dim, const int64_t *start, const int64_t *extent, SliceBox &bx, long long &total,
                   const char *what) {
    DL4S_REQUIRE(dim >= 0 && dim <= DL4S_HIP_MAX_DIM, DL4S_HIP_EINVALID_ARG, "%s: dim %d not in [0,%d]", what, dim, DL4S_HIP_MAX_DIM);
    DL4S_REQUIRE(dim == 0 || (shape && start && extent), DL4S_HIP_EINVALID_ARG, "%s: NULL shape / start / extent", what);
    long long strides[DL4S_HIP_MAX_DIM];
    long long s = 1;
    total = 1;
    for (int i = dim - 1; i >= 0; --i) {
        DL4S_REQUIRE(shape[i] >= 0 && start[i] >= 0 && extent[i] >= 0 && start[i] + extent[i] <= shape[i], DL4S_HIP_ESHAPE,
                     "%s: axis %d: [%lld, %lld) is not inside [0, %lld)", what, i, (long long)start[i], (long long)(start[i] + extent[i]),
                     (long long)shape[i]);
        strides[i] = s;
        s *= shape[i];
        total *= extent[i];
    }
    bx = SliceBox{};
    bx.run = 1;
    int i = dim - 1;
    for (; i >= 0; --i) {            // the run ends with the first axis (from the right) that is not taken whole
        bx.run *= extent[i];
        bx.base += start[i] * strides[i];
        if (extent[i] != shape[i]) { --i; break; }
    }
    for (int a = 0; a <= i; ++a) {   // outer axes, those of extent 1 only move the base
        bx.base += start[a] * strides[a];
        if (extent[a] == 1) continue;
        bx.count[bx.dim] = extent[a];
        bx.stride[bx.dim] = strides[a];
        ++bx.dim;
    }
    return DL4S_HIP_OK;
}

template <bool READ>
int launch_slice_copy(dl4s_hip_ctx *ctx, const float *src, float *dst, const SliceBox &bx, long long total, const float *tensor,
                      const float *buffer) {
    bool vec = bx.run % 4 == 0 && bx.base % 4 == 0 && ((reinterpret_cast<uintptr_t>(tensor) | reinterpret_cast<uintptr_t>(buffer)) & 15) == 0;
    for (int i = 0; i < bx.dim; ++i) vec = vec && bx.stride[i] % 4 == 0;
    if (vec) hipLaunchKernelGGL((slice_copy_f32<READ, 4>), dim3(grid_for(total / 4, 2)), dim3(TPB), 0, ctx->stream, src, dst, bx, total / 4);
    else hipLaunchKernelGGL((slice_copy_f32<READ, 1>), dim3(grid_for(total, 2)), dim3(TPB), 0, ctx->stream, src, dst, bx, total);
    return dl4s::launch_status(READ ? "subscriptRead" : "subscriptWrite");
}
}  // namespace

namespace dl4s {
int layernorm_apply(dl4s_hip_ctx *ctx, const float *x, const float *scale, const float *shift, float *y, const float *part,
                    long long items, long long n, long long D, int nblk) {
    DL4S_REQUIRE(nblk >= 1 && nblk <= TPB && items >= 1 && items <= 65535 && n % 4 == 0 && D % 4 == 0, DL4S_HIP_EINVALID_ARG,
                 "layernorm: bad partial-sum layout");
    const long long want = n / (TPB * 8);
    const unsigned gx = (unsigned)(want < 1 ? 1 : (want > 256 ? 256 : want));
    hipLaunchKernelGGL(ln_apply_f32<true>, dim3(gx, (unsigned)items), dim3(TPB), 0, ctx->stream, x, static_cast<const float *>(nullptr), scale,
                       shift, y, part, n, D, nblk);
    return launch_status("layernorm");
}
}  // namespace dl4s

extern "C" {

int dl4s_hip_fill_f32(dl4s_hip_ctx *ctx, float value, float *result, int64_t count) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(count >= 0, DL4S_HIP_EINVALID_ARG, "fill: negative count");
    if (count == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(result, DL4S_HIP_EINVALID_ARG, "fill: NULL pointer");
    hipLaunchKernelGGL(fill_f32, dim3(grid_for(count)), dim3(TPB), 0, ctx->stream, value, result, (long long)count);
    return dl4s::launch_status("fill");
}

int dl4s_hip_vadd_f32(dl4s_hip_ctx *c, const float *l, const float *r, float *y, int64_t n) { return launch_binary<DL4S_OP_ADD>(c, l, r, y, n, "vAdd"); }
int dl4s_hip_vsub_f32(dl4s_hip_ctx *c, const float *l, const float *r, float *y, int64_t n) { return launch_binary<DL4S_OP_SUB>(c, l, r, y, n, "vSub"); }
int dl4s_hip_vmul_f32(dl4s_hip_ctx *c, const float *l, const float *r, float *y, int64_t n) { return launch_binary<DL4S_OP_MUL>(c, l, r, y, n, "vMul"); }
int dl4s_hip_vdiv_f32(dl4s_hip_ctx *c, const float *l, const float *r, float *y, int64_t n) { return launch_binary<DL4S_OP_DIV>(c, l, r, y, n, "vDiv"); }
int dl4s_hip_vneg_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_NEG>(c, x, y, n, "vNeg"); }
int dl4s_hip_exp_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_EXP>(c, x, y, n, "exp"); }
int dl4s_hip_sqrt_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_SQRT>(c, x, y, n, "sqrt"); }
int dl4s_hip_relu_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_RELU>(c, x, y, n, "relu"); }
int dl4s_hip_tanh_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_TANH>(c, x, y, n, "tanh"); }
int dl4s_hip_log_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_LOG>(c, x, y, n, "log"); }
int dl4s_hip_sin_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_SIN>(c, x, y, n, "sin"); }
int dl4s_hip_cos_f32(dl4s_hip_ctx *c, const float *x, float *y, int64_t n) { return launch_unary<U_COS>(c, x, y, n, "cos"); }

int dl4s_hip_broadcast_f32(dl4s_hip_ctx *ctx, int op, const float *lhs, const int64_t *lhs_shape, int lhs_dim,
                           const float *rhs, const int64_t *rhs_shape, int rhs_dim, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(op >= DL4S_OP_ADD && op <= DL4S_OP_DIV, DL4S_HIP_EINVALID_ARG, "broadcast: unknown op %d", op);
    DL4S_REQUIRE(lhs_dim >= 0 && rhs_dim >= 0 && lhs_dim <= DL4S_HIP_MAX_DIM && rhs_dim <= DL4S_HIP_MAX_DIM,
                 DL4S_HIP_EINVALID_ARG, "broadcast: rank outside [0,%d]", DL4S_HIP_MAX_DIM);
    DL4S_REQUIRE((lhs_dim == 0 || lhs_shape) && (rhs_dim == 0 || rhs_shape), DL4S_HIP_EINVALID_ARG, "broadcast: NULL shape");
    const int dim = lhs_dim > rhs_dim ? lhs_dim : rhs_dim;
    long long ls[DL4S_HIP_MAX_DIM], rs[DL4S_HIP_MAX_DIM];
    Bcast bc{};
    bc.dim = dim;
    long long n = 1;
    for (int i = 0; i < dim; ++i) {
        ls[i] = i < dim - lhs_dim ? 1 : lhs_shape[i - (dim - lhs_dim)];
        rs[i] = i < dim - rhs_dim ? 1 : rhs_shape[i - (dim - rhs_dim)];
        DL4S_REQUIRE(ls[i] >= 0 && rs[i] >= 0, DL4S_HIP_EINVALID_ARG, "broadcast: negative extent");
        DL4S_REQUIRE(ls[i] == rs[i] || ls[i] == 1 || rs[i] == 1, DL4S_HIP_ESHAPE,
                     "broadcast: axis %d has sizes %lld and %lld", i, ls[i], rs[i]);
        bc.oshape[i] = ls[i] > rs[i] ? ls[i] : rs[i];
        if (ls[i] == 0 || rs[i] == 0) bc.oshape[i] = 0;
        n *= bc.oshape[i];
    }
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(lhs && rhs && result, DL4S_HIP_EINVALID_ARG, "broadcast: NULL pointer");
    long long lstride = 1, rstride = 1;
    for (int i = dim - 1; i >= 0; --i) {
        bc.ls[i] = ls[i] == 1 ? 0 : lstride;
        bc.rs[i] = rs[i] == 1 ? 0 : rstride;
        lstride *= ls[i];
        rstride *= rs[i];
    }
    // mode selection of Engine/CPU/CPUEngine.swift:117-176
    long long sc = 1;
    for (int i = dim - 1; i >= 0 && ls[i] == rs[i]; --i) sc *= ls[i];
    int mode = 0;
    if (sc <= 1)
        for (int i = dim - 1; i >= 0; --i) {
            if (ls[i] > rs[i]) { mode = 2; break; }
            if (rs[i] > ls[i]) { mode = 1; break; }
        }
    // Merge neighbouring axes that both operands treat alike (1 = only lhs runs along it, 2 = only rhs, 3 = both; axes of
    // extent 1 drop out).  Up to three groups and fewer than 2^31 elements: the fast kernel.
    long long ge[DL4S_HIP_MAX_DIM];
    int gt[DL4S_HIP_MAX_DIM], groups = 0;
    for (int i = 0; i < dim; ++i) {
        if (bc.oshape[i] == 1) continue;
        const int t = (ls[i] > 1 ? 1 : 0) | (rs[i] > 1 ? 2 : 0);
        if (groups && gt[groups - 1] == t) ge[groups - 1] *= bc.oshape[i];
        else { ge[groups] = bc.oshape[i]; gt[groups] = t; ++groups; }
    }
    if (groups >= 1 && groups <= 3 && n < (1ll << 31)) {
        long long e[3] = {1, 1, 1};
        int t[3] = {0, 0, 0};
        for (int i = 0; i < groups; ++i) { e[3 - groups + i] = ge[i]; t[3 - groups + i] = gt[i]; }
        // element strides of the two (dense) operands over the groups they run along
        unsigned sa[3] = {0, 0, 0}, sb[3] = {0, 0, 0};
        long long as = 1, bs = 1;
        for (int i = 2; i >= 0; --i) {
            if (t[i] & 1) { sa[i] = (unsigned)as; as *= e[i]; }
            if (t[i] & 2) { sb[i] = (unsigned)bs; bs *= e[i]; }
        }
        const auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
        const bool vec = e[2] % 4 == 0 && al16(result) && (!(t[2] & 1) || al16(lhs)) && (!(t[2] & 2) || al16(rhs));
        const unsigned e2v = (unsigned)(vec ? e[2] / 4 : e[2]), nvec = (unsigned)(vec ? n / 4 : n);
#define DL4S_BCAST3(OP_)                                                                                                               \
    if (vec) launch_broadcast3<OP_, 4>(ctx->stream, t[2], lhs, rhs, result, (unsigned)e[1], e2v, sa[0], sa[1], sb[0], sb[1], mode, nvec); \
    else launch_broadcast3<OP_, 1>(ctx->stream, t[2], lhs, rhs, result, (unsigned)e[1], e2v, sa[0], sa[1], sb[0], sb[1], mode, nvec)
        switch (op) {
            case DL4S_OP_ADD: DL4S_BCAST3(DL4S_OP_ADD); break;
            case DL4S_OP_SUB: DL4S_BCAST3(DL4S_OP_SUB); break;
            case DL4S_OP_MUL: DL4S_BCAST3(DL4S_OP_MUL); break;
            default: DL4S_BCAST3(DL4S_OP_DIV); break;
        }
#undef DL4S_BCAST3
        return dl4s::launch_status("broadcast");
    }
    const dim3 g(grid_for(n, 2)), b(TPB);
    switch (op) {
        case DL4S_OP_ADD: hipLaunchKernelGGL(broadcast_f32<DL4S_OP_ADD>, g, b, 0, ctx->stream, lhs, rhs, result, bc, mode, n); break;
        case DL4S_OP_SUB: hipLaunchKernelGGL(broadcast_f32<DL4S_OP_SUB>, g, b, 0, ctx->stream, lhs, rhs, result, bc, mode, n); break;
        case DL4S_OP_MUL: hipLaunchKernelGGL(broadcast_f32<DL4S_OP_MUL>, g, b, 0, ctx->stream, lhs, rhs, result, bc, mode, n); break;
        default: hipLaunchKernelGGL(broadcast_f32<DL4S_OP_DIV>, g, b, 0, ctx->stream, lhs, rhs, result, bc, mode, n); break;
    }
    return dl4s::launch_status("broadcast");
}

static int reduce_common(dl4s_hip_ctx *ctx, bool is_max, const float *values, const int64_t *shape, int dim,
                         const int32_t *axes, int naxes, float *result) {
    DL4S_REQUIRE(dim >= 0 && dim <= DL4S_HIP_MAX_DIM, DL4S_HIP_EINVALID_ARG, "reduce: rank outside [0,%d]", DL4S_HIP_MAX_DIM);
    DL4S_REQUIRE(naxes >= 0 && naxes <= dim && (dim == 0 || shape) && (naxes == 0 || axes), DL4S_HIP_EINVALID_ARG,
                 "reduce: bad axes");
    bool red[DL4S_HIP_MAX_DIM] = {false};
    for (int i = 0; i < naxes; ++i) {
        DL4S_REQUIRE(axes[i] >= 0 && axes[i] < dim && !red[axes[i]], DL4S_HIP_EINVALID_ARG, "reduce: axis %d invalid or repeated", axes[i]);
        red[axes[i]] = true;
    }
    Reduce rd{};
    long long stride[DL4S_HIP_MAX_DIM], s = 1, nout = 1;
    for (int i = dim - 1; i >= 0; --i) {
        DL4S_REQUIRE(shape[i] >= 0, DL4S_HIP_EINVALID_ARG, "reduce: negative extent");
        stride[i] = s;
        s *= shape[i];
    }
    rd.rcount = 1;
    // neighbouring axes of the same kind are merged (the tensor is contiguous), so that e.g. LayerNorm's sum over
    // (length, hidden) is one reduced axis of stride 1
    for (int i = 0; i < dim; ++i) {
        if (shape[i] == 1) continue;    // extent 1 contributes nothing to either index
        if (red[i]) {
            if (rd.rdim > 0 && i > 0 && red[i - 1] && shape[i - 1] != 1) { rd.rshape[rd.rdim - 1] *= shape[i]; rd.rstride[rd.rdim - 1] = stride[i]; }
            else { rd.rshape[rd.rdim] = shape[i]; rd.rstride[rd.rdim] = stride[i]; ++rd.rdim; }
            rd.rcount *= shape[i];
        } else {
            if (rd.kdim > 0 && i > 0 && !red[i - 1] && shape[i - 1] != 1) { rd.kshape[rd.kdim - 1] *= shape[i]; rd.kstride[rd.kdim - 1] = stride[i]; }
            else { rd.kshape[rd.kdim] = shape[i]; rd.kstride[rd.kdim] = stride[i]; ++rd.kdim; }
            nout *= shape[i];
        }
    }
    for (int i = 0; i < dim; ++i)
        if (shape[i] == 0) { if (red[i]) rd.rcount = 0; else nout = 0; }
    if (nout == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(values && result, DL4S_HIP_EINVALID_ARG, "reduce: NULL pointer");
    DL4S_REQUIRE(nout < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "reduce: too many output elements");
    // few outputs with long reduced ranges (LayerNorm statistics: one per batch item): split every range over several
    // workgroups, partial results in the scratch block, then reduce the parts
    long long parts = 1;
    if (nout < 2ll * ctx->cu_count && rd.rcount >= 64ll * TPB) {
        parts = (4ll * ctx->cu_count + nout - 1) / nout;
        const long long most = rd.rcount / (8ll * TPB);
        if (parts > most) parts = most;
        if (parts > 1024) parts = 1024;
        if (parts < 1) parts = 1;
    }
    // many short contiguous rows: one wavefront per row ([16384,512] 14.1 -> 7.2 us, [65536,128] 41 -> 12 us; rows beyond
    // about a thousand elements are better off with a workgroup each: [1100,4096] 4.7 us against 20 us)
    const bool rows_form = rd.rdim == 1 && rd.rstride[0] == 1 && rd.rcount <= 1024 && nout >= 4ll * ctx->cu_count &&
                           (rd.kdim == 0 || (rd.kdim == 1 && rd.kstride[0] == rd.rcount));
    if (rows_form) {
        const unsigned blocks = (unsigned)((nout + TPB / 64 - 1) / (TPB / 64));
        if (is_max) hipLaunchKernelGGL(reduce_rows_f32<true>, dim3(blocks), dim3(TPB), 0, ctx->stream, values, result, (long long)nout, (int)rd.rcount);
        else hipLaunchKernelGGL(reduce_rows_f32<false>, dim3(blocks), dim3(TPB), 0, ctx->stream, values, result, (long long)nout, (int)rd.rcount);
        return dl4s::launch_status("reduce");
    }
    if (parts == 1) {
        if (is_max) hipLaunchKernelGGL(reduce_f32<true>, dim3((unsigned)nout), dim3(TPB), 0, ctx->stream, values, result, rd, rd.rcount);
        else hipLaunchKernelGGL(reduce_f32<false>, dim3((unsigned)nout), dim3(TPB), 0, ctx->stream, values, result, rd, rd.rcount);
        return dl4s::launch_status("reduce");
    }
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    int rc = dl4s::ensure_scratch(ctx, (size_t)(nout * parts) * sizeof(float));
    if (rc) return rc;
    float *part = reinterpret_cast<float *>(ctx->scratch);
    const long long chunk = (rd.rcount + parts - 1) / parts;
    Reduce fin{};
    fin.kdim = 1; fin.kshape[0] = nout; fin.kstride[0] = parts;
    fin.rdim = 1; fin.rshape[0] = parts; fin.rstride[0] = 1; fin.rcount = parts;
    if (is_max) {
        hipLaunchKernelGGL(reduce_f32<true>, dim3((unsigned)nout, (unsigned)parts), dim3(TPB), 0, ctx->stream, values, part, rd, chunk);
        hipLaunchKernelGGL(reduce_f32<true>, dim3((unsigned)nout), dim3(TPB), 0, ctx->stream, part, result, fin, parts);
    } else {
        hipLaunchKernelGGL(reduce_f32<false>, dim3((unsigned)nout, (unsigned)parts), dim3(TPB), 0, ctx->stream, values, part, rd, chunk);
        hipLaunchKernelGGL(reduce_f32<false>, dim3((unsigned)nout), dim3(TPB), 0, ctx->stream, part, result, fin, parts);
    }
    return dl4s::launch_status("reduce");
}

int dl4s_hip_reduce_sum_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, const int32_t *axes,
                            int naxes, float *result) {
    DL4S_CHECK_CTX(ctx);
    return reduce_common(ctx, false, values, shape, dim, axes, naxes, result);
}

int dl4s_hip_reduce_max_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, int axis, float *result) {
    DL4S_CHECK_CTX(ctx);
    int32_t ax = axis;
    return reduce_common(ctx, true, values, shape, dim, &ax, 1, result);
}

int dl4s_hip_permute_axes_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim,
                              const int32_t *arrangement, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(dim >= 0 && dim <= DL4S_HIP_MAX_DIM && (dim == 0 || (shape && arrangement)), DL4S_HIP_EINVALID_ARG,
                 "permuteAxes: bad rank or NULL shape");
    Permute p{};
    p.dim = dim;
    long long dshape[DL4S_HIP_MAX_DIM], dstr[DL4S_HIP_MAX_DIM], n = 1;
    bool seen[DL4S_HIP_MAX_DIM] = {false};
    for (int i = 0; i < dim; ++i) {
        const int a = arrangement[i];
        DL4S_REQUIRE(a >= 0 && a < dim && !seen[a], DL4S_HIP_EINVALID_ARG, "permuteAxes: arrangement is not a permutation");
        DL4S_REQUIRE(shape[i] >= 0, DL4S_HIP_EINVALID_ARG, "permuteAxes: negative extent");
        seen[a] = true;
        dshape[a] = shape[i];
        p.sshape[i] = shape[i];
        n *= shape[i];
    }
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(values && result, DL4S_HIP_EINVALID_ARG, "permuteAxes: NULL pointer");
    long long s = 1;
    for (int i = dim - 1; i >= 0; --i) { dstr[i] = s; s *= dshape[i]; }
    for (int i = 0; i < dim; ++i) p.dstride[i] = dstr[arrangement[i]];
    hipLaunchKernelGGL(permute_f32, dim3(grid_for(n, 2)), dim3(TPB), 0, ctx->stream, values, result, p, n);
    return dl4s::launch_status("permuteAxes");
}

int dl4s_hip_subscript_read_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, const int64_t *start,
                                const int64_t *extent, float *result) {
    DL4S_CHECK_CTX(ctx);
    SliceBox bx;
    long long total = 0;
    const int rc = make_slice_box(shape, dim, start, extent, bx, total, "subscriptRead");
    if (rc != DL4S_HIP_OK || total == 0) return rc;
    DL4S_REQUIRE(values && result, DL4S_HIP_EINVALID_ARG, "subscriptRead: NULL pointer");
    return launch_slice_copy<true>(ctx, values, result, bx, total, values, result);
}

int dl4s_hip_subscript_write_f32(dl4s_hip_ctx *ctx, const float *values, float *result, const int64_t *shape, int dim,
                                 const int64_t *start, const int64_t *extent) {
    DL4S_CHECK_CTX(ctx);
    SliceBox bx;
    long long total = 0;
    const int rc = make_slice_box(shape, dim, start, extent, bx, total, "subscriptWrite");
    if (rc != DL4S_HIP_OK || total == 0) return rc;
    DL4S_REQUIRE(values && result, DL4S_HIP_EINVALID_ARG, "subscriptWrite: NULL pointer");
    return launch_slice_copy<false>(ctx, values, result, bx, total, result, values);
}

int dl4s_hip_band_f32(dl4s_hip_ctx *ctx, const float *buffer, float *result, int64_t rows, int64_t cols, int has_below,
                      int64_t below, int has_above, int64_t above) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(rows >= 0 && cols >= 0, DL4S_HIP_EINVALID_ARG, "band: negative extent");
    if (rows * cols == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(buffer && result, DL4S_HIP_EINVALID_ARG, "band: NULL pointer");
    const long long mx = rows > cols ? rows : cols;
    hipLaunchKernelGGL(band_f32, dim3(grid_for(rows * cols, 2)), dim3(TPB), 0, ctx->stream, buffer, result, (long long)rows,
                       (long long)cols, has_below ? (long long)below : mx, has_above ? (long long)above : mx);
    return dl4s::launch_status("band");
}

int dl4s_hip_stack_f32(dl4s_hip_ctx *ctx, const float *const *buffers, int64_t n, int64_t count, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(n >= 0 && count >= 0, DL4S_HIP_EINVALID_ARG, "stack: negative extent");
    if (n * count == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(buffers && result, DL4S_HIP_EINVALID_ARG, "stack: NULL pointer");
    for (int64_t i = 0; i < n; ++i) DL4S_REQUIRE(buffers[i], DL4S_HIP_EINVALID_ARG, "stack: buffer %lld is NULL", (long long)i);
    // one launch per 64 buffers instead of one copy per buffer (the reference stacks B*H score slices per attention call)
    for (int64_t at = 0; at < n; at += 64) {
        const int m = (int)(n - at < 64 ? n - at : 64);
        StackSrc src{};
        int vec = ((reinterpret_cast<uintptr_t>(result + at * count) & 15) == 0 && count % 4 == 0) ? 1 : 0;
        for (int i = 0; i < m; ++i) {
            src.p[i] = buffers[at + i];
            if (reinterpret_cast<uintptr_t>(buffers[at + i]) & 15) vec = 0;
        }
        long long want = (count / (vec ? 4 : 1) + TPB * 4 - 1) / (TPB * 4);
        if (want < 1) want = 1;
        if (want > 1024) want = 1024;
        hipLaunchKernelGGL(stack_f32, dim3((unsigned)want, (unsigned)m), dim3(TPB), 0, ctx->stream, src, result + at * count,
                           (long long)count, vec);
        const int rc = dl4s::launch_status("stack");
        if (rc != DL4S_HIP_OK) return rc;
    }
    return DL4S_HIP_OK;
}

int dl4s_hip_stack_axis_f32(dl4s_hip_ctx *ctx, const float *const *buffers, const int64_t *chunks, int64_t n, int64_t outer,
                            float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(n >= 0 && outer >= 0, DL4S_HIP_EINVALID_ARG, "stack: negative extent");
    if (n == 0 || outer == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(buffers && chunks && result, DL4S_HIP_EINVALID_ARG, "stack: NULL pointer");
    int64_t total = 0;
    for (int64_t i = 0; i < n; ++i) {
        DL4S_REQUIRE(chunks[i] >= 0, DL4S_HIP_EINVALID_ARG, "stack: negative extent");
        total += chunks[i];
    }
    int64_t at = 0;
    for (int64_t i = 0; i < n; ++i) {
        if (chunks[i] == 0) continue;
        DL4S_REQUIRE(buffers[i], DL4S_HIP_EINVALID_ARG, "stack: buffer %lld is NULL", (long long)i);
        DL4S_HIP_TRY(hipMemcpy2DAsync(result + at, (size_t)total * sizeof(float), buffers[i], (size_t)chunks[i] * sizeof(float),
                                      (size_t)chunks[i] * sizeof(float), (size_t)outer, hipMemcpyDeviceToDevice, ctx->stream));
        at += chunks[i];
    }
    return DL4S_HIP_OK;
}

int dl4s_hip_argmax_f32(dl4s_hip_ctx *ctx, const float *values, int64_t count, int64_t *out_index, float *out_value) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(count >= 0 && out_index && out_value, DL4S_HIP_EINVALID_ARG, "argmax: bad arguments");
    *out_index = 0;
    *out_value = -INFINITY;            // the reference's result for an empty buffer
    if (count == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(values, DL4S_HIP_EINVALID_ARG, "argmax: NULL pointer");
    DL4S_NOT_WHILE_CAPTURING(ctx);
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    int rc = dl4s::ensure_scratch(ctx, 16);
    if (rc) return rc;
    float *dv = reinterpret_cast<float *>(ctx->scratch);
    long long *di = reinterpret_cast<long long *>(reinterpret_cast<char *>(ctx->scratch) + 8);
    hipLaunchKernelGGL(argmax_f32, dim3(1), dim3(1024), 0, ctx->stream, values, (long long)count, dv, di);
    rc = dl4s::launch_status("argmax");
    if (rc) return rc;
    struct { float v; float pad; long long i; } host;
    DL4S_HIP_TRY(hipMemcpyAsync(&host, ctx->scratch, 16, hipMemcpyDeviceToHost, ctx->stream));
    DL4S_HIP_TRY(hipStreamSynchronize(ctx->stream));
    *out_index = host.i;
    *out_value = host.v;
    return DL4S_HIP_OK;
}

int dl4s_hip_argmax_to_f32(dl4s_hip_ctx *ctx, const float *values, int64_t count, int32_t *out_index_dev, int32_t *counter_dev) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(values && out_index_dev && count > 0 && count < (1ll << 31), DL4S_HIP_EINVALID_ARG,
                 "argmax_to: NULL pointer or count outside [1, 2^31)");
    hipLaunchKernelGGL(argmax_f32, dim3(1), dim3(1024), 0, ctx->stream, values, (long long)count, (float *)nullptr, (long long *)nullptr,
                       out_index_dev, counter_dev);
    return dl4s::launch_status("argmax_to");
}

int dl4s_hip_embed_at_f32(dl4s_hip_ctx *ctx, const float *table, int64_t vocab, int64_t D, const int32_t *token_dev,
                          const float *scale, const float *positions, int64_t position_rows, const int32_t *position_dev,
                          float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(vocab >= 0 && D >= 0 && position_rows >= 0, DL4S_HIP_EINVALID_ARG, "embed_at: negative extent");
    if (D == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(table && token_dev && result && (!positions || position_dev), DL4S_HIP_EINVALID_ARG, "embed_at: NULL pointer");
    hipLaunchKernelGGL(embed_at_f32, dim3(grid_for(D)), dim3(TPB), 0, ctx->stream, table, token_dev, positions, position_dev, result,
                       (long long)vocab, (long long)D, (long long)position_rows, scale ? *scale : 1.0f, scale ? 1 : 0);
    return dl4s::launch_status("embed_at");
}

int dl4s_hip_embed_positions_f32(dl4s_hip_ctx *ctx, const float *table, int64_t vocab, int64_t D, const int32_t *tokens,
                                 int64_t batch, int64_t L, int32_t ignore_index, const float *scale, const float *positions,
                                 float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(vocab >= 0 && D >= 0 && batch >= 0 && L >= 0, DL4S_HIP_EINVALID_ARG, "embedding: negative extent");
    const long long n = batch * L * D;
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(table && tokens && result, DL4S_HIP_EINVALID_ARG, "embedding: NULL pointer");
    hipLaunchKernelGGL(embed_positions_f32, dim3(grid_for(n)), dim3(TPB), 0, ctx->stream, table, tokens, positions, result,
                       (long long)(batch * L), (long long)L, (long long)D, (long long)vocab, (int)ignore_index,
                       scale ? *scale : 1.0f, scale ? 1 : 0);
    return dl4s::launch_status("embedding");
}

int dl4s_hip_log_softmax_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t n, float *result) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(rows >= 0 && n >= 0, DL4S_HIP_EINVALID_ARG, "logSoftmax: negative extent");
    if (rows * n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(x && result, DL4S_HIP_EINVALID_ARG, "logSoftmax: NULL pointer");
    DL4S_REQUIRE(rows < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "logSoftmax: too many rows");
    hipLaunchKernelGGL(log_softmax_f32, dim3((unsigned)rows), dim3(256), 0, ctx->stream, x, result, (long long)n);
    return dl4s::launch_status("logSoftmax");
}

int dl4s_hip_layernorm_f32(dl4s_hip_ctx *ctx, const float *x, const float *residual, const float *scale, const float *shift,
                           float *result, int64_t B, int64_t rows, int64_t D) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && rows >= 0 && D >= 0, DL4S_HIP_EINVALID_ARG, "layernorm: negative extent");
    const long long n = rows * D;
    if (B * n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(x && scale && shift && result, DL4S_HIP_EINVALID_ARG, "layernorm: NULL pointer");
    DL4S_REQUIRE(B < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "layernorm: batch too large");
    const auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec = n % 4 == 0 && D % 4 == 0 && a16(x) && a16(residual) && a16(scale) && a16(shift) && a16(result);
    if (n <= 16384) {
        // rows beyond 4096 elements (the joint (L, D) LayerNorm of a short decoded prefix): 1024 threads, so that a thread's
        // loads are few enough to be in flight together
        if (n > 4096) {
            if (vec) hipLaunchKernelGGL((ln_small_f32<true, 1024>), dim3((unsigned)B), dim3(1024), 0, ctx->stream, x, residual, scale, shift, result, n, (long long)D);
            else hipLaunchKernelGGL((ln_small_f32<false, 1024>), dim3((unsigned)B), dim3(1024), 0, ctx->stream, x, residual, scale, shift, result, n, (long long)D);
        } else {
            if (vec) hipLaunchKernelGGL((ln_small_f32<true, TPB>), dim3((unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, scale, shift, result, n, (long long)D);
            else hipLaunchKernelGGL((ln_small_f32<false, TPB>), dim3((unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, scale, shift, result, n, (long long)D);
        }
        return dl4s::launch_status("layernorm");
    }
    DL4S_REQUIRE(B <= 65535, DL4S_HIP_EUNSUPPORTED, "layernorm: batch above 65535 with long rows");
    long long want = n / (TPB * 8);
    int nblk = (int)(want < 1 ? 1 : (want > 256 ? 256 : want));
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    int rc = dl4s::ensure_scratch(ctx, (size_t)B * nblk * 2 * sizeof(float));
    if (rc) return rc;
    float *part = reinterpret_cast<float *>(ctx->scratch);
    if (vec) {
        hipLaunchKernelGGL(ln_partial_f32<true>, dim3(nblk, (unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, part, n, nblk);
        hipLaunchKernelGGL(ln_apply_f32<true>, dim3(nblk, (unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, scale, shift, result, part,
                           n, (long long)D, nblk);
    } else {
        hipLaunchKernelGGL(ln_partial_f32<false>, dim3(nblk, (unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, part, n, nblk);
        hipLaunchKernelGGL(ln_apply_f32<false>, dim3(nblk, (unsigned)B), dim3(TPB), 0, ctx->stream, x, residual, scale, shift, result, part,
                           n, (long long)D, nblk);
    }
    return dl4s::launch_status("layernorm");
}

int dl4s_hip_layernorm_reference_order_f32(dl4s_hip_ctx *ctx, const float *x, const float *residual, const float *scale,
                                           const float *shift, float *result, int64_t B, int64_t rows, int64_t D) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && rows >= 0 && D >= 0, DL4S_HIP_EINVALID_ARG, "layernorm: negative extent");
    const long long n = rows * D, R = B * rows;
    if (B * n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(x && scale && shift && result, DL4S_HIP_EINVALID_ARG, "layernorm: NULL pointer");
    DL4S_REQUIRE(R < (1ll << 36) && B < (1ll << 31), DL4S_HIP_EUNSUPPORTED, "layernorm: too many rows");
    const auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec = n % 4 == 0 && D % 4 == 0 && a16(x) && a16(residual) && a16(scale) && a16(shift) && a16(result);
    std::lock_guard<std::mutex> scratch_lock(ctx->scratch_mu);
    // per-row pairs, then (items of more than one row) per-item pairs behind them
    const size_t row_floats = (size_t)R * 2, item_floats = rows > 1 ? (size_t)B * 2 : 0;
    int rc = dl4s::ensure_scratch(ctx, (row_floats + item_floats) * sizeof(float));
    if (rc) return rc;
    float *rowpart = reinterpret_cast<float *>(ctx->scratch), *itempart = rows > 1 ? rowpart + row_floats : rowpart;
    if (vec && R < 32ll * 2 * ctx->cu_count)
        hipLaunchKernelGGL(ln_row_sums_seq_vec_f32<8>, dim3((unsigned)((R + 7) / 8)), dim3(64), 0, ctx->stream, x, residual, rowpart, R, (long long)D);
    else if (vec)
        hipLaunchKernelGGL(ln_row_sums_seq_vec_f32<32>, dim3((unsigned)((R + 31) / 32)), dim3(64), 0, ctx->stream, x, residual, rowpart, R, (long long)D);
    else
        hipLaunchKernelGGL(ln_row_sums_seq_f32, dim3((unsigned)((R + LN_SEQ_ROWS - 1) / LN_SEQ_ROWS)), dim3(64), 0, ctx->stream, x, residual,
                           rowpart, R, (long long)D);
    if (rows > 1) hipLaunchKernelGGL(ln_item_sums_seq_f32, dim3((unsigned)B), dim3(64), 0, ctx->stream, rowpart, itempart, (long long)rows);
    // the normalising pass of the tree-sum kernels on one pair per item (0 + the pair: exact)
    const long long want = n / (TPB * 8);
    const unsigned gx = (unsigned)(want < 1 ? 1 : (want > 256 ? 256 : want));
    for (long long b0 = 0; b0 < B; b0 += 65535) {
        const unsigned nb = (unsigned)(B - b0 < 65535 ? B - b0 : 65535);
        const float *xp = x + b0 * n, *rp = residual ? residual + b0 * n : nullptr;
        if (vec)
            hipLaunchKernelGGL(ln_apply_f32<true>, dim3(gx, nb), dim3(TPB), 0, ctx->stream, xp, rp, scale, shift, result + b0 * n,
                               itempart + b0 * 2, n, (long long)D, 1);
        else
            hipLaunchKernelGGL(ln_apply_f32<false>, dim3(gx, nb), dim3(TPB), 0, ctx->stream, xp, rp, scale, shift, result + b0 * n,
                               itempart + b0 * 2, n, (long long)D, 1);
    }
    return dl4s::launch_status("layernorm_reference_order");
}

int dl4s_hip_bias_gelu_f32(dl4s_hip_ctx *ctx, const float *x, const float *bias, float *result, int64_t rows, int64_t D) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(rows >= 0 && D >= 0, DL4S_HIP_EINVALID_ARG, "bias_gelu: negative extent");
    const long long n = rows * D;
    if (n == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(x && result, DL4S_HIP_EINVALID_ARG, "bias_gelu: NULL pointer");
    hipLaunchKernelGGL(bias_gelu_f32, dim3(grid_for(n)), dim3(TPB), 0, ctx->stream, x, bias, result, n, (long long)D);
    return dl4s::launch_status("bias_gelu");
}

}  // extern "C"

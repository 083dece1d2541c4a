// Shared internals of libdl4s_hip.so: the context object, error reporting and launch helpers.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/dl4s_hip.h"

struct dl4s_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    int cu_count = 0;
    int clock_khz = 0;
    char name[256] = {0};
    std::mutex mu;
    // pooled allocator: live blocks (base -> rounded size) and free lists per rounded size
    std::map<uintptr_t, size_t> live;
    std::unordered_map<size_t, std::vector<void *>> pool;
    size_t bytes_in_use = 0, bytes_pooled = 0;
    // scratch owned by the library for split-K partial results (grown on demand, never shrunk)
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    // Held by an entry point from the launch that fills the scratch block to the launch that reads it, so that calls
    // from several host threads cannot interleave their use of it (the kernels themselves are ordered by the stream).
    std::mutex scratch_mu;
    // Device address, on this context's GPU, of the fixed block dl4s_hip_sdpa_decode_noalloc_f32 keeps its partial records in.
    float *static_scratch = nullptr;
    // Recorded behind every use of that block by this context; a call on another context of the same GPU waits for it.
    hipEvent_t static_scratch_done = nullptr;
    // Stream capture (dl4s_hip_graph_begin .. dl4s_hip_graph_end): entry points that would wait for the stream, copy to or
    // from host memory or change device allocations refuse to run while it is set.  scratch_generation counts the
    // regrowths of the scratch block; a captured graph holds the block's address and is refused once it has moved.
    std::atomic<bool> capturing{false};
    unsigned long long scratch_generation = 0;
    // Blocks handed back with dl4s_hip_free while a graph is being recorded: the recorded kernels still use them on every
    // replay, so they stay out of the pool until the graph is destroyed (dl4s_hip_graph_end moves the list to the graph).
    // Allocations made later in the same recording may take them.
    std::vector<std::pair<void *, size_t>> held_by_recording;
    size_t bytes_held = 0;
    // One bit per (kernel family, mask kind): the dynamic-LDS limit of those kernels has been raised on this context's
    // device (hipFuncSetAttribute is per device; two host threads that both find a bit clear both set the attribute, which
    // is harmless, and then the bit).
    std::atomic<unsigned long long> lds_limit_raised[2] = {{0}, {0}};   // bit family * 8 + kind
};

struct dl4s_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    dl4s_hip_ctx *owner = nullptr;
    size_t nodes = 0;
    unsigned long long scratch_generation = 0;
    std::vector<std::pair<void *, size_t>> held;   // temporaries freed during the recording, returned to the pool on destroy
};

namespace dl4s {

int set_error(int code, const char *fmt, ...);
int hip_error(hipError_t e, const char *what);
// Grows ctx->scratch to at least `bytes`; returns 0 or a status.
int ensure_scratch(dl4s_hip_ctx *ctx, size_t bytes);
// The normalising pass of the LayerNorm kernels on partial sums some other kernel left (nblk <= 256 pairs per item, laid
// out [item][nblk][2]); x and y may be the same tensor.  The caller holds the scratch mutex when `part` lies there.
int layernorm_apply(dl4s_hip_ctx *ctx, const float *x, const float *scale, const float *shift, float *y, const float *part,
                    long long items, long long n, long long D, int nblk);
// dl4s_hip_gemm_batched_f32 for callers inside the library whose batch fills the GPU by itself: always the tiled kernels,
// never the skinny form that a single product of the shape would take (so not the bits of the public entry for such shapes).
int gemm_batched_tiled(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols, int64_t lhs_stride, const float *rhs,
                       int64_t rhs_rows, int64_t rhs_cols, int64_t rhs_stride, float *result, int64_t result_stride, int64_t batch,
                       float alpha, float beta, int transpose_first, int transpose_second, int triangle = 0);
// (triangle: 0, or a product with a causal triangle - 1: only output tiles that reach column <= row are computed, the
// rest of the result is left untouched; 2: lhs^T is zero before the diagonal, the contraction starts at the output tile's
// first row; 3: lhs is zero beyond the diagonal, the contraction ends with the output tile's last row.  Tiles are at most
// 128 wide and start at multiples of their width.  Operands the fast tiled kernels do not take - extents that are not
// multiples of 4, operands off the 16-byte grid - fail with DL4S_HIP_EUNSUPPORTED before anything is launched.)
// Looks up the device address of the decode kernels' fixed scratch block (sdpa_decode.hip) for the current GPU.
int decode_static_scratch_init(dl4s_hip_ctx *ctx);
void decode_static_scratch_release(dl4s_hip_ctx *ctx);

#define DL4S_CHECK_CTX(ctx)                                                        \
    do {                                                                           \
        if (!(ctx)) return dl4s::set_error(DL4S_HIP_EINVALID_ARG, "%s: ctx is NULL", __func__); \
        hipError_t e__ = hipSetDevice((ctx)->device);                              \
        if (e__ != hipSuccess) return dl4s::hip_error(e__, "hipSetDevice");        \
    } while (0)

// For entry points that cannot be recorded into a graph.
#define DL4S_NOT_WHILE_CAPTURING(ctx)                                                                       \
    do {                                                                                                    \
        if ((ctx)->capturing)                                                                               \
            return dl4s::set_error(DL4S_HIP_EUNSUPPORTED,                                                   \
                                   "%s cannot be recorded into a graph (it waits for the stream, copies to or from " \
                                   "host memory or allocates)", __func__);                                  \
    } while (0)

#define DL4S_HIP_TRY(expr)                                               \
    do {                                                                 \
        hipError_t e__ = (expr);                                         \
        if (e__ != hipSuccess) return dl4s::hip_error(e__, #expr);       \
    } while (0)

#define DL4S_REQUIRE(cond, code, ...)                                    \
    do {                                                                 \
        if (!(cond)) return dl4s::set_error((code), __VA_ARGS__);        \
    } while (0)

// Kernel families of dl4s_hip_ctx::lds_limit_raised.
enum { LDS_PREFILL_SPLIT = 0, LDS_PREFILL = 1, LDS_PREFILL_D128 = 2, LDS_BWD = 3, LDS_BWD_D128 = 4, LDS_GEMM_DEEP = 5, LDS_PREFILL_W192 = 6,
       LDS_PREFILL_W256 = 7, LDS_PREFILL_W160 = 8, LDS_GEMM_HALVES = 9 };
inline bool lds_limit_pending(const dl4s_hip_ctx *ctx, int family, int kind) {
    const int bit = family * 8 + kind;
    return !(ctx->lds_limit_raised[bit >> 6].load(std::memory_order_acquire) & (1ull << (bit & 63)));
}
inline void lds_limit_done(dl4s_hip_ctx *ctx, int family, int kind) {
    const int bit = family * 8 + kind;
    ctx->lds_limit_raised[bit >> 6].fetch_or(1ull << (bit & 63), std::memory_order_release);
}

inline int launch_status(const char *kernel) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_error(e, kernel);
    return DL4S_HIP_OK;
}

// Sum over the 64 lanes of a wavefront, the same value (same bits) in every lane: four exchanges inside the rows of 16
// lanes through the vector ALU's lane permutes (xor 1, xor 2, mirror of 8, mirror of 16 - after each step the lanes
// that exchange hold the same partial sums, so a mirror adds what an xor would), then the four row sums in order.  No
// trip through the LDS pipe: about 60 cycles where six `__shfl_xor` steps take 700.
template <int CTRL>
__device__ __forceinline__ float dpp_lanes(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_lanes<0xB1>(v);       // quad_perm [1,0,3,2]
    v += dpp_lanes<0x4E>(v);       // quad_perm [2,3,0,1]
    v += dpp_lanes<0x141>(v);      // row_half_mirror
    v += dpp_lanes<0x140>(v);      // row_mirror
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return ((r0 + r1) + r2) + r3;
}

}  // namespace dl4s

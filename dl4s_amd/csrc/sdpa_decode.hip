// Single-query attention over a key/value cache (one decode step), split over the keys.
//
// The cache is [B,H,Tcap,64] fp32.  A workgroup (4 wavefronts) owns one (batch, head) and one chunk
// of CHUNK keys; each wavefront streams 64 keys: a 16-lane group reads one 256-byte key row with one
// 128-bit load per lane, so every load instruction of a wavefront covers four whole rows and all the
// K loads and V loads of the wavefront are in flight together.  The dot product is reduced inside
// the 16-lane group with DPP adds.  Each workgroup leaves (max, sum, 64 partial outputs) in a scratch
// buffer; the last workgroup of a (batch, head) to finish (agent-scope ticket) merges the partials
// with the usual softmax rescaling and writes the output, so that one launch serves a whole step.
#include "common.h"

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 64;
constexpr int WAVES = 4;
constexpr int KEYS_PER_WAVE = 64;
constexpr int CHUNK = WAVES * KEYS_PER_WAVE;  // keys per workgroup
constexpr int PSTR = 68;                      // floats per partial record: o[0..63], m, l, pad
constexpr float LOG2E = 1.44269504088896340736f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
// Sum over the 16 lanes of a DPP row; every lane of the row ends up with the total.
__device__ __forceinline__ float row16_sum(float x) {
    x += dpp<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp<0x4E>(x);   // quad_perm [2,3,0,1]
    x += dpp<0x141>(x);  // row_half_mirror
    x += dpp<0x140>(x);  // row_mirror
    return x;
}

template <bool APPEND>
__global__ __launch_bounds__(256) void sdpa_decode_splitk_f32(const float *__restrict__ q, float *kcache,
                                                               float *vcache, const float *__restrict__ k_new,
                                                               const float *__restrict__ v_new,
                                                               float *__restrict__ out, float *part,
                                                               unsigned int *tickets, int T, int Tcap, int pos,
                                                               float rT, int nsplit) {
    __shared__ float sm_o[WAVES][HD];
    __shared__ float sm_m[WAVES], sm_l[WAVES];
    __shared__ int sm_last;
    const int split = blockIdx.x;
    const int bh = blockIdx.y;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, c = lane & 15;

    f32x4 qv = *reinterpret_cast<const f32x4 *>(q + (long long)bh * HD + 4 * c);
    qv.x *= rT; qv.y *= rT; qv.z *= rT; qv.w *= rT;

    const int kbeg = split * CHUNK + wave * KEYS_PER_WAVE + g;
    const long long base = (long long)bh * Tcap * HD + 4 * c;
    f32x4 kk[16], vv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int key = kbeg + 4 * i;
        const int kc = key < T ? key : T - 1;
        if (APPEND && kc == pos) {
            kk[i] = *reinterpret_cast<const f32x4 *>(k_new + (long long)bh * HD + 4 * c);
            if (key == pos) *reinterpret_cast<f32x4 *>(kcache + base + (long long)pos * HD) = kk[i];
        } else {
            kk[i] = *reinterpret_cast<const f32x4 *>(kcache + base + (long long)kc * HD);
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int key = kbeg + 4 * i;
        const int kc = key < T ? key : T - 1;
        if (APPEND && kc == pos) {
            vv[i] = *reinterpret_cast<const f32x4 *>(v_new + (long long)bh * HD + 4 * c);
            if (key == pos) *reinterpret_cast<f32x4 *>(vcache + base + (long long)pos * HD) = vv[i];
        } else {
            vv[i] = *reinterpret_cast<const f32x4 *>(vcache + base + (long long)kc * HD);
        }
    }

    float s[16];
    float mw = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        float d = qv.x * kk[i].x;
        d += qv.y * kk[i].y;
        d += qv.z * kk[i].z;
        d += qv.w * kk[i].w;
        d = row16_sum(d);
        if (kbeg + 4 * i >= T) d = -INFINITY;
        s[i] = d;
        mw = fmaxf(mw, d);
    }
    mw = fmaxf(mw, __shfl_xor(mw, 16, 64));
    mw = fmaxf(mw, __shfl_xor(mw, 32, 64));
    const float m_use = (mw == -INFINITY) ? 0.f : mw;
    float l = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float p = fast_exp2((s[i] - m_use) * LOG2E);
        l += p;
        acc.x += p * vv[i].x; acc.y += p * vv[i].y; acc.z += p * vv[i].z; acc.w += p * vv[i].w;
    }
#pragma unroll
    for (int o = 16; o <= 32; o <<= 1) {
        l += __shfl_xor(l, o, 64);
        acc.x += __shfl_xor(acc.x, o, 64); acc.y += __shfl_xor(acc.y, o, 64);
        acc.z += __shfl_xor(acc.z, o, 64); acc.w += __shfl_xor(acc.w, o, 64);
    }
    if (g == 0) *reinterpret_cast<f32x4 *>(&sm_o[wave][4 * c]) = acc;
    if (lane == 0) { sm_m[wave] = mw; sm_l[wave] = l; }
    __syncthreads();

    float *rec = part + ((long long)bh * nsplit + split) * PSTR;
    if (tid < HD) {
        float M = sm_m[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) M = fmaxf(M, sm_m[w]);
        const float Mu = (M == -INFINITY) ? 0.f : M;
        float L = 0.f, O = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = fast_exp2((sm_m[w] - Mu) * LOG2E);
            L += sm_l[w] * f;
            O += sm_o[w][tid] * f;
        }
        if (nsplit == 1) {
            out[(long long)bh * HD + tid] = O * (1.0f / L);
        } else {
            rec[tid] = O;
            if (tid == 0) { rec[HD] = M; rec[HD + 1] = L; }
        }
    }
    if (nsplit == 1) return;

    // Ticket: the workgroup that takes the last one merges all partial records of this (batch, head).
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        unsigned int t = __hip_atomic_fetch_add(&tickets[bh], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        sm_last = (t == (unsigned int)(nsplit - 1));
    }
    __syncthreads();
    if (!sm_last) return;
    __threadfence();
    if (tid < HD) {
        const float *recs = part + (long long)bh * nsplit * PSTR;
        float M = -INFINITY;
        for (int sidx = 0; sidx < nsplit; ++sidx)
            M = fmaxf(M, __builtin_nontemporal_load(recs + sidx * PSTR + HD));
        const float Mu = (M == -INFINITY) ? 0.f : M;
        float L = 0.f, O = 0.f;
        for (int sidx = 0; sidx < nsplit; ++sidx) {
            const float f = fast_exp2((__builtin_nontemporal_load(recs + sidx * PSTR + HD) - Mu) * LOG2E);
            L += __builtin_nontemporal_load(recs + sidx * PSTR + HD + 1) * f;
            O += __builtin_nontemporal_load(recs + sidx * PSTR + tid) * f;
        }
        out[(long long)bh * HD + tid] = O * (1.0f / L);
    }
    if (tid == 0) __hip_atomic_store(&tickets[bh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
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

int decode_launch(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache, const float *k_new,
                  const float *v_new, float *out, int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t pos,
                  int64_t d, float rT, bool append) {
    const int64_t BH = B * H;
    if (BH == 0) return DL4S_HIP_OK;
    DL4S_REQUIRE(q && kcache && vcache && out, DL4S_HIP_EINVALID_ARG, "sdpa_decode: NULL tensor pointer");
    DL4S_REQUIRE(d == HD, DL4S_HIP_EUNSUPPORTED, "sdpa_decode: head dim %lld (only 64 is implemented)", (long long)d);
    DL4S_REQUIRE(T >= 1 && T <= Tcap, DL4S_HIP_ESHAPE, "sdpa_decode: T=%lld must be in [1, Tcap=%lld]", (long long)T,
                 (long long)Tcap);
    DL4S_REQUIRE(BH <= 65535 && Tcap < (1ll << 30), DL4S_HIP_EUNSUPPORTED, "sdpa_decode: B*H=%lld above 65535", (long long)BH);
    const int nsplit = (int)((T + CHUNK - 1) / CHUNK);
    // partial records live in the context's scratch block; size it for the whole cache capacity so that
    // the following steps of the same sequence do not grow it again
    const int cap_split = (int)((Tcap + CHUNK - 1) / CHUNK);
    int rc = dl4s::ensure_scratch(ctx, (size_t)BH * cap_split * PSTR * sizeof(float));
    if (rc) return rc;
    float *part = reinterpret_cast<float *>(ctx->scratch);
    unsigned int *tickets = ctx->tickets;  // BH <= 65535 entries, zero between launches
    dim3 grid(nsplit, (unsigned)BH);
    if (append)
        hipLaunchKernelGGL(sdpa_decode_splitk_f32<true>, grid, dim3(256), 0, ctx->stream, q, kcache, vcache, k_new, v_new,
                           out, part, tickets, (int)T, (int)Tcap, (int)pos, rT, nsplit);
    else
        hipLaunchKernelGGL(sdpa_decode_splitk_f32<false>, grid, dim3(256), 0, ctx->stream, q, kcache, vcache, k_new, v_new,
                           out, part, tickets, (int)T, (int)Tcap, -1, rT, nsplit);
    return dl4s::launch_status("sdpa_decode_splitk_f32");
}

}  // namespace

extern "C" {

int dl4s_hip_sdpa_decode_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache, float *out,
                             int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d, float inv_temperature) {
    DL4S_CHECK_CTX(ctx);
    DL4S_REQUIRE(B >= 0 && H >= 0, DL4S_HIP_EINVALID_ARG, "sdpa_decode: negative extent");
    return decode_launch(ctx, q, const_cast<float *>(kcache), const_cast<float *>(vcache), nullptr, nullptr, out, B, H, T,
                         Tcap, -1, d, inv_temperature, false);
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

}  // extern "C"

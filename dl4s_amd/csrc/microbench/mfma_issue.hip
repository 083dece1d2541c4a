// Microbenchmark behind the prefill kernel's ceiling: how much of the fp32 MFMA peak a wavefront program keeps when
// vector-ALU work is interleaved with a stream of v_mfma_f32_32x32x2_f32, on the prefill kernel's shape (64 MFMAs per
// 32-key tile, operands from LDS on a 68-float row stride, one barrier per tile, 3 workgroups of 4 wavefronts per CU).
// The VALU work does not depend on the accumulators, so what is measured is issue, not a data hazard.
//
//   build:  hipcc --offload-arch=gfx950 -O3 -o dl4s_amd/mfma_issue dl4s_amd/csrc/microbench/mfma_issue.hip
//           (python -m dl4s_amd.build does it)
//   run:    dl4s_amd/mfma_issue
//
// Output: one line per variant with the time per launch, TFLOP/s and the fraction of 157.3 TFLOP/s.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                      \
    do {                                                                              \
        hipError_t e__ = (x);                                                         \
        if (e__ != hipSuccess) {                                                      \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e__));                  \
            exit(1);                                                                  \
        }                                                                             \
    } while (0)

// LDS_OPS: A operands read from LDS (one 128-bit read per 4 MFMAs) instead of a register.
// BARRIER: one workgroup barrier per tile.
// NADD: plain VALU instructions (v_add_f32) per tile.   NEXP: v_exp_f32 (quarter rate) per tile, each with its subtract.
template <bool LDS_OPS, bool BARRIER, int NADD, int NEXP>
__global__ __launch_bounds__(256, 3) void mfma_stream(float *out, int tiles, float a, float b) {
    __shared__ __align__(16) float lds[2][32 * 68];
    const int tid = threadIdx.x, lane = tid & 63, ln = lane & 31, half = lane >> 5;
    for (int i = tid; i < 2 * 32 * 68; i += 256) (&lds[0][0])[i] = (float)(i & 7) * 0.125f;
    __syncthreads();
    f32x16 acc0, acc1;
    for (int i = 0; i < 16; ++i) { acc0[i] = 0.f; acc1[i] = 0.f; }
    float q[32];
    for (int i = 0; i < 32; ++i) q[i] = b + i * 0.001f;
    float side[8];
    for (int i = 0; i < 8; ++i) side[i] = a * i;
    for (int t = 0; t < tiles; ++t) {
        const float *Kb = &lds[t & 1][ln * 68 + half * 32];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                f32x4 av = {a, a, a, a};
                if (LDS_OPS) av = *reinterpret_cast<const f32x4 *>(Kb + 4 * j + h * 16 * 68);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, q[4 * j + 0], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, q[4 * j + 1], acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, q[4 * j + 2], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, q[4 * j + 3], acc1, 0, 0, 0);
            }
        }
        // eight independent chains, so that the instructions can issue back to back
#pragma unroll
        for (int i = 0; i < NADD; ++i) side[i & 7] = side[i & 7] + b;
#pragma unroll
        for (int i = 0; i < NEXP; ++i) side[i & 7] = __builtin_amdgcn_exp2f(side[i & 7] - a);
        if (BARRIER) __syncthreads();
    }
    float s = 0.f;
    for (int i = 0; i < 8; ++i) s += side[i];
    for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i];
    out[blockIdx.x * 256 + tid] = s;
}

template <bool LDS_OPS, bool BARRIER, int NADD, int NEXP>
void run(const char *what, float *out, int cus) {
    const int tiles = 512, grid = cus * 3;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int w = 0; w < 30; ++w) hipLaunchKernelGGL((mfma_stream<LDS_OPS, BARRIER, NADD, NEXP>), dim3(grid), dim3(256), 0, 0, out, tiles, 1.0f, 0.5f);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0));
    const int reps = 20;
    for (int w = 0; w < reps; ++w) hipLaunchKernelGGL((mfma_stream<LDS_OPS, BARRIER, NADD, NEXP>), dim3(grid), dim3(256), 0, 0, out, tiles, 1.0f, 0.5f);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= reps;
    const double flops = (double)grid * 4 * tiles * 64 * 4096.0;
    printf("%-62s %7.3f ms  %6.1f TFLOP/s  %5.1f %% of peak\n", what, ms, flops / ms / 1e9, flops / ms / 1e9 / 1.573);
    fflush(stdout);
}

int main() {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    float *out = nullptr;
    CHECK(hipMalloc(&out, (size_t)cus * 3 * 256 * sizeof(float)));
    printf("%s, %d CUs; 64 MFMAs (32x32x2 f32) per tile, 3 workgroups of 4 wavefronts per CU\n", prop.gcnArchName, cus);
    run<false, false, 0, 0>("MFMA only, operands in registers", out, cus);
    run<true, false, 0, 0>("MFMA, A operands from LDS", out, cus);
    run<true, true, 0, 0>("MFMA, LDS operands, barrier per tile", out, cus);
    run<true, true, 16, 0>("  + 16 v_add per tile", out, cus);
    run<true, true, 32, 0>("  + 32 v_add per tile", out, cus);
    run<true, true, 64, 0>("  + 64 v_add per tile", out, cus);
    run<true, true, 107, 0>("  + 107 v_add per tile", out, cus);
    run<true, true, 0, 16>("  + 16 (v_sub, v_exp) per tile", out, cus);
    run<true, true, 75, 16>("  + 75 v_add + 16 (v_sub, v_exp): the prefill tile's VALU count", out, cus);
    CHECK(hipFree(out));
    return 0;
}

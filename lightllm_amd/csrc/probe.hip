// Measurement aid: the arithmetic of the block-scaled GEMM's inner loop with everything else taken away.
//
// A workgroup of 4 or 8 waves (one or two per SIMD) on every compute unit; each wave holds a 128 x 64 sub-tile of fp32
// accumulators and runs, per iteration, the 32 products v_mfma_f32_16x16x128_f8f6f4 of one K step on operand
// fragments that stay in registers - either accumulating in the matrix core (fold = 0) or as the kernels must,
// product by product with C = 0 and the fp32 scale fold acc += part * s two products behind (fold = 1).  No LDS, no
// memory traffic in the loop.  What this loop reaches with random e4m3 operands is the ceiling of any kernel built
// on these instructions: the part lowers its clock under the load (the data-sheet peak assumes 2.4 GHz), and more
// so the more the operands toggle.
#include "common.hpp"

namespace mi355 {

template <bool FOLD>
__global__ __launch_bounds__(512) void mfma_probe_kernel(const v8i *__restrict__ src, float *__restrict__ sink, int iters) {
    const int tid = threadIdx.x, lane = tid & 63;
    v8i wf[4], xf[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wf[j] = src[(j * 64 + lane) + (tid >> 6) * 512];
#pragma unroll
    for (int i = 0; i < 4; ++i) xf[i] = src[((4 + i) * 64 + lane) + (tid >> 6) * 512];
    float xs[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xs[i] = 1.0f + 0.001f * (float)((lane + i) & 15);
    v4f acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if constexpr (!FOLD) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[h * 4 + e / 4][e % 4] = mfma_16x16x128_fp8(wf[e % 4], xf[e / 4], acc[h * 4 + e / 4][e % 4]);
            } else {
                constexpr int E = 16, kLag = 2;
                v4f parts[kLag + 1];
#pragma unroll
                for (int e = 0; e < E + kLag; ++e) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (e < E) parts[e % (kLag + 1)] = mfma_16x16x128_fp8(wf[e % 4], xf[e / 4], v4f{0.f, 0.f, 0.f, 0.f});
                    if (e >= kLag) {
                        const int f = e - kLag;
                        acc[h * 4 + f / 4][f % 4] += parts[f % (kLag + 1)] * xs[h * 4 + f / 4];
                    }
                    if (e < E && e >= kLag) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                    }
                }
            }
            // the fragments count as new for the compiler after every half step (a real kernel reloads them): the
            // products of the two halves are not merged
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(xf[i]));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    sink[blockIdx.x * blockDim.x + tid] = s;
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_probe_mfma(const void *operands, void *sink, int32_t fold, int32_t waves, int32_t iters,
                                void *stream) {
    if (!operands || !sink || iters <= 0 || (waves != 4 && waves != 8)) return MI355_EINVAL;
    if (((uintptr_t)operands & 31) || ((uintptr_t)sink & 3)) return MI355_EALIGN;
    const int cus = device_cus();
    // one workgroup per compute unit: 100 KiB of (unused) LDS keeps a second one off the unit
    constexpr int kLds = 100 * 1024;
    if (fold) {
        if (!allow_lds<mfma_probe_kernel<true>>(kLds)) return MI355_ELAUNCH;
        return launch(mfma_probe_kernel<true>, dim3(cus), dim3(64 * waves), kLds, (hipStream_t)stream,
                      (const v8i *)operands, (float *)sink, (int)iters);
    }
    if (!allow_lds<mfma_probe_kernel<false>>(kLds)) return MI355_ELAUNCH;
    return launch(mfma_probe_kernel<false>, dim3(cus), dim3(64 * waves), kLds, (hipStream_t)stream,
                  (const v8i *)operands, (float *)sink, (int)iters);
}

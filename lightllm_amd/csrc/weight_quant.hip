// Load-time 128x128 block weight quantizer (float -> e4m3fn + one fp32 scale per block).
// One workgroup per block.  bf16 weights with K % 8 == 0 take the vector kernel (16-byte loads, 16 lanes per
// 256-byte row segment, 8-byte stores); everything else the element-wise one.  Both divide in IEEE fp32.
// Semantics (fp8w8a8_block_quant_kernel.py:18-27 of the reference): scale = amax/448 is stored, values are
// divided by (scale + 1e-6) and cast without clamping; elements outside the matrix count as 0 for the amax.
#include "common.hpp"

namespace mi355 {

#pragma clang fp contract(off)

template <typename T>
__device__ __forceinline__ float load_as_f32(const T *p);
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t *p) { return as_f32((uint32_t)*p << 16); }
template <>
__device__ __forceinline__ float load_as_f32<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<_Float16>(const _Float16 *p) { return (float)*p; }

template <typename T>
__global__ __launch_bounds__(256) void block_weight_quant_kernel(const T *__restrict__ w, uint8_t *__restrict__ q,
                                                                 float *__restrict__ s, int64_t N, int64_t K,
                                                                 int kblocks) {
    __shared__ float red[4];
    const int bj = blockIdx.x, bi = blockIdx.y;
    const int tid = threadIdx.x;
    const int row = tid >> 1, half = tid & 1;
    const int64_t n = (int64_t)bi * 128 + row;
    const int64_t k0 = (int64_t)bj * 128 + half * 64;
    float v[64];
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 64; ++i) {
        const bool ok = n < N && k0 + i < K;
        v[i] = ok ? load_as_f32<T>(w + n * K + k0 + i) : 0.f;
        amax = fmaxf(amax, fabsf(v[i]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float scale = amax / 448.0f;
    const float div = scale + 1e-6f;
#pragma unroll
    for (int i = 0; i < 64; i += 4) {
        int pk = 0;
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[i] / div, v[i + 1] / div, pk, false);
        pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[i + 2] / div, v[i + 3] / div, pk, true);
        if (n < N) {
            if (k0 + i + 3 < K && (K & 3) == 0) {
                *(int *)(q + n * K + k0 + i) = pk;
            } else {
                for (int e = 0; e < 4; ++e)
                    if (k0 + i + e < K) q[n * K + k0 + i + e] = (uint8_t)((uint32_t)pk >> (8 * e));
            }
        }
    }
    if (tid == 0) s[(int64_t)bi * kblocks + bj] = scale;
}

// bf16, K % 8 == 0, 16-byte aligned rows: thread t owns chunks t, t+256, ... of the block's 128 x 16 chunks.
__global__ __launch_bounds__(256) void block_weight_quant_bf16_kernel(const uint16_t *__restrict__ w,
                                                                      uint8_t *__restrict__ q, float *__restrict__ s,
                                                                      int64_t N, int64_t K, int kblocks) {
    __shared__ float red[4];
    const int bj = blockIdx.x, bi = blockIdx.y;
    const int tid = threadIdx.x;
    v4i v[8];
    uint32_t m = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int c = tid + 256 * u;
        const int64_t n = (int64_t)bi * 128 + (c >> 4), k = (int64_t)bj * 128 + (c & 15) * 8;
        v[u] = (n < N && k < K) ? *(const v4i *)(w + n * K + k) : v4i{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t d = (uint32_t)v[u][i] & 0x7fff7fffu;  // |x| as integers keeps the float order
            m = max(m, max(d >> 16, d & 0xffffu));
        }
    }
    float amax = as_f32(m << 16);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float scale = amax / 448.0f;
    const float div = scale + 1e-6f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int c = tid + 256 * u;
        const int64_t n = (int64_t)bi * 128 + (c >> 4), k = (int64_t)bj * 128 + (c & 15) * 8;
        if (n >= N || k >= K) continue;
        float f[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = as_f32((uint32_t)v[u][i] << 16) / div;
            f[2 * i + 1] = as_f32((uint32_t)v[u][i] & 0xffff0000u) / div;
        }
        int w0 = 0, w1 = 0;
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w1, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
        *(v2i *)(q + n * K + k) = v2i{w0, w1};
    }
    if (tid == 0) s[(int64_t)bi * kblocks + bj] = scale;
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_block_weight_quant_fp8(const void *w, int32_t w_dtype, void *q, float *s, int64_t N, int64_t K,
                                            int32_t block, void *stream) {
    if (N < 0 || K < 0 || w_dtype < 0 || w_dtype > 2) return MI355_EINVAL;
    if (block != 128) return MI355_EUNSUPPORTED;
    if (N == 0 || K == 0) return MI355_OK;
    if (!w || !q || !s) return MI355_EINVAL;
    if ((uintptr_t)q & 3) return MI355_EALIGN;
    const int64_t nb = (N + 127) / 128, kb = (K + 127) / 128;
    if (nb > 65535 || kb >= (1ll << 31)) return MI355_EUNSUPPORTED;
    dim3 grid((uint32_t)kb, (uint32_t)nb);
    hipStream_t st = (hipStream_t)stream;
    if (w_dtype == 0 && K % 8 == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)q & 7) == 0)
        return launch(block_weight_quant_bf16_kernel, grid, dim3(256), 0, st, (const uint16_t *)w, (uint8_t *)q, s,
                           N, K, (int)kb);
    else if (w_dtype == 0)
        return launch(block_weight_quant_kernel<uint16_t>, grid, dim3(256), 0, st, (const uint16_t *)w,
                           (uint8_t *)q, s, N, K, (int)kb);
    else if (w_dtype == 1)
        return launch(block_weight_quant_kernel<float>, grid, dim3(256), 0, st, (const float *)w, (uint8_t *)q, s,
                           N, K, (int)kb);
    else
        return launch(block_weight_quant_kernel<_Float16>, grid, dim3(256), 0, st, (const _Float16 *)w,
                           (uint8_t *)q, s, N, K, (int)kb);
}

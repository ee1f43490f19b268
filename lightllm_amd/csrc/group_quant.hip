// per_token_group_quant_fp8 for gfx950: an HBM-streaming kernel.
//
// Data layout: x is bf16 [M,K] contiguous, so every group of 128 elements is 256 contiguous bytes
// and the whole tensor is a flat array of 16-byte chunks (8 bf16).  One lane owns one chunk; the 16
// lanes of a DPP row own one group; a wave covers 4 groups (1 KiB) per load instruction and keeps
// UNROLL such loads in flight.  The group amax is reduced inside the DPP row (4 steps), the scale
// is written by the row's first lane, and each lane writes its 8 output bytes with one 8-byte store.
//
// Algorithmic traffic per group: 256 B read + 128 B + 4 B written.
//
// Arithmetic (must reproduce IEEE fp32 division results bit for bit, see
// lightllm/common/basemodel/triton_kernel/quantization/fp8act_quant_kernel.py:53-57, 239-251):
//     amax = max(max|x|, eps);  s = amax / 448;  q = e4m3fn_rtne(clamp(x / s, -448, 448))
// Doing two IEEE divisions per element would make the kernel VALU-bound, so:
//   * s = amax/448 is formed as q0 = amax*c, s = fma(fma(-q0,448,amax), c, q0) with c = RN(1/448);
//     this equals RN(amax/448) for every bf16 amax and for the default eps (checked exhaustively on
//     the CPU); for any other eps the kernel takes a true division.
//   * x/s is formed as y0 = x*r, y = fma(fma(-y0,s,x), r, y0) with r = RN(1/s) (a true division,
//     once per lane).  For every pair (bf16 amax, bf16 |x| <= amax) this equals RN(x/s) whenever
//     |x/s| >= 2^-10, and below that both round to the e4m3 zero - also checked exhaustively on the CPU
//     (oracle_fast_quant_mismatches in the test oracle replays exactly these operations).
#include "common.hpp"

namespace mi355 {

#pragma clang fp contract(off)

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
    uint32_t t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
    return t > v ? t : v;
}

__device__ __forceinline__ uint32_t row16_max_u32(uint32_t v) {
    v = dpp_max_u32<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_max_u32<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_max_u32<0x141>(v);  // row_half_mirror: lane i <-> 7-i inside each half row
    v = dpp_max_u32<0x140>(v);  // row_mirror:      lane i <-> 15-i inside the row
    return v;
}

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    us2 x = __builtin_bit_cast(us2, a), y = __builtin_bit_cast(us2, b);
    us2 r = __builtin_elementwise_max(x, y);
    return __builtin_bit_cast(uint32_t, r);
}

// RN(x/s) wherever it matters (see the header), with the sign taken from x: the correction step turns
// -0 into +0, and the reference's -0/s = -0 keeps its sign bit through the cast (byte 0x80).
// No clamp is needed: |x| <= amax and s = RN(max(amax,eps)/448) bound |x/s| by 448*(1+2^-23), which the
// e4m3 cast rounds to 448, exactly what clamp-then-cast gives.
__device__ __forceinline__ float quot(float x, float s, float r) {
    float y0 = x * r;
    float e = __builtin_fmaf(-y0, s, x);
    float y = __builtin_fmaf(e, r, y0);
    return as_f32((as_u32(y) & 0x7fffffffu) | (as_u32(x) & 0x80000000u));
}

// Quantize one 16-byte chunk; the group amax is shared through the DPP row.
__device__ __forceinline__ void quant_chunk(const v4i &v, float eps, bool eps_is_default, v2i &out, float &scale) {
    uint32_t d0 = (uint32_t)v[0], d1 = (uint32_t)v[1], d2 = (uint32_t)v[2], d3 = (uint32_t)v[3];
    // |x| as integers: for non-negative floats the integer order is the float order.
    uint32_t m = pk_max_u16(pk_max_u16(d0 & 0x7fff7fffu, d1 & 0x7fff7fffu),
                            pk_max_u16(d2 & 0x7fff7fffu, d3 & 0x7fff7fffu));
    uint32_t hi = m >> 16, lo = m & 0xffffu;
    uint32_t mx = (hi > lo ? hi : lo) << 16;
    mx = row16_max_u32(mx);
    float amax = as_f32(mx);
    amax = amax > eps ? amax : eps;
    float s;
    if (eps_is_default) {
        const float c = 1.0f / 448.0f;
        float q0 = amax * c;
        s = __builtin_fmaf(__builtin_fmaf(-q0, 448.0f, amax), c, q0);
    } else {
        s = amax / 448.0f;
    }
    float r = 1.0f / s;
    float f[8];
    f[0] = as_f32(d0 << 16); f[1] = as_f32(d0 & 0xffff0000u);
    f[2] = as_f32(d1 << 16); f[3] = as_f32(d1 & 0xffff0000u);
    f[4] = as_f32(d2 << 16); f[5] = as_f32(d2 & 0xffff0000u);
    f[6] = as_f32(d3 << 16); f[7] = as_f32(d3 & 0xffff0000u);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = quot(f[i], s, r);
    int w0 = 0, w1 = 0;
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w1, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
    out[0] = w0;
    out[1] = w1;
    scale = s;
}

template <int UNROLL, bool ROW_MAJOR_SCALES>
__global__ __launch_bounds__(256) void group_quant_kernel(const v4i *__restrict__ x, v2i *__restrict__ q,
                                                          float *__restrict__ s, uint32_t total_chunks,
                                                          uint32_t groups_per_row, int64_t s_stride_m,
                                                          int64_t s_stride_g, float eps, int eps_is_default) {
    const uint32_t base = blockIdx.x * (256u * UNROLL) + threadIdx.x;
    v4i v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        uint32_t c = base + u * 256u;
        if (c < total_chunks) v[u] = __builtin_nontemporal_load(x + c);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        uint32_t c = base + u * 256u;
        if (c < total_chunks) {  // total_chunks is a multiple of 16: a DPP row is active or idle as a whole
            v2i o;
            float sc;
            quant_chunk(v[u], eps, eps_is_default != 0, o, sc);
            __builtin_nontemporal_store(o, q + c);
            if ((threadIdx.x & 15u) == 0) {
                uint32_t g = c >> 4;
                if (ROW_MAJOR_SCALES) {
                    s[g] = sc;
                } else {
                    uint32_t row = g / groups_per_row, col = g - row * groups_per_row;
                    s[(int64_t)row * s_stride_m + (int64_t)col * s_stride_g] = sc;
                }
            }
        }
    }
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_group_quant_fp8(const void *x, void *q, float *s, int64_t M, int64_t K, int32_t group,
                                     float eps, int64_t s_stride_m, int64_t s_stride_g, void *stream) {
    if (M < 0 || K < 0) return MI355_EINVAL;
    if (group != 128) return MI355_EUNSUPPORTED;
    if (K % group != 0) return MI355_ESHAPE;
    if (M == 0 || K == 0) return MI355_OK;
    if (!x || !q || !s) return MI355_EINVAL;
    if (((uintptr_t)x & 15) || ((uintptr_t)q & 7) || ((uintptr_t)s & 3)) return MI355_EALIGN;
    int64_t chunks = M * K / 8;
    if (chunks >= (int64_t)1 << 32) return MI355_EUNSUPPORTED;
    const uint32_t G = (uint32_t)(K / group);
    const bool row_major = (s_stride_g == 1 && s_stride_m == (int64_t)G) || (M == 1 && s_stride_g == 1) ||
                           (G == 1 && s_stride_m == 1);
    const int eps_default = (eps == 1e-10f) ? 1 : 0;
    constexpr int UNROLL = 4;
    uint32_t blocks = (uint32_t)((chunks + 256 * UNROLL - 1) / (256 * UNROLL));
    hipStream_t st = (hipStream_t)stream;
    if (row_major)
        hipLaunchKernelGGL((group_quant_kernel<UNROLL, true>), dim3(blocks), dim3(256), 0, st, (const v4i *)x,
                           (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g, eps, eps_default);
    else
        hipLaunchKernelGGL((group_quant_kernel<UNROLL, false>), dim3(blocks), dim3(256), 0, st, (const v4i *)x,
                           (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g, eps, eps_default);
    return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ELAUNCH;
}

// Device-side arithmetic of the 1x128 group quantizer (bf16 / fp16 / fp32 -> e4m3fn + fp32 scale), shared by the
// stand-alone quantizer and by the kernels that quantize what they have just computed.
//
// Arithmetic (must reproduce IEEE fp32 division results bit for bit, see
// lightllm/common/basemodel/triton_kernel/quantization/fp8act_quant_kernel.py:53-57, 239-251):
//     amax = max(max|x|, eps);  s = amax / 448;  q = e4m3fn_rtne(clamp(x / s, -448, 448))
// Doing two IEEE divisions per element would make the kernels VALU-bound, so:
//   * s = amax/448 is formed as q0 = amax*c, s = fma(fma(-q0,448,amax), c, q0) with c = RN(1/448);
//     this equals RN(amax/448) for every bf16 amax and for the default eps (checked exhaustively on
//     the CPU); calls with any other eps do not come here (they take quant_chunk_f32).
//   * x/s is formed as y0 = x*r, y = fma(fma(-y0,s,x), r, y0) with r = RN(1/s) (a true division,
//     once per lane).  For every pair (bf16 amax, bf16 |x| <= amax) this equals RN(x/s) whenever
//     |x/s| >= 2^-10, and below that both round to the e4m3 zero - also checked exhaustively on the CPU
//     (oracle_fast_quant_mismatches in the test oracle replays exactly these operations).
#pragma once
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

// A group that holds a NaN or an infinity (outside the reference's contract: its max and clamp leave NaN
// unspecified) is poisoned as a whole: scale = NaN, every byte 0x7F with the sign bit of its element.
__device__ __forceinline__ void nonfinite_chunk(uint32_t s0, uint32_t s1, uint32_t s2, uint32_t s3, uint32_t s4,
                                                uint32_t s5, uint32_t s6, uint32_t s7, v2i &out, float &scale) {
    out[0] = (int)(0x7f7f7f7fu | (s0 << 7) | (s1 << 15) | (s2 << 23) | (s3 << 31));
    out[1] = (int)(0x7f7f7f7fu | (s4 << 7) | (s5 << 15) | (s6 << 23) | (s7 << 31));
    scale = as_f32(0x7fc00000u);
}

// Quantize 8 consecutive fp32 values (fp16 / fp32 activations, widened by the caller) with true IEEE divisions:
// the two-FMA quotient above is only proven for bf16 inputs.
__device__ __forceinline__ void quant_chunk_f32(const float (&f)[8], float eps, v2i &out, float &scale) {
    uint32_t mx = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t a = as_u32(f[i]) & 0x7fffffffu;
        mx = a > mx ? a : mx;
    }
    mx = row16_max_u32(mx);
    if (mx > 0x7f7fffffu) {
        nonfinite_chunk(as_u32(f[0]) >> 31, as_u32(f[1]) >> 31, as_u32(f[2]) >> 31, as_u32(f[3]) >> 31,
                        as_u32(f[4]) >> 31, as_u32(f[5]) >> 31, as_u32(f[6]) >> 31, as_u32(f[7]) >> 31, out, scale);
        return;
    }
    float amax = as_f32(mx);
    amax = amax > eps ? amax : eps;
    const float s = amax / 448.0f;
    float y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        y[i] = f[i] / s;
        y[i] = y[i] > 448.0f ? 448.0f : y[i];
        y[i] = y[i] < -448.0f ? -448.0f : y[i];
    }
    int w0 = 0, w1 = 0;
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
    out[0] = w0;
    out[1] = w1;
    scale = s;
}

// Quantize one 16-byte chunk of bf16 with the default floor eps = 1e-10; the group amax is shared through the DPP row.
__device__ __forceinline__ void quant_chunk(const v4i &v, v2i &out, float &scale) {
    constexpr float eps = 1e-10f;
    uint32_t d0 = (uint32_t)v[0], d1 = (uint32_t)v[1], d2 = (uint32_t)v[2], d3 = (uint32_t)v[3];
    // |x| as integers: for non-negative floats the integer order is the float order.
    uint32_t m = pk_max_u16(pk_max_u16(d0 & 0x7fff7fffu, d1 & 0x7fff7fffu),
                            pk_max_u16(d2 & 0x7fff7fffu, d3 & 0x7fff7fffu));
    uint32_t hi = m >> 16, lo = m & 0xffffu;
    uint32_t mx = (hi > lo ? hi : lo) << 16;
    mx = row16_max_u32(mx);
    if (mx > 0x7f7fffffu) {  // the same for all 16 lanes of the group
        nonfinite_chunk((d0 >> 15) & 1u, d0 >> 31, (d1 >> 15) & 1u, d1 >> 31, (d2 >> 15) & 1u, d2 >> 31,
                        (d3 >> 15) & 1u, d3 >> 31, out, scale);
        return;
    }
    float amax = as_f32(mx);
    amax = amax > eps ? amax : eps;
    const float c = 1.0f / 448.0f;
    float q0 = amax * c;
    const float s = __builtin_fmaf(__builtin_fmaf(-q0, 448.0f, amax), c, q0);
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

}  // namespace mi355

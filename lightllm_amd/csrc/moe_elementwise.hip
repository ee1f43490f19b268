// The element-wise steps that sit between and after the two expert GEMMs of a MoE / FFN layer, for gfx950:
//
//   silu_and_mul                 bf16 [M, 2H] = [gate | up]  ->  bf16 [M, H]
//                                (lightllm/common/basemodel/triton_kernel/fused_moe/moe_silu_and_mul.py:9-93, "blocked" layout)
//   silu_and_mul + group quant   same input -> e4m3fn [M, H] + fp32 scale per 1x128 group, optionally only the
//                                first masked_m[e] rows of every expert of a [E, T, 2H] input
//                                (fused_moe/moe_silu_and_mul_mix_quant_ep.py:9-141)
//   moe_sum_reduce               bf16 [T, topk, H] -> bf16 [T, H], fp32 accumulation in ascending slot order
//                                (fused_moe/moe_sum_reduce.py:8-108)
//   block weight dequant         e4m3fn [N, K] * fp32 scale per 128x128 block -> bf16 [N, K]
//                                (lightllm/models/deepseek2/triton_kernel/weight_dequant.py:9-59)
//
// All four are HBM-streaming kernels: one lane owns 16 bytes of the narrowest operand, a wave covers whole
// contiguous 1 KiB runs, and several loads are kept in flight per lane.  Algorithmic bytes per output element:
// silu_and_mul 4 + 2, fused silu+quant 4 + 1 + 4/128, sum_reduce 2*topk + 2, dequant 1 + 2.
//
// SiLU arithmetic.  The reference computes  g = gate.to(f32); a = (g / (1 + exp(-g))).to(bf16); out = a * up
// (product rounded to bf16).  Here exp(-g) = 2^(-g*c1) * 2^(-g*c2) with log2(e) = c1 + c2 and c1 of 16
// significant bits, so the first product is exact for a bf16 g and the second factor is 1 + (a tiny term);
// the quotient is one reciprocal plus a residual correction.  Both are accurate to about an fp32 ulp, far
// below the bf16 rounding that follows.  The fused kernel runs exactly this code and then exactly the
// stand-alone quantizer's code, so its bytes and scales equal those of silu_and_mul followed by the group
// quantizer.
#include "quant_core.hpp"
#include <string.h>

namespace mi355 {

#pragma clang fp contract(off)

// FINITE: the caller knows that g is finite (silu_mul_chunk tests a whole chunk at once).
template <bool FINITE = false>
__device__ __forceinline__ float silu_f32(float g) {
    const float c1 = 1.44268798828125f;                // log2(e) rounded to 16 significant bits
    const float c2ln2 = 4.888495152e-06f;              // (log2(e) - c1) * ln(2)
    // below -88 the exponential would overflow; silu is below 1e-36 in magnitude from there on, so the
    // argument is held at -88 (the reference gives -0 or a subnormal there)
    const float gin = g;
    g = __builtin_fmaxf(g, -88.0f);
    float e0 = __builtin_amdgcn_exp2f(g * -c1);
    float e = __builtin_fmaf(e0, g * -c2ln2, e0);      // 2^(hi+lo) ~ 2^hi * (1 + lo*ln2)
    float d = 1.0f + e;
    float r = __builtin_amdgcn_rcpf(d);
    float y0 = g * r;
    float res = __builtin_fmaf(-y0, d, g);
    float out = __builtin_fmaf(res, r, y0);
    if constexpr (!FINITE) {
        // non-finite gates as g / (1 + exp(-g)) has them: NaN and -inf give NaN (-inf / inf), +inf gives +inf
        if (__builtin_amdgcn_classf(gin, 0x007)) out = __builtin_nanf("");
        if (__builtin_amdgcn_classf(gin, 0x200)) out = gin;
    }
    return out;
}

// bf16(silu(gate)) * up -> bf16, for the two bf16 values packed in one dword.
template <bool FINITE = false>
__device__ __forceinline__ uint32_t silu_mul_pk(uint32_t g2, uint32_t u2) {
    float g0 = as_f32(g2 << 16), g1 = as_f32(g2 & 0xffff0000u);
    float u0 = as_f32(u2 << 16), u1 = as_f32(u2 & 0xffff0000u);
    uint32_t a = pack_bf16x2(silu_f32<FINITE>(g0), silu_f32<FINITE>(g1));
    return pack_bf16x2(as_f32(a << 16) * u0, as_f32(a & 0xffff0000u) * u1);
}

// The kernels are bound by this arithmetic, so the non-finite cases (two class tests and two selects per element)
// are tested once per chunk: a bf16 is non-finite when its exponent field is all ones, and adding 0x0080 to the
// masked field of either half of a dword then carries into that half's top bit.
__device__ __forceinline__ v4i silu_mul_chunk(const v4i &g, const v4i &u) {
    uint32_t nonfinite = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) nonfinite |= (((uint32_t)g[i] & 0x7f807f80u) + 0x00800080u) & 0x80008000u;
    v4i o;
    if (nonfinite == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (int)silu_mul_pk<true>((uint32_t)g[i], (uint32_t)u[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (int)silu_mul_pk<false>((uint32_t)g[i], (uint32_t)u[i]);
    }
    return o;
}

// Row/column of output chunk c (8 elements) when a row holds cpr chunks.
struct ChunkPos {
    uint32_t row, col;
};
__device__ __forceinline__ ChunkPos chunk_pos(uint32_t c, uint32_t cpr) {
    ChunkPos p;
    p.row = c / cpr;
    p.col = c - p.row * cpr;
    return p;
}
// The position 256 chunks further on (q256 = 256 / cpr, r256 = 256 % cpr): no second division.
__device__ __forceinline__ ChunkPos chunk_next(ChunkPos p, uint32_t cpr, uint32_t q256, uint32_t r256) {
    p.row += q256;
    p.col += r256;
    if (p.col >= cpr) {
        p.col -= cpr;
        p.row += 1;
    }
    return p;
}

template <int UNROLL>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                           uint32_t total_chunks, uint32_t cpr, uint32_t q256,
                                                           uint32_t r256, int64_t in_stride_m, int64_t out_stride_m) {
    const uint32_t base = blockIdx.x * (256u * UNROLL) + threadIdx.x;
    v4i g[UNROLL], u[UNROLL];
    ChunkPos p[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        p[k] = k == 0 ? chunk_pos(base, cpr) : chunk_next(p[k - 1], cpr, q256, r256);
        if (base + k * 256u < total_chunks) {
            const uint16_t *row = in + (int64_t)p[k].row * in_stride_m;
            g[k] = __builtin_nontemporal_load((const v4i *)(row + (size_t)p[k].col * 8));
            u[k] = __builtin_nontemporal_load((const v4i *)(row + ((size_t)cpr + p[k].col) * 8));
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        if (base + k * 256u < total_chunks) {
            v4i o = silu_mul_chunk(g[k], u[k]);
            __builtin_nontemporal_store(o, (v4i *)(out + (int64_t)p[k].row * out_stride_m + (size_t)p[k].col * 8));
        }
    }
}

// Any H: one element per lane.
__global__ __launch_bounds__(256) void silu_and_mul_scalar_kernel(const uint16_t *__restrict__ in,
                                                                  uint16_t *__restrict__ out, int64_t total, int64_t H,
                                                                  int64_t in_stride_m, int64_t out_stride_m) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int64_t row = i / H, col = i - row * H;
    uint32_t g = in[row * in_stride_m + col], u = in[row * in_stride_m + H + col];
    out[row * out_stride_m + col] = (uint16_t)(silu_mul_pk(g, u) & 0xffffu);
}

// The other forms of the reference kernel (moe_silu_and_mul.py:46-71): "interleaved" input [g0, u0, g1, u1, ...]
// and the clamped variant  g = min(g, limit); u = clamp(u, -limit, limit);  out = (u + 1) * bf16(g * sigmoid(alpha*g)),
// where u stays bf16 (so the bound is limit rounded to bf16 and u + 1 is rounded to bf16 before the product).
// One element per lane: these forms are not on the fp8 block-quantized path.
__global__ __launch_bounds__(256) void silu_and_mul_general_kernel(const uint16_t *__restrict__ in,
                                                                   uint16_t *__restrict__ out, int64_t total, int64_t H,
                                                                   int64_t in_stride_m, int64_t out_stride_m,
                                                                   int interleaved, int use_limit, float limit,
                                                                   float limit_bf16, float alpha) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int64_t row = i / H, col = i - row * H;
    const uint16_t *r = in + row * in_stride_m;
    uint32_t gb = interleaved ? r[2 * col] : r[col];
    uint32_t ub = interleaved ? r[2 * col + 1] : r[H + col];
    if (!use_limit) {
        out[row * out_stride_m + col] = (uint16_t)(silu_mul_pk(gb, ub) & 0xffffu);
        return;
    }
    float g = as_f32(gb << 16), u = as_f32(ub << 16);
    g = g < limit ? g : (g != g ? g : limit);                  // min that keeps a NaN gate
    u = u > -limit_bf16 ? u : (u != u ? u : -limit_bf16);
    u = u < limit_bf16 ? u : (u != u ? u : limit_bf16);
    // 1 / (1 + exp(-g*alpha)) * g, the reference's order of operations
    const float c1 = 1.44269504088896341f;
    const float t = g * alpha;
    const float e = __builtin_amdgcn_exp2f(__builtin_fmaxf(t, -88.0f) * -c1);
    const float d = 1.0f + e;
    float rcp = __builtin_amdgcn_rcpf(d);
    rcp = __builtin_fmaf(__builtin_fmaf(-d, rcp, 1.0f), rcp, rcp);   // one Newton step: 1/d to an ulp
    const float sg = rcp * g;
    const float gs = as_f32(f32_to_bf16_bits(sg) << 16);
    const float up1 = as_f32(f32_to_bf16_bits(u + 1.0f) << 16);
    out[row * out_stride_m + col] = (uint16_t)f32_to_bf16_bits(up1 * gs);
}

// One lane = one 8-element chunk of the OUTPUT; 16 lanes (a DPP row) = one quantization group.
// A group never straddles rows (H % 128 == 0), so the masked-row test is uniform inside a DPP row.
template <int UNROLL, bool MASKED>
__global__ __launch_bounds__(256) void silu_mul_quant_kernel(const uint16_t *__restrict__ in, v2i *__restrict__ q,
                                                             float *__restrict__ s, uint32_t total_chunks,
                                                             uint32_t cpr, uint32_t q256, uint32_t r256,
                                                             int64_t in_stride_m, int64_t s_stride_m,
                                                             int64_t s_stride_g, const int32_t *__restrict__ masked_m,
                                                             uint32_t rows_per_expert) {
    const uint32_t base = blockIdx.x * (256u * UNROLL) + threadIdx.x;
    v4i g[UNROLL], u[UNROLL];
    ChunkPos p[UNROLL];
    bool live[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        p[k] = k == 0 ? chunk_pos(base, cpr) : chunk_next(p[k - 1], cpr, q256, r256);
        live[k] = base + k * 256u < total_chunks;
        if (MASKED && live[k]) {
            uint32_t e = p[k].row / rows_per_expert, t = p[k].row - e * rows_per_expert;
            live[k] = (int32_t)t < masked_m[e];
        }
        if (live[k]) {
            const uint16_t *row = in + (int64_t)p[k].row * in_stride_m;
            g[k] = __builtin_nontemporal_load((const v4i *)(row + (size_t)p[k].col * 8));
            u[k] = __builtin_nontemporal_load((const v4i *)(row + ((size_t)cpr + p[k].col) * 8));
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; ++k) {
        if (live[k]) {
            v4i a = silu_mul_chunk(g[k], u[k]);
            v2i o;
            float sc;
            quant_chunk(a, o, sc);
            __builtin_nontemporal_store(o, q + (base + k * 256u));
            if ((threadIdx.x & 15u) == 0)
                s[(int64_t)p[k].row * s_stride_m + (int64_t)(p[k].col >> 4) * s_stride_g] = sc;
        }
    }
}

template <int UNROLL>
__global__ __launch_bounds__(256) void moe_sum_reduce_kernel(const v4i *__restrict__ in, v4i *__restrict__ out,
                                                             uint32_t total_chunks, uint32_t cpr, int32_t topk) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= total_chunks) return;
    ChunkPos p = chunk_pos(c, cpr);
    const v4i *src = in + (size_t)p.row * topk * cpr + p.col;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    int k = 0;
    for (; k + UNROLL <= topk; k += UNROLL) {
        v4i v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) v[j] = __builtin_nontemporal_load(src + (size_t)(k + j) * cpr);
#pragma unroll
        for (int j = 0; j < UNROLL; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t d = (uint32_t)v[j][i];
                acc[2 * i] += as_f32(d << 16);
                acc[2 * i + 1] += as_f32(d & 0xffff0000u);
            }
    }
    for (; k < topk; ++k) {
        v4i v = __builtin_nontemporal_load(src + (size_t)k * cpr);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t d = (uint32_t)v[i];
            acc[2 * i] += as_f32(d << 16);
            acc[2 * i + 1] += as_f32(d & 0xffff0000u);
        }
    }
    v4i o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (int)pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
    __builtin_nontemporal_store(o, out + c);
}

__global__ __launch_bounds__(256) void moe_sum_reduce_scalar_kernel(const uint16_t *__restrict__ in,
                                                                    uint16_t *__restrict__ out, int64_t total, int64_t H,
                                                                    int32_t topk) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int64_t row = i / H, col = i - row * H;
    float acc = 0.f;
    for (int k = 0; k < topk; ++k) acc += as_f32((uint32_t)in[(row * topk + k) * H + col] << 16);
    out[i] = (uint16_t)f32_to_bf16_bits(acc);
}

// fp32 -> bf16 bits that also keeps NaN a NaN (an e4m3fn weight byte 0x7f/0xff decodes to NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits_nan(float f) {
    uint32_t u = as_u32(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return f32_to_bf16_bits(f);
}

// One lane = two pieces of 8 consecutive weights (K % 16 == 0), 256 pieces apart: a wave reads 512 contiguous bytes
// and writes 1 KiB contiguous bytes per instruction (16 weights per lane in one piece made the two 16-byte stores of
// a lane 32 bytes apart from its neighbours': 198 us for [36864,7168] against 124).
__global__ __launch_bounds__(256) void weight_dequant_kernel(const v2i *__restrict__ q, const float *__restrict__ s,
                                                             v4i *__restrict__ out, uint32_t total_pieces, uint32_t ppr,
                                                             uint32_t kblocks) {
    const uint32_t first = blockIdx.x * 512u + threadIdx.x;
    v2i v[2];
    float sc[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t c = first + 256u * h;
        if (c < total_pieces) {
            ChunkPos p = chunk_pos(c, ppr);
            sc[h] = s[(size_t)(p.row >> 7) * kblocks + (p.col >> 4)];
            v[h] = __builtin_nontemporal_load(q + c);
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t c = first + 256u * h;
        if (c >= total_pieces) continue;
        v4i o;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            auto a = __builtin_amdgcn_cvt_pk_f32_fp8(v[h][i], false);
            auto b = __builtin_amdgcn_cvt_pk_f32_fp8(v[h][i], true);
            o[2 * i] = (int)(f32_to_bf16_bits_nan(a[0] * sc[h]) | (f32_to_bf16_bits_nan(a[1] * sc[h]) << 16));
            o[2 * i + 1] = (int)(f32_to_bf16_bits_nan(b[0] * sc[h]) | (f32_to_bf16_bits_nan(b[1] * sc[h]) << 16));
        }
        __builtin_nontemporal_store(o, out + c);
    }
}

__global__ __launch_bounds__(256) void weight_dequant_scalar_kernel(const uint8_t *__restrict__ q,
                                                                    const float *__restrict__ s,
                                                                    uint16_t *__restrict__ out, int64_t total, int64_t K,
                                                                    int64_t kblocks) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int64_t row = i / K, col = i - row * K;
    auto a = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[i], false);
    out[i] = (uint16_t)f32_to_bf16_bits_nan(a[0] * s[(row >> 7) * kblocks + (col >> 7)]);
}

// host-side bf16 rounding (nearest even) of the clamp bound
static inline uint32_t f32_to_bf16_bits_host(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
static inline float as_f32_host(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_silu_and_mul(const void *in, void *out, int64_t M, int64_t H, int64_t in_stride_m,
                                  int64_t out_stride_m, void *stream) {
    if (M < 0 || H < 0) return MI355_EINVAL;
    if (M == 0 || H == 0) return MI355_OK;
    if (!in || !out) return MI355_EINVAL;
    if (in_stride_m < 2 * H || out_stride_m < H) return MI355_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (H % 8 == 0) && (in_stride_m % 8 == 0) && (out_stride_m % 8 == 0) && !((uintptr_t)in & 15) &&
                     !((uintptr_t)out & 15);
    if (vec) {
        int64_t chunks = M * (H / 8);
        if (chunks >= (int64_t)1 << 32) return MI355_EUNSUPPORTED;
        constexpr int UNROLL = 4;
        const uint32_t cpr = (uint32_t)(H / 8);
        uint32_t blocks = (uint32_t)((chunks + 256 * UNROLL - 1) / (256 * UNROLL));
        return launch((silu_and_mul_kernel<UNROLL>), dim3(blocks), dim3(256), 0, st, (const uint16_t *)in,
                           (uint16_t *)out, (uint32_t)chunks, cpr, 256u / cpr, 256u % cpr, in_stride_m, out_stride_m);
    } else {
        int64_t total = M * H;
        if ((total + 255) / 256 >= (int64_t)1 << 31) return MI355_EUNSUPPORTED;
        return launch(silu_and_mul_scalar_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st,
                           (const uint16_t *)in, (uint16_t *)out, total, H, in_stride_m, out_stride_m);
    }
}

extern "C" int mi355_silu_and_mul_ex(const void *in, void *out, int64_t M, int64_t H, int64_t in_stride_m,
                                     int64_t out_stride_m, int32_t interleaved, int32_t use_limit, float limit,
                                     float alpha, void *stream) {
    if (M < 0 || H < 0) return MI355_EINVAL;
    if (M == 0 || H == 0) return MI355_OK;
    if (!in || !out) return MI355_EINVAL;
    if (in_stride_m < 2 * H || out_stride_m < H) return MI355_ESHAPE;
    if (!interleaved && !use_limit) return mi355_silu_and_mul(in, out, M, H, in_stride_m, out_stride_m, stream);
    const int64_t total = M * H;
    if ((total + 255) / 256 >= (int64_t)1 << 31) return MI355_EUNSUPPORTED;
    const float limit_bf16 = as_f32_host((uint32_t)f32_to_bf16_bits_host(limit) << 16);
    return launch(silu_and_mul_general_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                  (const uint16_t *)in, (uint16_t *)out, total, H, in_stride_m, out_stride_m, interleaved ? 1 : 0,
                  use_limit ? 1 : 0, limit, limit_bf16, alpha);
}

extern "C" int mi355_silu_and_mul_group_quant_fp8(const void *in, void *q, float *s, int64_t M, int64_t H,
                                                  int64_t in_stride_m, int32_t group, int64_t s_stride_m,
                                                  int64_t s_stride_g, const int32_t *masked_m,
                                                  int64_t rows_per_expert, void *stream) {
    if (M < 0 || H < 0) return MI355_EINVAL;
    if (group != 128) return MI355_EUNSUPPORTED;
    if (H % group != 0) return MI355_ESHAPE;
    if (M == 0 || H == 0) return MI355_OK;
    if (!in || !q || !s) return MI355_EINVAL;
    if (in_stride_m < 2 * H) return MI355_ESHAPE;
    if (masked_m && (rows_per_expert <= 0 || M % rows_per_expert != 0)) return MI355_ESHAPE;
    if (((uintptr_t)in & 15) || (in_stride_m % 8) || ((uintptr_t)q & 7) || ((uintptr_t)s & 3)) return MI355_EALIGN;
    int64_t chunks = M * (H / 8);
    if (chunks >= (int64_t)1 << 32) return MI355_EUNSUPPORTED;
    constexpr int UNROLL = 4;
    const uint32_t cpr = (uint32_t)(H / 8);
    uint32_t blocks = (uint32_t)((chunks + 256 * UNROLL - 1) / (256 * UNROLL));
    hipStream_t st = (hipStream_t)stream;
    if (masked_m)
        return launch((silu_mul_quant_kernel<UNROLL, true>), dim3(blocks), dim3(256), 0, st,
                           (const uint16_t *)in, (v2i *)q, s, (uint32_t)chunks, cpr, 256u / cpr, 256u % cpr,
                           in_stride_m, s_stride_m, s_stride_g, masked_m, (uint32_t)rows_per_expert);
    else
        return launch((silu_mul_quant_kernel<UNROLL, false>), dim3(blocks), dim3(256), 0, st,
                           (const uint16_t *)in, (v2i *)q, s, (uint32_t)chunks, cpr, 256u / cpr, 256u % cpr,
                           in_stride_m, s_stride_m, s_stride_g, masked_m, 1u);
}

extern "C" int mi355_moe_sum_reduce(const void *in, void *out, int64_t T, int32_t topk, int64_t H, void *stream) {
    if (T < 0 || H < 0 || topk < 0) return MI355_EINVAL;
    if (T == 0 || H == 0) return MI355_OK;
    if (!out || (!in && topk > 0)) return MI355_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (H % 8 == 0 && !((uintptr_t)in & 15) && !((uintptr_t)out & 15)) {
        int64_t chunks = T * (H / 8);
        if (chunks >= (int64_t)1 << 32) return MI355_EUNSUPPORTED;
        return launch((moe_sum_reduce_kernel<4>), dim3((uint32_t)((chunks + 255) / 256)), dim3(256), 0, st,
                           (const v4i *)in, (v4i *)out, (uint32_t)chunks, (uint32_t)(H / 8), topk);
    } else {
        int64_t total = T * H;
        if ((total + 255) / 256 >= (int64_t)1 << 31) return MI355_EUNSUPPORTED;
        return launch(moe_sum_reduce_scalar_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st,
                           (const uint16_t *)in, (uint16_t *)out, total, H, topk);
    }
}

extern "C" int mi355_block_weight_dequant(const void *q, const float *s, void *out, int64_t N, int64_t K,
                                          int32_t block, void *stream) {
    if (N < 0 || K < 0) return MI355_EINVAL;
    if (block != 128) return MI355_EUNSUPPORTED;
    if (N == 0 || K == 0) return MI355_OK;
    if (!q || !s || !out) return MI355_EINVAL;
    const int64_t kblocks = (K + block - 1) / block;
    hipStream_t st = (hipStream_t)stream;
    if (K % 16 == 0 && !((uintptr_t)q & 15) && !((uintptr_t)out & 15)) {
        int64_t pieces = N * (K / 8);
        if (pieces >= (int64_t)1 << 32) return MI355_EUNSUPPORTED;
        return launch(weight_dequant_kernel, dim3((uint32_t)((pieces + 511) / 512)), dim3(256), 0, st,
                           (const v2i *)q, s, (v4i *)out, (uint32_t)pieces, (uint32_t)(K / 8), (uint32_t)kblocks);
    } else {
        int64_t total = N * K;
        if ((total + 255) / 256 >= (int64_t)1 << 31) return MI355_EUNSUPPORTED;
        return launch(weight_dequant_scalar_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st,
                           (const uint8_t *)q, s, (uint16_t *)out, total, K, kblocks);
    }
}

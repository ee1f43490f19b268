// per_token_group_quant_fp8 for gfx950: an HBM-streaming kernel.
//
// Data layout (bf16, the hot path): x is [M,K] contiguous, so every group of 128 elements is 256 contiguous bytes
// and the whole tensor is a flat array of 16-byte chunks (8 bf16).  One lane owns one chunk; the 16
// lanes of a DPP row own one group; a wave covers 4 groups (1 KiB) per load instruction and keeps
// UNROLL such loads in flight.  The group amax is reduced inside the DPP row (4 steps), the scale
// is written by the row's first lane, and each lane writes its 8 output bytes with one 8-byte store.
//
// Algorithmic traffic per group: 256 B read + 128 B + 4 B written.
//
// The arithmetic (exact IEEE quotients without per-element divisions) lives in quant_core.hpp.
#include <type_traits>

#include "quant_core.hpp"

namespace mi355 {

#pragma clang fp contract(off)

template <int UNROLL, bool ROW_MAJOR_SCALES>
__global__ __launch_bounds__(256) void group_quant_kernel(const v4i *__restrict__ x, v2i *__restrict__ q,
                                                          float *__restrict__ s, uint32_t total_chunks,
                                                          uint32_t groups_per_row, int64_t s_stride_m,
                                                          int64_t s_stride_g) {
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
            quant_chunk(v[u], o, sc);
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

// fp16 and fp32 activations (the reference widens any input dtype to fp32 first,
// quantization/fp8act_quant_kernel.py:52): one lane = 8 elements, true divisions.  Not the hot path.
template <typename T>
__global__ __launch_bounds__(256) void group_quant_wide_kernel(const T *__restrict__ x, v2i *__restrict__ q,
                                                               float *__restrict__ s, uint32_t total_chunks,
                                                               uint32_t groups_per_row, int64_t s_stride_m,
                                                               int64_t s_stride_g, float eps) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= total_chunks) return;  // total_chunks is a multiple of 16: a DPP row is active or idle as a whole
    float f[8];
    if constexpr (sizeof(T) == 4) {
        const v4i a = __builtin_nontemporal_load((const v4i *)x + 2 * (size_t)c);
        const v4i b = __builtin_nontemporal_load((const v4i *)x + 2 * (size_t)c + 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[i] = as_f32((uint32_t)a[i]);
            f[4 + i] = as_f32((uint32_t)b[i]);
        }
    } else if constexpr (sizeof(T) == 2 && !__is_same(T, _Float16)) {
        // bf16 bits (T = uint16_t): the path of a non-default eps, whose floor is no bf16 value
        const v4i a = __builtin_nontemporal_load((const v4i *)x + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = as_f32((uint32_t)a[i] << 16);
            f[2 * i + 1] = as_f32((uint32_t)a[i] & 0xffff0000u);
        }
    } else {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 h = __builtin_bit_cast(h8, __builtin_nontemporal_load((const v4i *)x + c));
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
    }
    v2i o;
    float sc;
    quant_chunk_f32(f, eps, o, sc);
    __builtin_nontemporal_store(o, q + c);
    if ((threadIdx.x & 15u) == 0) {
        const uint32_t g = c >> 4;
        const uint32_t row = g / groups_per_row, col = g - row * groups_per_row;
        s[(int64_t)row * s_stride_m + (int64_t)col * s_stride_g] = sc;
    }
}

// Any other group size (the reference's kernel takes whatever divides K, e.g. the whole row for a per-token
// scale: quantization/fp8act_quant_kernel.py:18-60): one wave per group, two passes over the group (the second
// one is served by the caches), true IEEE divisions, the same rule for groups that hold a NaN or an infinity.
// VEC: 8 elements per lane and access (group % 8 == 0 and 16-byte aligned rows), else one element.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void group_quant_any_kernel(const T *__restrict__ x, uint8_t *__restrict__ q,
                                                              float *__restrict__ s, int64_t total_groups,
                                                              int64_t groups_per_row, int64_t K, int32_t group,
                                                              int64_t s_stride_m, int64_t s_stride_g, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t g = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= total_groups) return;  // the same for the whole wave
    const int64_t row = g / groups_per_row, col = g - row * groups_per_row;
    const T *xg = x + row * K + col * group;
    uint8_t *qg = q + row * K + col * group;
    // 8 consecutive elements (VEC) or one, widened to fp32
    auto fetch = [&](int c, float (&f)[VEC ? 8 : 1]) {
        if constexpr (!VEC) {
            if constexpr (std::is_same<T, uint16_t>::value) f[0] = as_f32((uint32_t)xg[c] << 16);
            else f[0] = (float)xg[c];
        } else if constexpr (sizeof(T) == 4) {
            const v4i a = *((const v4i *)xg + 2 * c), b = *((const v4i *)xg + 2 * c + 1);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f[i] = as_f32((uint32_t)a[i]);
                f[4 + i] = as_f32((uint32_t)b[i]);
            }
        } else if constexpr (std::is_same<T, uint16_t>::value) {
            const v4i a = *((const v4i *)xg + c);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f[2 * i] = as_f32((uint32_t)a[i] << 16);
                f[2 * i + 1] = as_f32((uint32_t)a[i] & 0xffff0000u);
            }
        } else {
            typedef _Float16 h8 __attribute__((ext_vector_type(8)));
            const h8 h = __builtin_bit_cast(h8, *((const v4i *)xg + c));
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
        }
    };
    constexpr int W = VEC ? 8 : 1;
    const int n = group / W;  // accesses per group
    uint32_t mx = 0;
    for (int c = lane; c < n; c += 64) {
        float f[W];
        fetch(c, f);
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const uint32_t a = as_u32(f[i]) & 0x7fffffffu;
            mx = a > mx ? a : mx;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)mx, off, 64);
        mx = o > mx ? o : mx;
    }
    const bool poisoned = mx > 0x7f7fffffu;
    float amax = as_f32(mx);
    amax = amax > eps ? amax : eps;
    const float sc = poisoned ? as_f32(0x7fc00000u) : amax / 448.0f;
    for (int c = lane; c < n; c += 64) {
        float f[W];
        fetch(c, f);
        uint8_t b[W];
#pragma unroll
        for (int i = 0; i < W; ++i) {
            if (poisoned) {
                b[i] = (uint8_t)(0x7fu | ((as_u32(f[i]) >> 31) << 7));
            } else {
                float y = f[i] / sc;
                y = y > 448.0f ? 448.0f : y;
                y = y < -448.0f ? -448.0f : y;
                b[i] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false) & 0xff);
            }
        }
        if constexpr (VEC) {
            v2i o;
            o[0] = (int)((uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24));
            o[1] = (int)((uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24));
            *((v2i *)qg + c) = o;
        } else {
            qg[c] = b[0];
        }
    }
    if (lane == 0) s[row * s_stride_m + col * s_stride_g] = sc;
}

template <typename T>
static int launch_any(const void *x, void *q, float *s, int64_t M, int64_t K, int32_t group, float eps,
                      int64_t s_stride_m, int64_t s_stride_g, hipStream_t st) {
    const int64_t G = K / group, total = M * G;
    if ((total + 3) / 4 >= (1ll << 31)) return MI355_EUNSUPPORTED;
    const dim3 grid((uint32_t)((total + 3) / 4));
    const bool vec = group % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 7) == 0;
    if (vec)
        return launch((group_quant_any_kernel<T, true>), grid, dim3(256), 0, st, (const T *)x, (uint8_t *)q, s, total, G, K,
                      group, s_stride_m, s_stride_g, eps);
    return launch((group_quant_any_kernel<T, false>), grid, dim3(256), 0, st, (const T *)x, (uint8_t *)q, s, total, G, K,
                  group, s_stride_m, s_stride_g, eps);
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_group_quant_fp8(const void *x, int32_t x_dtype, void *q, float *s, int64_t M, int64_t K,
                                     int32_t group, float eps, int64_t s_stride_m, int64_t s_stride_g, void *stream) {
    if (M < 0 || K < 0 || x_dtype < 0 || x_dtype > 2) return MI355_EINVAL;
    if (group <= 0) return MI355_EINVAL;
    if (K % group != 0) return MI355_ESHAPE;
    if (M == 0 || K == 0) return MI355_OK;
    if (!x || !q || !s) return MI355_EINVAL;
    if (group != 128) {
        if ((uintptr_t)s & 3) return MI355_EALIGN;
        hipStream_t st_any = (hipStream_t)stream;
        if (x_dtype == MI355_DTYPE_F32) return launch_any<float>(x, q, s, M, K, group, eps, s_stride_m, s_stride_g, st_any);
        if (x_dtype == MI355_DTYPE_F16) return launch_any<_Float16>(x, q, s, M, K, group, eps, s_stride_m, s_stride_g, st_any);
        return launch_any<uint16_t>(x, q, s, M, K, group, eps, s_stride_m, s_stride_g, st_any);
    }
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
    if (x_dtype == MI355_DTYPE_F32)
        return launch(group_quant_wide_kernel<float>, dim3((uint32_t)((chunks + 255) / 256)), dim3(256), 0, st,
                      (const float *)x, (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g, eps);
    if (x_dtype == MI355_DTYPE_F16)
        return launch(group_quant_wide_kernel<_Float16>, dim3((uint32_t)((chunks + 255) / 256)), dim3(256), 0, st,
                      (const _Float16 *)x, (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g, eps);
    // The two-FMA quotient of the bf16 kernel is proven for scales RN(amax/448) of a bf16 amax and of the default
    // floor 1e-10 only; with any other eps a group below the floor has a scale outside that set, so such calls take
    // the kernel with true divisions (fp8act_quant_kernel.py:63-113 hands eps through to the kernel).
    if (!eps_default)
        return launch(group_quant_wide_kernel<uint16_t>, dim3((uint32_t)((chunks + 255) / 256)), dim3(256), 0, st,
                      (const uint16_t *)x, (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g, eps);
    if (row_major)
        return launch((group_quant_kernel<UNROLL, true>), dim3(blocks), dim3(256), 0, st, (const v4i *)x,
                           (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g);
    else
        return launch((group_quant_kernel<UNROLL, false>), dim3(blocks), dim3(256), 0, st, (const v4i *)x,
                           (v2i *)q, s, (uint32_t)chunks, G, s_stride_m, s_stride_g);
}

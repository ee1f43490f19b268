// Shared device helpers for the gfx950 block-FP8 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>
#include <utility>

#include "../../include/mi355_fp8.h"

namespace mi355 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short us2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kBlockK = 128;  // K extent of one scale step (= the 128x128 weight block, the 1x128 activation group)
constexpr int kBlockN = 128;

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// fp32 -> bf16 bits, round to nearest even, NaN kept a NaN: gfx950 converts two floats per instruction
// (v_cvt_pk_bf16_f32).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    v2f v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    return (uint32_t)__builtin_bit_cast(unsigned short, (__bf16)f);
}
// The GEMM outputs: bf16, or fp16 when the caller's tensors are (the reference casts the fp32 accumulator to the
// dtype of C, quantization/fp8w8a8_block_gemm_kernel.py:78).  `f16` is the same for every lane of a launch.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_out2(float lo, float hi, int f16) {
    v2f v = {lo, hi};
    if (f16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t out_bits(float f, int f16) {
    if (f16) return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
    return f32_to_bf16_bits(f);
}

// D(16x16, fp32) = A(16x128, e4m3) * B(128x16, e4m3) + C on the CDNA4 matrix core.
// Lane l feeds row/col (l % 16) and the 32 K-bytes numbered (l / 16); both operands use the same
// K numbering, so any consistent placement of K bytes in the two registers gives the same dot product.
// D: lane l holds column (l % 16), rows 4*(l/16) + 0..3.
// Format selectors 0/0 = e4m3 for both operands; block-scale operands 0/0 select the unscaled instruction.
__device__ __forceinline__ v4f mfma_16x16x128_fp8(v8i a, v8i b, v4f c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// Byte address of a __shared__ object inside the workgroup's LDS allocation.
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

// Asynchronous 16-byte-per-lane copy global -> LDS that bypasses the register file.
// Lane l's 16 bytes at (gbase + voff) land at LDS byte (lds_base + 16*l): one call fills 1 KiB.
// lds_base and gbase are wave-uniform.  Completion is tracked by vmcnt; the compiler does not
// see the LDS write, so the caller orders it with wait_vmcnt<>() and a workgroup barrier.
__device__ __forceinline__ void dma_g2l_b128(uint32_t lds_base, const void *gbase, uint32_t voff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_base), "v"(voff), "s"(gbase)
        : "memory");
}
// Same with 4 bytes per lane (256 B per call), used for scale vectors.
__device__ __forceinline__ void dma_g2l_b32(uint32_t lds_base, const void *gbase, uint32_t voff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dword %1, %2"
        :
        : "s"(lds_base), "v"(voff), "s"(gbase)
        : "memory");
}

// 16-byte loads and stores that read past / write through the per-XCD L2 (cache policy sc1, what an agent-scope
// relaxed atomic access compiles to on gfx950), for data exchanged between workgroups of one launch.  They are
// ordinary memory operations to the compiler, so a batch of loads is issued back to back and waited for once.
// The buffer resource covers 2 GiB from `base`.
struct Sc1Buffer {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ explicit Sc1Buffer(const void *base)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7fffffff, 0x00020000)) {}
    __device__ __forceinline__ v4f load(uint32_t byte_off) const {
        return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_off, 0, 16));
    }
    __device__ __forceinline__ void store(uint32_t byte_off, v4f v) const {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), rsrc, (int)byte_off, 0, 16);
    }
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // gfx9 encoding of s_waitcnt: vmcnt low bits [3:0], high bits [15:14]; expcnt [6:4]=7, lgkmcnt [11:8]=15 (no wait).
    __builtin_amdgcn_s_waitcnt((N & 0xf) | ((N >> 4) << 14) | (0x7 << 4) | (0xf << 8));
}

// Workgroup barrier that waits for this wave's LDS traffic only (lgkmcnt 0; vmcnt untouched).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xf | (0x3 << 14) | (0x7 << 4) | (0 << 8));
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // compiler only: no LDS access may move across the barrier
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
}

// 16B-chunk swizzle for LDS tiles with 128-byte rows (8 chunks per row): physical chunk = logical ^ swz(row).
// For 16 consecutive rows read at one logical chunk the (row parity, physical chunk) pairs are all
// distinct, and for 8 consecutive rows the physical chunks are all distinct, so a ds_read_b128 of a
// 16-row operand slice is bank-conflict free whether the LDS serves 128 or 256 bytes per clock.
__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row & 7u) ^ ((row >> 3) & 1u); }

// ---- host side: launches and per-device facts ------------------------------------------------------------
// A launch reports the status of its own hipLaunchKernel call.  (hipGetLastError() after a <<<>>> launch
// would also return, and clear, an error left behind by an unrelated earlier runtime call of the host
// framework.)
namespace detail {
template <typename... P, size_t... I>
inline hipError_t launch_impl(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t st,
                              std::tuple<P...> &params, std::index_sequence<I...>) {
    void *ptrs[] = {(void *)&std::get<I>(params)...};
    return hipLaunchKernel((const void *)kernel, grid, block, ptrs, lds, st);
}
}  // namespace detail

template <typename... P, typename... A>
inline int launch(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds, hipStream_t st, A &&...args) {
    static_assert(sizeof...(P) == sizeof...(A), "argument count differs from the kernel's parameter list");
    std::tuple<P...> params{static_cast<P>(args)...};
    return detail::launch_impl(kernel, grid, block, lds, st, params, std::index_sequence_for<P...>{}) == hipSuccess
               ? MI355_OK
               : MI355_ELAUNCH;
}

constexpr int kMaxDevices = 64;

inline int current_device() {
    int dev = 0;
    return hipGetDevice(&dev) == hipSuccess ? dev : -1;
}

// Compute units of the current device (looked up once per device).
inline int device_cus() {
    static std::atomic<int> cus[kMaxDevices];
    const int dev = current_device();
    if (dev >= 0 && dev < kMaxDevices) {
        const int known = cus[dev].load(std::memory_order_relaxed);
        if (known > 0) return known;
    }
    int n = 0;
    if (dev < 0 || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    if (dev >= 0 && dev < kMaxDevices) cus[dev].store(n, std::memory_order_relaxed);
    return n;
}

// Raises the dynamic-LDS ceiling of Kernel to `bytes` on the current device, once per device: the attribute
// belongs to the device's copy of the function.  Setting it enqueues nothing.
template <auto Kernel>
inline bool allow_lds(int bytes) {
    static std::atomic<uint64_t> done{0};
    const int dev = current_device();
    const bool tracked = dev >= 0 && dev < kMaxDevices;
    if (tracked && ((done.load(std::memory_order_acquire) >> dev) & 1u)) return true;
    if (hipFuncSetAttribute((const void *)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
        return false;
    if (tracked) done.fetch_or(1ull << dev, std::memory_order_release);
    return true;
}

}  // namespace mi355

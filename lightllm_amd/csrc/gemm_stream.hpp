// Block-scaled FP8 GEMM for decode-size M (<= 64) on gfx950: a weight-streaming kernel.
//
// At these sizes the GEMM is a single pass over the N x K weight bytes, so the kernel is built around the
// memory system, not the MFMA: every wave issues plain 16-byte-per-lane global loads in which 8 consecutive
// lanes cover one 128-byte row segment (fully coalesced), keeps 1-3 K-steps of them in flight in registers,
// and only then rearranges the bytes into MFMA operand order through a small wave-private LDS area
// (ds_write_b128 / ds_read_b128, no workgroup barrier in the loop).  Loads that target LDS directly
// (global_load_lds) sustain visibly less HBM bandwidth than plain loads on this part, which is why the
// streaming path does not use them.
//
// Work decomposition
//   CTA = 4 waves, owns 16*TNW weight rows (n) and a contiguous range of K steps (cross-CTA split-K only when N
//   alone gives too few CTAs; TNW is picked so that N / (16*TNW) is about the number of CUs).  Inside the CTA
//   the waves take the K steps round-robin, so the four waves together read 512 consecutive bytes of every
//   row; each wave multiplies all its rows (TNW MFMA row blocks) by all 16*MT token rows for its own K steps
//   and folds the scales exactly like the tiled kernel
//   (acc += partial * (Xs[m,kb] * Ws[nb,kb])).  After the loop the four partial accumulators are added
//   through LDS; with cross-CTA splits the sum goes to the workspace and the last CTA to arrive adds the
//   splits in order (deterministic) before the bf16 store.
//
// The activation scales of the CTA's K range are staged in LDS by one coalesced pass at the start: gathered per
// step (16 rows x 4 bytes per request) they cost as many cache-line accesses as the X block itself, 5-6 us of a
// 30-40 us launch at M = 32..64.
//
// Algorithmic bytes per K step and CTA: 16*TNW*128 weight bytes + 16*MT*128 activation bytes (L2 resident).
#pragma once
#include "gemm_tile.hpp"

namespace mi355 {

constexpr int kStreamWaves = 4;

template <int MT, int TNW>
struct StreamCfg {
    static_assert(TNW == 1 || TNW == 2 || TNW == 4 || TNW == 8, "a tile must sit inside one 128-row scale block");
    static constexpr int BN = 16 * TNW;
    // K steps in flight per wave.  Occupancy counts for more than depth: the deepest pipeline that still leaves a
    // wave within 256 registers, i.e. two CTAs per CU (measured: M=32 28.9 us at depth 3 -> 25.6 at depth 2,
    // M=64 36.6 us at depth 2 -> 33.9 at depth 1, M<=16 best at depth 3).
    static constexpr int depth(bool xs_in_lds) {
        if (xs_in_lds) return MT == 1 ? 3 : (MT == 2 ? 2 : 1);
        const int set = 8 * TNW + 9 * MT + 1;  // registers of one in-flight K step
        return set * 6 <= 150 ? 6 : (150 / set < 2 ? 2 : 150 / set);
    }
    static constexpr int kXOff = 16 * TNW * 128;                  // X block follows the W block
    static constexpr int kWaveLds = (16 * TNW + 16 * MT) * 128;
    static constexpr int kAccLds = TNW * MT * 1024;               // one wave's accumulators (fp32)
    static constexpr int kWaveBytes = kWaveLds > kAccLds ? kWaveLds : kAccLds;
    static constexpr int kLds = kStreamWaves * kWaveBytes + 16;   // + the split-K arrival word
    static constexpr int kTileElems = 16 * MT * BN;
    // activation scales of the CTA's K range, staged once: [step][16*MT rows + 1 pad] floats behind kLds
    static constexpr int kScaleStride = 16 * MT + 1;
    static constexpr int kMaxScaleSteps = 15 * 1024 / (kScaleStride * 4) < 64 ? 15 * 1024 / (kScaleStride * 4) : 64;
    static constexpr int scale_lds_bytes(int steps) { return steps * kScaleStride * 4; }
};

template <int MT, int TNW>
struct StreamRegs {
    v4i w[2 * TNW];  // 16*TNW rows x 128 B of W: instruction i holds rows 8i + lane/8, 16-byte chunk lane%8
    v4i x[2 * MT];   // 16*MT rows x 128 B of X, same arrangement
    float xs[MT];    // activation scales of rows 16*mt + lane%16 (unused when they are staged in LDS)
    float ws;        // weight scale of this (n block, K step)
};

// XSL: the activation scales of the CTA's K range are staged in LDS by one coalesced pass at the start (the host
// checks that the range fits); otherwise every wave gathers them per step, which costs as many cache-line
// accesses as the X block itself (16 rows x 4 bytes per request).
template <int MT, int TNW, bool SPLIT, bool XSL>
__global__ __launch_bounds__(256) void block_fp8_gemm_stream_kernel(const GemmArgs p) {
    using Cfg = StreamCfg<MT, TNW>;
    constexpr int D = Cfg::depth(XSL);
    constexpr int BN = Cfg::BN;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4;
    const int sub = lane >> 3, pch = lane & 7;

    uint32_t tile_n, split = 0;
    if constexpr (SPLIT) {
        tile_n = blockIdx.x / (uint32_t)p.splits;
        split = blockIdx.x - tile_n * (uint32_t)p.splits;
    } else {
        tile_n = blockIdx.x;
    }
    const int n0 = (int)tile_n * BN;
    const int KB = p.K / kBlockK;
    int kb_begin = 0, kb_end = KB;
    if constexpr (SPLIT) {
        const int per = KB / p.splits, rem = KB % p.splits;
        kb_begin = (int)split * per + min((int)split, rem);
        kb_end = kb_begin + per + ((int)split < rem ? 1 : 0);
    }
    // this wave's K steps: kb_begin + wave, + 4, ...
    const int first = kb_begin + wave;
    const int steps = first < kb_end ? (kb_end - first + kStreamWaves - 1) / kStreamWaves : 0;

    // ---- per-lane global offsets (rows past the matrix are clamped; their results are never stored)
    uint32_t woff[2 * TNW];
#pragma unroll
    for (int i = 0; i < 2 * TNW; ++i) woff[i] = (uint32_t)min(n0 + 8 * i + sub, p.N - 1) * (uint32_t)p.ldw + (uint32_t)pch * 16u;
    uint32_t xoff[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) xoff[i] = (uint32_t)min(8 * i + sub, p.M - 1) * (uint32_t)p.ldx + (uint32_t)pch * 16u;
    uint32_t soff[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) soff[t] = (uint32_t)min(16 * t + r16, p.M - 1) * (uint32_t)p.xs_m;
    const int NB = (p.N + kBlockN - 1) / kBlockN;
    const float *wsp = p.Ws + (int64_t)min(n0 / kBlockN, NB - 1) * p.ws_n;

    // ---- stage the activation scales: thread (row group tid/32, step tid%32) walks rows +8 and steps +32, so a
    // row-major scale row is read as whole cache lines; indices past the range repeat the last valid element
    float *xs_lds = (float *)(lds + Cfg::kLds);
    constexpr int kSvRows = 2 * MT, kSvSteps = (Cfg::kMaxScaleSteps + 31) / 32;
    float sv[XSL ? kSvRows * kSvSteps : 1];
    const int steps_cta = kb_end - kb_begin;
    if constexpr (XSL) {
#pragma unroll
        for (int a = 0; a < kSvRows; ++a)
#pragma unroll
            for (int b = 0; b < kSvSteps; ++b) {
                const int m = min(8 * a + (tid >> 5), p.M - 1);
                const int kb = min(kb_begin + min(32 * b + (tid & 31), max(steps_cta - 1, 0)), KB - 1);
                sv[a * kSvSteps + b] = p.Xs[(int64_t)m * p.xs_m + (int64_t)kb * p.xs_k];
            }
    }

    auto load = [&](StreamRegs<MT, TNW> &r, int kb) {
        const uint8_t *wk = p.W + (int64_t)kb * kBlockK;
        const uint8_t *xk = p.X + (int64_t)kb * kBlockK;
#pragma unroll
        for (int i = 0; i < 2 * TNW; ++i) r.w[i] = __builtin_nontemporal_load((const v4i *)(wk + woff[i]));
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) r.x[i] = *(const v4i *)(xk + xoff[i]);
        if constexpr (!XSL) {
#pragma unroll
            for (int t = 0; t < MT; ++t) r.xs[t] = p.Xs[soff[t] + (int64_t)kb * p.xs_k];
        }
        r.ws = wsp[(int64_t)kb * p.ws_k];
    };

    // ---- wave-private LDS: W block rows in MFMA order, then the X block; 128-byte rows, swizzled chunks.
    // Weight row 4*TNW*a + 4*tn + b of the tile sits in LDS row 16*tn + 4*a + b, so that the values a lane gets
    // from the TNW MFMA blocks are 4*TNW consecutive output columns (see gemm_tile.hpp).
    uint8_t *my = lds + wave * Cfg::kWaveBytes;
    uint32_t wst[2 * TNW];
#pragma unroll
    for (int i = 0; i < 2 * TNW; ++i) {
        const int nl = 8 * i + sub;
        const int a = nl / (4 * TNW), rem = nl % (4 * TNW);
        const int rho = 16 * (rem >> 2) + 4 * a + (rem & 3);
        wst[i] = (uint32_t)rho * 128u + (((uint32_t)pch ^ swz((uint32_t)rho)) * 16u);
    }
    uint32_t xst[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int row = 8 * i + sub;
        xst[i] = (uint32_t)Cfg::kXOff + (uint32_t)row * 128u + (((uint32_t)pch ^ swz((uint32_t)row)) * 16u);
    }
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t rd0 = (uint32_t)r16 * 128u + c0 * 16u, rd1 = (uint32_t)r16 * 128u + c1 * 16u;

    v4f acc[MT][TNW];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < TNW; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](const StreamRegs<MT, TNW> &r, int kb) {
        float xsv[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            if constexpr (XSL) xsv[t] = xs_lds[(kb - kb_begin) * Cfg::kScaleStride + 16 * t + r16];
            else xsv[t] = r.xs[t];
        }
#pragma unroll
        for (int i = 0; i < 2 * TNW; ++i) *(v4i *)(my + wst[i]) = r.w[i];
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) *(v4i *)(my + xst[i]) = r.x[i];
        // LDS operations of one wave execute in order: the reads below see the writes above
        v8i wf[TNW];
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
            const v4i lo = *(const v4i *)(my + rd0 + j * 2048);
            const v4i hi = *(const v4i *)(my + rd1 + j * 2048);
            wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const v4i lo = *(const v4i *)(my + Cfg::kXOff + rd0 + t * 2048);
            const v4i hi = *(const v4i *)(my + Cfg::kXOff + rd1 + t * 2048);
            const v8i xf = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const float sc = xsv[t] * r.ws;
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
                const v4f part = mfma_16x16x128_fp8(wf[j], xf, v4f{0.f, 0.f, 0.f, 0.f});
                acc[t][j] += part * sc;
            }
        }
    };

    // ---- the stream: DEPTH register sets rotate; the compiler places the vmcnt waits
    StreamRegs<MT, TNW> regs[D];
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < steps) load(regs[d], first + d * kStreamWaves);
    if constexpr (XSL) {
        // the scale loads were issued before the prologue loads, so only they are waited for here
#pragma unroll
        for (int a = 0; a < kSvRows; ++a)
#pragma unroll
            for (int b = 0; b < kSvSteps; ++b) {
                const int j = 32 * b + (tid & 31);
                if (j < steps_cta) xs_lds[j * Cfg::kScaleStride + 8 * a + (tid >> 5)] = sv[a * kSvSteps + b];
            }
        __syncthreads();
    }
    for (int j = 0; j < steps; j += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (j + d < steps) {
                consume(regs[d], first + (j + d) * kStreamWaves);
                if (j + d + D < steps) load(regs[d], first + (j + d + D) * kStreamWaves);
            }
        }
    }

    // ---- add the four waves' accumulators; wave w ends up owning the MFMA blocks f = mt*TNW + tn with f % 4 == w
    // (each wave first overwrites its own transposition area: LDS operations of a wave execute in order)
    constexpr int F = MT * TNW;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < TNW; ++j) *(v4f *)(my + ((t * TNW + j) * 64 + lane) * 16) = acc[t][j];
    __syncthreads();
    constexpr int FW = (F + kStreamWaves - 1) / kStreamWaves;  // blocks per wave
    v4f sum[FW];
#pragma unroll
    for (int q = 0; q < FW; ++q) {
        const int f = q * kStreamWaves + wave;
        v4f s = v4f{0.f, 0.f, 0.f, 0.f};
        if (f < F) {
#pragma unroll
            for (int w = 0; w < kStreamWaves; ++w) s += *(const v4f *)(lds + w * Cfg::kWaveBytes + (f * 64 + lane) * 16);
        }
        sum[q] = s;
    }

    if constexpr (SPLIT) {
        // same exchange protocol as the tiled split-K kernel (sc1 stores and loads, no cache-wide fence)
        const Sc1Buffer xch(p.partials + (int64_t)tile_n * p.splits * Cfg::kTileElems);
        const uint32_t lane_off = (uint32_t)lane * 16u;
#pragma unroll
        for (int q = 0; q < FW; ++q) {
            const int f = q * kStreamWaves + wave;
            if (f < F) xch.store(split * (uint32_t)(Cfg::kTileElems * 4) + (uint32_t)f * 1024u + lane_off, sum[q]);
        }
        wait_vmcnt<0>();
        __syncthreads();
        volatile uint32_t *arrived = (volatile uint32_t *)(lds + kStreamWaves * Cfg::kWaveBytes);
        if (tid == 0)
            *arrived = __hip_atomic_fetch_add(p.counters + tile_n, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*arrived != (uint32_t)p.splits - 1u) return;
        // the last workgroup adds the partials in split order, four splits per memory round trip
        constexpr int kBatch = 4;
        for (int sp0 = 0; sp0 < p.splits; sp0 += kBatch) {
            v4f t[FW][kBatch];
#pragma unroll
            for (int q = 0; q < FW; ++q) {
                const int f = q * kStreamWaves + wave;
#pragma unroll
                for (int d = 0; d < kBatch; ++d)
                    if (f < F && sp0 + d < p.splits)
                        t[q][d] = xch.load((uint32_t)(sp0 + d) * (uint32_t)(Cfg::kTileElems * 4) + (uint32_t)f * 1024u + lane_off);
            }
#pragma unroll
            for (int q = 0; q < FW; ++q) {
                const int f = q * kStreamWaves + wave;
#pragma unroll
                for (int d = 0; d < kBatch; ++d)
                    if (f < F && sp0 + d < p.splits) sum[q] = (sp0 + d == 0) ? t[q][d] : sum[q] + t[q][d];
            }
        }
        if (tid == 0) __hip_atomic_store(p.counters + tile_n, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- store: block f = (mt, tn): lane (r16, g4) holds row m = 16*mt + r16, columns n0 + 4*TNW*g4 + 4*tn + [0,4)
#pragma unroll
    for (int q = 0; q < FW; ++q) {
        const int f = q * kStreamWaves + wave;
        if (f >= F) continue;
        const int t = f / TNW, j = f % TNW;
        const int m = 16 * t + r16;
        const int ncol = n0 + 4 * TNW * g4 + 4 * j;
        if (m >= p.M) continue;
        uint16_t *cp = p.C + (int64_t)m * p.ldc + ncol;
        if (p.vec_store && ncol + 4 <= p.N) {
            *(v2i *)cp = v2i{(int)pack_out2(sum[q][0], sum[q][1], p.out_f16), (int)pack_out2(sum[q][2], sum[q][3], p.out_f16)};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (ncol + e < p.N) cp[e] = (uint16_t)out_bits(sum[q][e], p.out_f16);
        }
    }
}

}  // namespace mi355

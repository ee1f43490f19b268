// Block-scaled FP8 GEMM for decode-size M on gfx950, second weight-streaming kernel: the activation block of a K
// step is shared by the workgroup.
//
// The first streaming kernel (gemm_stream.hpp) lets every wave take its own K steps, so every wave loads its own
// activation block: at M = 32..64 that is as many requests, and as many registers per K step in flight, as the
// weights themselves, and the registers bound the depth of the stream.  Here the four waves of a workgroup work
// on the SAME K step and split the weight rows instead:
//
//   workgroup = 4 waves, owns 64*TNW weight rows and a contiguous range of K steps (cross-workgroup split-K only
//   when N alone gives too few workgroups); wave w owns rows [16*TNW*w, 16*TNW*(w+1)) of them.
//   Per K step a wave loads its 16*TNW x 128 B of W (plain coalesced 16-byte loads, 8 lanes per row segment) and
//   a quarter of the 16*MT x 128 B activation block, DEPTH steps ahead, into registers; at its turn it writes the
//   W bytes to a wave-private LDS area and its share of X to a double-buffered area that all four waves read
//   after one workgroup barrier, both in the swizzled [row][128 B] layout the MFMA operand reads want
//   (see gemm_tile.hpp).  A wave sees every K step of the workgroup's range, so there is no cross-wave reduction.
//   Scales are folded exactly as in the other kernels: acc += partial * (Xs[m,kb] * Ws[nb,kb]).
//
// The activation scales of the workgroup's K range are staged in LDS by one coalesced pass at the start.
//
// The price is one workgroup barrier per K step.  The host uses this kernel only where that is cheaper than the
// private activation blocks of the first kernel (see block_gemm.hip).
#pragma once
#include "gemm_tile.hpp"

namespace mi355 {

template <int MT, int TNW, int DEPTH>
struct ShareCfg {
    static_assert(TNW == 1 || TNW == 2, "a wave's rows must sit inside one 128-row scale block");
    static constexpr int kWaves = 4;
    static constexpr int BN = 16 * TNW * kWaves;
    static constexpr int XG = 2 * MT;                            // 8-row groups of the activation block
    static constexpr int NX = XG >= kWaves ? XG / kWaves : 1;    // groups a wave loads (waves repeat groups if fewer)
    static constexpr int kXStage = 16 * MT * 128;
    static constexpr int kWOff = 2 * kXStage;                    // wave-private W areas follow the two X stages
    static constexpr int kWPriv = 16 * TNW * 128;                // one of a wave's two W buffers
    static constexpr int kLds = kWOff + kWaves * 2 * kWPriv + 16;  // + the split-K arrival word
    static constexpr int kTileElems = 16 * MT * BN;
    static constexpr int kScaleStride = 16 * MT + 1;
    static constexpr int kMaxScaleSteps = 128;                   // K range per workgroup up to 16384
    static constexpr int scale_lds_bytes(int steps) { return steps * kScaleStride * 4; }
};

template <int MT, int TNW, int DEPTH, bool SPLIT>
__global__ __launch_bounds__(256) void block_fp8_gemm_xshare_kernel(const GemmArgs p) {
    using Cfg = ShareCfg<MT, TNW, DEPTH>;
    constexpr int D = DEPTH, NX = Cfg::NX, BN = Cfg::BN;
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
    const int nw = n0 + 16 * TNW * wave;  // first weight row of this wave
    const int KB = p.K / kBlockK;
    int kb_begin = 0, kb_end = KB;
    if constexpr (SPLIT) {
        const int per = KB / p.splits, rem = KB % p.splits;
        kb_begin = (int)split * per + min((int)split, rem);
        kb_end = kb_begin + per + ((int)split < rem ? 1 : 0);
    }
    const int steps = kb_end - kb_begin;

    // ---- per-lane global offsets (rows past the matrix are clamped; their results are never stored)
    uint32_t woff[2 * TNW];
#pragma unroll
    for (int i = 0; i < 2 * TNW; ++i) woff[i] = (uint32_t)min(nw + 8 * i + sub, p.N - 1) * (uint32_t)p.ldw + (uint32_t)pch * 16u;
    uint32_t xoff[NX], xst[NX];
#pragma unroll
    for (int i = 0; i < NX; ++i) {
        const int g = (wave + i * Cfg::kWaves) % Cfg::XG;  // waves beyond the block repeat a group (same bytes)
        const int row = 8 * g + sub;
        xoff[i] = (uint32_t)min(row, p.M - 1) * (uint32_t)p.ldx + (uint32_t)pch * 16u;
        xst[i] = (uint32_t)row * 128u + (((uint32_t)pch ^ swz((uint32_t)row)) * 16u);
    }
    const int NB = (p.N + kBlockN - 1) / kBlockN;
    const float *wsp = p.Ws + (int64_t)min(nw / kBlockN, NB - 1) * p.ws_n;

    // ---- stage the activation scales: thread (row group tid/32, step tid%32) walks rows +8 and steps +32, so a
    // row-major scale row is read as whole cache lines.  The loads are issued first, the LDS writes follow the
    // first weight loads.
    float *xs_lds = (float *)(lds + Cfg::kLds);
    constexpr int kSvRows = 2 * MT, kSvSteps = Cfg::kMaxScaleSteps / 32;
    float sv[kSvRows * kSvSteps];
#pragma unroll
    for (int a = 0; a < kSvRows; ++a)
#pragma unroll
        for (int b = 0; b < kSvSteps; ++b) {
            const int m = min(8 * a + (tid >> 5), p.M - 1);
            const int kb = kb_begin + min(32 * b + (tid & 31), max(steps - 1, 0));
            sv[a * kSvSteps + b] = p.Xs[(int64_t)m * p.xs_m + (int64_t)kb * p.xs_k];
        }

    struct Regs {
        v4i w[2 * TNW];
        v4i x[NX];
        float ws;
    };
    auto load = [&](Regs &r, int kb) {
        const uint8_t *wk = p.W + (int64_t)kb * kBlockK;
        const uint8_t *xk = p.X + (int64_t)kb * kBlockK;
#pragma unroll
        for (int i = 0; i < 2 * TNW; ++i) r.w[i] = __builtin_nontemporal_load((const v4i *)(wk + woff[i]));
#pragma unroll
        for (int i = 0; i < NX; ++i) r.x[i] = *(const v4i *)(xk + xoff[i]);
        r.ws = wsp[(int64_t)kb * p.ws_k];
    };

    // ---- LDS offsets: wave-private W block in MFMA row order (weight row 4*TNW*a + 4*tn + b of the wave's rows sits
    // in LDS row 16*tn + 4*a + b, so that a lane's TNW blocks give 4*TNW consecutive output columns)
    uint8_t *my = lds + Cfg::kWOff + wave * 2 * Cfg::kWPriv;
    uint32_t wst[2 * TNW];
#pragma unroll
    for (int i = 0; i < 2 * TNW; ++i) {
        const int nl = 8 * i + sub;
        const int a = nl / (4 * TNW), rem = nl % (4 * TNW);
        const int rho = 16 * (rem >> 2) + 4 * a + (rem & 3);
        wst[i] = (uint32_t)rho * 128u + (((uint32_t)pch ^ swz((uint32_t)rho)) * 16u);
    }
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t rd0 = (uint32_t)r16 * 128u + c0 * 16u, rd1 = (uint32_t)r16 * 128u + c1 * 16u;

    v4f acc[MT][TNW];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < TNW; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // A step is published (its bytes written to LDS) one step before it is computed, so the LDS writes of step
    // it + 1, the operand reads and MFMAs of step it and the global loads of later steps overlap; the one barrier
    // per step makes the published step visible and tells that the buffers of step it may be overwritten.
    auto publish = [&](const Regs &r, int it) {
        uint8_t *xs_stage = lds + (it & 1) * Cfg::kXStage;
        uint8_t *wb = my + (it & 1) * Cfg::kWPriv;
#pragma unroll
        for (int i = 0; i < 2 * TNW; ++i) *(v4i *)(wb + wst[i]) = r.w[i];
#pragma unroll
        for (int i = 0; i < NX; ++i) *(v4i *)(xs_stage + xst[i]) = r.x[i];
    };
    auto compute = [&](float ws, int it) {
        const uint8_t *xs_stage = lds + (it & 1) * Cfg::kXStage;
        const uint8_t *wb = my + (it & 1) * Cfg::kWPriv;
        v8i wf[TNW];
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
            const v4i lo = *(const v4i *)(wb + rd0 + j * 2048);
            const v4i hi = *(const v4i *)(wb + rd1 + j * 2048);
            wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const v4i lo = *(const v4i *)(xs_stage + rd0 + t * 2048);
            const v4i hi = *(const v4i *)(xs_stage + rd1 + t * 2048);
            const v8i xf = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const float sc = xs_lds[it * Cfg::kScaleStride + 16 * t + r16] * ws;
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
                const v4f part = mfma_16x16x128_fp8(wf[j], xf, v4f{0.f, 0.f, 0.f, 0.f});
                acc[t][j] += part * sc;
            }
        }
    };

    // ---- the stream: D register sets rotate; the compiler places the vmcnt waits
    Regs regs[D];
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < steps) load(regs[d], kb_begin + d);
#pragma unroll
    for (int a = 0; a < kSvRows; ++a)
#pragma unroll
        for (int b = 0; b < kSvSteps; ++b) {
            const int j = 32 * b + (tid & 31);
            if (j < steps) xs_lds[j * Cfg::kScaleStride + 8 * a + (tid >> 5)] = sv[a * kSvSteps + b];
        }
    float ws_cur = 0.f;
    if (steps > 0) {
        publish(regs[0], 0);
        ws_cur = regs[0].ws;
        if (D < steps) load(regs[0], kb_begin + D);
    }
    lds_barrier();  // the staged scales and step 0 are visible
    for (int j = 0; j < steps; j += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int it = j + d;
            if (it < steps) {
                const int dn = (d + 1) % D;  // register set of step it + 1 (a constant once the loop is unrolled)
                float ws_next = 0.f;
                if (it + 1 < steps) {
                    publish(regs[dn], it + 1);
                    ws_next = regs[dn].ws;
                    if (it + 1 + D < steps) load(regs[dn], kb_begin + it + 1 + D);
                }
                compute(ws_cur, it);
                ws_cur = ws_next;
                lds_barrier();
            }
        }
    }

    // ---- split-K: same exchange as the other kernels (sc1 stores and loads, no cache-wide fence)
    constexpr int F = MT * TNW;
    if constexpr (SPLIT) {
        const Sc1Buffer xch(p.partials + (int64_t)tile_n * p.splits * Cfg::kTileElems);
        const uint32_t lane_off = (uint32_t)(wave * F * 64 + lane) * 16u;
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int j = 0; j < TNW; ++j)
                xch.store(split * (uint32_t)(Cfg::kTileElems * 4) + (uint32_t)(t * TNW + j) * 1024u + lane_off, acc[t][j]);
        wait_vmcnt<0>();
        __syncthreads();
        volatile uint32_t *arrived = (volatile uint32_t *)(lds + Cfg::kLds - 16);
        if (tid == 0)
            *arrived = __hip_atomic_fetch_add(p.counters + tile_n, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*arrived != (uint32_t)p.splits - 1u) return;
        // the last workgroup adds the partials in split order, two splits per memory round trip
        for (int sp0 = 0; sp0 < p.splits; sp0 += 2) {
            v4f part[2][F];
#pragma unroll
            for (int d = 0; d < 2; ++d)
                if (sp0 + d < p.splits) {
#pragma unroll
                    for (int f = 0; f < F; ++f)
                        part[d][f] = xch.load((uint32_t)(sp0 + d) * (uint32_t)(Cfg::kTileElems * 4) + (uint32_t)f * 1024u + lane_off);
                }
#pragma unroll
            for (int d = 0; d < 2; ++d)
                if (sp0 + d < p.splits) {
#pragma unroll
                    for (int f = 0; f < F; ++f)
                        acc[f / TNW][f % TNW] = (sp0 + d == 0) ? part[d][f] : acc[f / TNW][f % TNW] + part[d][f];
                }
        }
        if (tid == 0) __hip_atomic_store(p.counters + tile_n, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- store: block (t, j): lane (r16, g4) holds row m = 16*t + r16, columns nw + 4*TNW*g4 + 4*j + [0,4)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + r16;
        if (m >= p.M) continue;
        uint16_t *cp = p.C + (int64_t)m * p.ldc + nw + 4 * TNW * g4;
        if (p.vec_store && nw + 16 * TNW <= p.N) {
            if constexpr (TNW == 2) {
                *(v4i *)cp = v4i{(int)pack_out2(acc[t][0][0], acc[t][0][1], p.out_f16), (int)pack_out2(acc[t][0][2], acc[t][0][3], p.out_f16),
                                 (int)pack_out2(acc[t][1][0], acc[t][1][1], p.out_f16), (int)pack_out2(acc[t][1][2], acc[t][1][3], p.out_f16)};
            } else {
                *(v2i *)cp = v2i{(int)pack_out2(acc[t][0][0], acc[t][0][1], p.out_f16), (int)pack_out2(acc[t][0][2], acc[t][0][3], p.out_f16)};
            }
        } else {
#pragma unroll
            for (int j = 0; j < TNW; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (nw + 4 * TNW * g4 + 4 * j + e < p.N) cp[4 * j + e] = (uint16_t)out_bits(acc[t][j][e], p.out_f16);
        }
    }
}

}  // namespace mi355

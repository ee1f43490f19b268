// Block-scaled FP8 GEMM for decode-size M on gfx950: the weight stream cut into one equal share per compute unit.
//
// The streaming kernel of gemm_stream.hpp hands out tiles of 16, 32 or 64 weight rows.  Where N / 64 is not a
// multiple of the number of compute units its last round is partly empty (N = 28672 on 256 units: 448 tiles, 192
// units stream two of them and 64 units one), and where N / 64 is below that number it has to share K between
// workgroups and exchange partial sums through memory (N = 4096: 13 us for a 59 MB stream of 10).  This kernel
// fits the tile to the device instead:
//
//   tile = TNW 16-row blocks of W with TNW = ceil(N / 16 / compute units), 1..5 - any count, not only the powers
//   of two that sit inside one 128-row scale block: a tile may straddle two scale blocks, and each lane picks, per
//   MFMA block, the scale of the 128-row block its own output columns lie in.
//   One workgroup of 8 waves per tile and the whole K range: the waves take the K steps round-robin (together
//   they read 1 KiB of every row at a time), each multiplies all TNW row blocks by all 16*MT token rows for its
//   own steps, and the eight partial accumulators are added through LDS at the end - no traffic between
//   workgroups, no second launch.
//   Per K step a wave issues 2*TNW weight loads and one or two activation loads (one when M <= 8: rows 8..15 of the
//   MFMA block are never stored) and nothing else: the activation scales and the weight scales of the tile's two
//   scale blocks are staged in LDS for the whole K range by one pass at the start.
//
// Everything else is the streaming kernel's: plain coalesced 16-byte loads (8 lanes per 128-byte row segment), a
// few K steps in flight in registers, the transposition into MFMA operand order through a wave-private LDS area
// with no barrier in the loop, the activation scales of the whole K range staged in LDS by one coalesced pass.
#pragma once
#include "gemm_stream.hpp"

namespace mi355 {

template <int MT, int TB>
struct CuStreamCfg {
    static_assert(TB >= 1 && TB <= 8, "a tile of up to 128 rows touches at most two 128-row scale blocks");
    static constexpr int kWaves = 8, kThreads = 512;
    static constexpr int KW = kWaves;                    // K phases
    static constexpr int BN = 16 * TB;
    static constexpr int kSet = 8 * TB + 8 * MT;         // registers of one K step in flight
    static constexpr int kDepth = kSet * 6 <= 132 ? 6 : (132 / kSet < 1 ? 1 : 132 / kSet);
    static constexpr int kXOff = 16 * TB * 128;
    static constexpr int kWaveLds = (16 * TB + 16 * MT) * 128;
    static constexpr int kAccLds = TB * MT * 1024;
    static constexpr int kWaveBytes = kWaveLds > kAccLds ? kWaveLds : kAccLds;
    static constexpr int kLds = kWaves * kWaveBytes;
    static constexpr int kScaleStride = 16 * MT + 1;  // floats per K step in the staged scales
    static constexpr int kMaxScaleUnits = 5;          // registers a thread stages scales through: K / 128 <= 160 / MT
    static constexpr int max_steps() { return 32 * (kMaxScaleUnits / MT); }
    // behind the waves' areas: activation scales [KB][16*MT + 1], then weight scales [2][KB]
    static constexpr int ws_off(int KB) { return kLds + KB * kScaleStride * 4; }
    static constexpr int lds_bytes(int KB) { return ws_off(KB) + 2 * KB * 4; }
};

template <int MT, int TB>
struct CuStreamRegs {
    v4i w[2 * TB];
    v4i x[2 * MT];
};

// XHI: M > 8, rows 8..15 of the first activation row block exist and are loaded.
template <int MT, int TB, bool XHI>
__global__ __launch_bounds__(512) void block_fp8_gemm_streamcu_kernel(const GemmArgs p) {
    using Cfg = CuStreamCfg<MT, TB>;
    constexpr int D = Cfg::kDepth, KW = Cfg::KW, nblk = TB;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int phase = wave;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int sub = lane >> 3, pch = lane & 7;
    const int n0 = (int)blockIdx.x * Cfg::BN;
    const int KB = p.K / kBlockK;
    // this wave's K steps: phase, phase + KW, ...
    const int steps = phase < KB ? (KB - phase + KW - 1) / KW : 0;
    constexpr bool x_hi = XHI;

    // ---- per-lane global offsets (rows past the matrix are clamped; their results are never stored)
    uint32_t woff[2 * TB];
#pragma unroll
    for (int i = 0; i < 2 * TB; ++i) woff[i] = (uint32_t)min(n0 + 8 * i + sub, p.N - 1) * (uint32_t)p.ldw + (uint32_t)pch * 16u;
    uint32_t xoff[2 * MT];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) xoff[i] = (uint32_t)min(8 * i + sub, p.M - 1) * (uint32_t)p.ldx + (uint32_t)pch * 16u;
    // the two 128-row scale blocks the sub-tile can touch, and which of them each of the lane's MFMA blocks reads:
    // block tn of lane group g4 holds output columns n0 + 4*nblk*g4 + 4*tn + [0, 4)
    const int NB = (p.N + kBlockN - 1) / kBlockN;
    const int nb0 = min(n0 / kBlockN, NB - 1);
    const float *wsp = p.Ws + (int64_t)min(nb0 + (tid >= 256 ? 1 : 0), NB - 1) * p.ws_n;
    uint32_t second = 0;  // bit tn: the block's columns lie in the second scale block
#pragma unroll
    for (int j = 0; j < TB; ++j)
        if ((n0 + 4 * nblk * g4 + 4 * j) / kBlockN > nb0) second |= 1u << j;

    // ---- the activation scales of the whole K range are staged in LDS: element (row r, step kb) at
    // xs_lds[kb * stride + r].  Thread (row group tid / 32, step tid % 32) walks rows + 16 and steps + 32, so a
    // row-major scale row is read as whole cache lines.  The loads are issued here, ahead of the first weight loads,
    // and stored to LDS behind them (memory operations return in order: the store waits for the scales only).
    float *xs_lds = (float *)(lds + Cfg::kLds);
    constexpr int kSv = Cfg::kMaxScaleUnits;
    const int sv_units = ((KB + 31) / 32) * MT;  // (step group, row group) units of 32 steps x 16 rows
    float sv[kSv];
#pragma unroll
    for (int u = 0; u < kSv; ++u) {
        const int uu = min(u, sv_units - 1);
        const int row = (uu % MT) * 16 + (tid >> 5), kb = (uu / MT) * 32 + (tid & 31);
        sv[u] = p.Xs[(int64_t)min(row, p.M - 1) * p.xs_m + (int64_t)min(kb, KB - 1) * p.xs_k];
    }
    // weight scales: thread t < 256 takes step t of the first scale block, thread 256 + t that of the second
    float *ws_lds = (float *)(lds + Cfg::ws_off(KB));
    const float wsv = wsp[(int64_t)min(tid & 255, KB - 1) * p.ws_k];

    auto load = [&](CuStreamRegs<MT, TB> &r, int kb) {
        const uint8_t *wk = p.W + (int64_t)kb * kBlockK;
        const uint8_t *xk = p.X + (int64_t)kb * kBlockK;
#pragma unroll
        for (int i = 0; i < 2 * TB; ++i) r.w[i] = __builtin_nontemporal_load((const v4i *)(wk + woff[i]));
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i)
            if (i != 1 || x_hi) r.x[i] = *(const v4i *)(xk + xoff[i]);
    };

    // ---- wave-private LDS: W block rows in MFMA order, then the X block; 128-byte rows, swizzled chunks.
    // Weight row 4*nblk*a + 4*tn + b of the sub-tile sits in LDS row 16*tn + 4*a + b, so that the values a lane gets
    // from the nblk MFMA blocks are 4*nblk consecutive output columns.
    uint8_t *my = lds + wave * Cfg::kWaveBytes;
    uint32_t wst[2 * TB];
#pragma unroll
    for (int i = 0; i < 2 * TB; ++i) {
        const int nl = 8 * i + sub;
        const int a = nl / (4 * TB), rem = nl % (4 * TB);
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

    v4f acc[MT][TB];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < TB; ++j) acc[t][j] = v4f{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](const CuStreamRegs<MT, TB> &r, int kb) {
        float xsv[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) xsv[t] = xs_lds[kb * Cfg::kScaleStride + 16 * t + r16];
#pragma unroll
        for (int i = 0; i < 2 * TB; ++i) *(v4i *)(my + wst[i]) = r.w[i];
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) *(v4i *)(my + xst[i]) = r.x[(i == 1 && !x_hi) ? 0 : i];
        const float ws0 = ws_lds[kb], ws1 = ws_lds[KB + kb];
        // LDS operations of one wave execute in order: the reads below see the writes above
        v8i xf[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const v4i lo = *(const v4i *)(my + Cfg::kXOff + rd0 + t * 2048);
            const v4i hi = *(const v4i *)(my + Cfg::kXOff + rd1 + t * 2048);
            xf[t] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < TB; ++j) {
            const v4i lo = *(const v4i *)(my + rd0 + j * 2048);
            const v4i hi = *(const v4i *)(my + rd1 + j * 2048);
            const v8i wf = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const float wsj = ((second >> j) & 1u) ? ws1 : ws0;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const v4f part = mfma_16x16x128_fp8(wf, xf[t], v4f{0.f, 0.f, 0.f, 0.f});
                acc[t][j] += part * (xsv[t] * wsj);
            }
        }
    };

    // ---- the stream: D register sets rotate; the compiler places the vmcnt waits
    CuStreamRegs<MT, TB> regs[D];
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < steps) load(regs[d], phase + d * KW);
#pragma unroll
    for (int u = 0; u < kSv; ++u) {
        const int row = (u % MT) * 16 + (tid >> 5), kb = (u / MT) * 32 + (tid & 31);
        if (u < sv_units && kb < KB) xs_lds[kb * Cfg::kScaleStride + row] = sv[u];
    }
    if ((tid & 255) < KB) ws_lds[(tid >> 8) * KB + (tid & 255)] = wsv;
    __syncthreads();  // the staged scales are visible
    for (int j = 0; j < steps; j += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            if (j + d < steps) {
                consume(regs[d], phase + (j + d) * KW);
                if (j + d + D < steps) load(regs[d], phase + (j + d + D) * KW);
            }
        }
    }

    // ---- add the eight waves' accumulators; wave w ends up owning the MFMA blocks f = mt*TB + tn with f % 8 == w
    // (each wave first overwrites its own transposition area: LDS operations of a wave execute in order)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < TB; ++j) *(v4f *)(my + ((t * TB + j) * 64 + lane) * 16) = acc[t][j];
    __syncthreads();
    constexpr int F = MT * TB;
    constexpr int FW = (F + KW - 1) / KW;  // blocks per wave
    const uint8_t *grp_lds = lds;
#pragma unroll
    for (int q = 0; q < FW; ++q) {
        const int f = q * KW + phase;
        const int t = f / TB, j = f % TB;
        if (f >= F) continue;
        v4f s = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < KW; ++w) s += *(const v4f *)(grp_lds + w * Cfg::kWaveBytes + (f * 64 + lane) * 16);
        // block (mt, tn): lane (r16, g4) holds row m = 16*mt + r16, columns n0 + 4*nblk*g4 + 4*tn + [0, 4)
        const int m = 16 * t + r16;
        const int ncol = n0 + 4 * nblk * g4 + 4 * j;
        if (m >= p.M) continue;
        uint16_t *cp = p.C + (int64_t)m * p.ldc + ncol;
        if (p.vec_store && ncol + 4 <= p.N) {
            *(v2i *)cp = v2i{(int)pack_out2(s[0], s[1], p.out_f16), (int)pack_out2(s[2], s[3], p.out_f16)};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (ncol + e < p.N) cp[e] = (uint16_t)out_bits(s[e], p.out_f16);
        }
    }
}

}  // namespace mi355

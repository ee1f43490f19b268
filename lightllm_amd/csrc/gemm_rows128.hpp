// Block-scaled FP8 GEMM for at most 384 activation rows on gfx950: a weight stream with the activation block in LDS.
//
// With so few rows of X every weight byte is used once (TN = 2) per launch, so the launch is a stream over W, and
// the square tiles spend it badly: a 128x128 tile keeps 16 KiB of W per K step in flight and one round of such tiles
// is bound by the latency of its steps, not by the memory.  This kernel is the 64-row tile of the grouped GEMM
// (gemm_small.hpp) with more rows and a dense epilogue:
//
//   16*MT activation rows (MT MFMA row blocks) x 128*TN weight rows, K step 128.
//     TN = 2: up to 128 rows (MT <= 8; 16 on two ring slots) against 256 weight rows; TN = 1: up to 384 rows
//     (MT <= 24) against 128.
//   WV waves (8; fewer for some unsplit launches, see below), wave w owns 16*TN weight rows and all activation rows:
//   MT x TN MFMA blocks per K step (the X operand blocks are read from LDS eight at a time).
//   NS ring slots of { X 16*MT x 128 B, W 128*TN x 128 B }.  A wave fetches its own W rows (2*TN requests of 1 KiB
//   per step) into its own part of a slot and is the only one to read them, so the W stream needs no barrier: the rows
//   of step kb + NS are requested as soon as the wave has read those of step kb.  The X block is shared: one barrier
//   per step makes step kb visible and frees the slot of step kb - 1 for step kb + NS - 1.
//   X scales come in [rows][8 steps] chunks by 4-byte requests (any scale layout); the W scales of the tile's
//   128-wide n blocks are copied to LDS once.
//   A compute unit pulls 35 to 40 GB/s from HBM through this tile, so the launch wants a workgroup on every unit:
//   when the tiles are too few for that the K range is shared between workgroups.  Their partial sums are
//   16*MT x 128*TN floats each, too many for the last workgroup of a tile to add alone (one compute unit reads
//   about 40 GB/s): they go to the workspace and a second, device-wide launch adds them in split order.
//
//   What a unit pulls is X and W together - the X block comes from L2, but through the same requests - so a launch
//   whose 256-row tiles leave units idle and whose K cannot be shared usefully runs narrower workgroups instead
//   (WV = 5 or 6: 160 or 192 weight rows), as many as there are units: every unit then loads less per K step.
//   The same holds for 129..208 rows on a wide N, whose 128-row tiles need a second round and whose 256x256 tiles
//   leave units idle: workgroups of 4..7 waves at TN = 1 (64..112 weight rows) or, on a wider N still, 5..8 waves at
//   TN = 2 with up to 13 row blocks (160..256 weight rows), whichever makes one round.  Every wave reads the whole X
//   block from LDS, so the time of such a launch grows with M and the square tiles take over from about 220 rows.
//
//   (Half-width tiles of four waves on two slots, two workgroups to a unit, were tried for shapes whose 256-row
//   tiles leave units idle and cannot share K usefully - N = 36864: 144 tiles on 256 units - and were slower: 85 us
//   against 69 at M = 128.)
//
// Arithmetic, operand layouts in LDS and the epilogue are those of the other tiled kernels (gemm_tile.hpp).
#pragma once
#include "gemm_tile.hpp"

namespace mi355 {

template <int MT, int NS, int TN_ = 2, int WV = 8>
struct Rows128Cfg {
    static_assert(WV >= 4 && WV <= 8 && MT >= 1 && MT <= (TN_ == 2 ? 16 : 24) && (NS == 2 || NS == 3) && (TN_ == 1 || TN_ == 2), "");
    static constexpr int TN = TN_, WNS = 16 * TN, kWaves = WV, kThreads = 64 * WV, BN = WNS * WV;
    static constexpr int NBLK = (BN + 2 * kBlockN - 2) / kBlockN;  // 128-wide n blocks a tile can touch
    static constexpr int NWW = 2 * TN;                         // W requests per wave and step (8 rows each)
    static constexpr int XG = 2 * MT;                          // 8-row request groups of the X block
    static constexpr int NXW = (XG + kWaves - 1) / kWaves;     // X requests per wave (groups repeat if XG % 8 != 0)
    static constexpr int XH = MT < 8 ? MT : 8;                 // X row blocks read from LDS at a time
    static constexpr int kXBytes = 16 * MT * 128, kWBytes = BN * 128;
    static constexpr int kStage = kXBytes + kWBytes;
    static constexpr int kWsOff = NS * kStage;                 // W scales [NBLK][steps]
    static constexpr int kChunkBytes = 16 * MT * 32;           // one [rows][8 steps] chunk of X scales
    static constexpr int kTileElems = 16 * MT * BN;
    static constexpr int chunk_off(int steps) { return (kWsOff + NBLK * steps * 4 + 127) & ~127; }
    static constexpr int lds_bytes(int steps) { return chunk_off(steps) + 2 * kChunkBytes; }
};

// One lane's 4*TN consecutive outputs of row `row`: columns nbase + 4*TN*g4 + [0, 4*TN).
template <int TN>
__device__ __forceinline__ void rows128_store(const GemmArgs &p, int row, int nbase, int g4, const float *o) {
    uint16_t *cp = p.C + (int64_t)row * p.ldc + nbase + lane_col<TN>(g4, 0);
    if (p.vec_store && nbase + 16 * TN <= p.N) {
        if constexpr (TN == 2) {
            *(v4i *)cp = v4i{(int)pack_out2(o[0], o[1], p.out_f16), (int)pack_out2(o[2], o[3], p.out_f16),
                             (int)pack_out2(o[4], o[5], p.out_f16), (int)pack_out2(o[6], o[7], p.out_f16)};
        } else {
            *(v2i *)cp = v2i{(int)pack_out2(o[0], o[1], p.out_f16), (int)pack_out2(o[2], o[3], p.out_f16)};
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4 * TN; ++e)
            if (nbase + lane_col<TN>(g4, 0) + e < p.N) cp[e] = (uint16_t)out_bits(o[e], p.out_f16);
    }
}

template <int MT, int NS, int TN, int WV, bool SPLIT>
__global__ __launch_bounds__(64 * WV) void block_fp8_gemm_rows128_kernel(const GemmArgs p) {
    using Cfg = Rows128Cfg<MT, NS, TN, WV>;
    constexpr int WNS = Cfg::WNS, NXW = Cfg::NXW, XG = Cfg::XG, NWW = Cfg::NWW, XH = Cfg::XH;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4, sub = lane >> 3;
    const uint32_t pch = (uint32_t)(lane & 7);

    uint32_t tile_n, tile_m = 0, split = 0;
    if constexpr (SPLIT) {
        tile_n = blockIdx.x / (uint32_t)p.splits;
        split = blockIdx.x - tile_n * (uint32_t)p.splits;
    } else if (p.tiles_m > 1) {
        // more rows than one block holds: tiles_m x tiles_n tiles, n fastest, one contiguous run per XCD (workgroup
        // ids go round-robin over the 8 XCDs), so the workgroups that share an L2 share their activation rows
        const uint32_t per_xcd = gridDim.x >> 3;  // the grid is a multiple of 8
        const uint32_t logical = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (logical >= (uint32_t)p.total_tiles) return;
        tile_m = logical / (uint32_t)p.tiles_n;
        tile_n = logical - tile_m * (uint32_t)p.tiles_n;
    } else {
        tile_n = blockIdx.x;
    }
    const int n0 = (int)tile_n * Cfg::BN;
    const int m0 = (int)tile_m * (16 * MT);
    const int KB = p.K / kBlockK;
    int kb_begin = 0, kb_end = KB;
    if constexpr (SPLIT) {
        const int per = KB / p.splits, rem = KB % p.splits;
        kb_begin = (int)split * per + min((int)split, rem);
        kb_end = kb_begin + per + ((int)split < rem ? 1 : 0);
    }
    const int steps = kb_end - kb_begin;
    const uint32_t lds0 = lds_addr(lds);

    // ---- request offsets (rows past the matrices are clamped; their results are never stored)
    uint32_t xoff[NXW], xdst[NXW], sc_row[NXW], sdst[NXW];
#pragma unroll
    for (int i = 0; i < NXW; ++i) {
        const int g = (wave + Cfg::kWaves * i) % XG;  // waves beyond the block repeat a group (same bytes)
        const int row = 8 * g + sub;
        const uint32_t src = (uint32_t)min(m0 + row, p.M - 1);
        xoff[i] = src * (uint32_t)p.ldx + (pch ^ swz((uint32_t)row)) * 16u;
        xdst[i] = (uint32_t)g * 1024u;
        sc_row[i] = src * (uint32_t)p.xs_m;
        sdst[i] = (uint32_t)g * 256u;
    }
    uint32_t woff[NWW];
#pragma unroll
    for (int i = 0; i < NWW; ++i) {
        const int w = 8 * i + sub;  // LDS row inside the wave's span of 16*TN rows
        const int tn = w >> 4, gg = (w >> 2) & 3, vv = w & 3;
        const int nl = wave * WNS + lane_col<TN>(gg, tn) + vv;
        const int nc = min(n0 + nl, p.N - 1) - n0;
        woff[i] = (uint32_t)nc * (uint32_t)p.ldw + (pch ^ swz((uint32_t)w)) * 16u;
    }
    const uint8_t *wg = p.W + (int64_t)n0 * p.ldw + (int64_t)kb_begin * kBlockK;
    const uint8_t *xg = p.X + (int64_t)kb_begin * kBlockK;
    const uint32_t wdst = (uint32_t)Cfg::kXBytes + (uint32_t)wave * (WNS * 128u);
    const uint32_t chunk_off = (uint32_t)Cfg::chunk_off(steps);

    auto issue_w = [&](int slot, int it) {
        const uint32_t sb = lds0 + (uint32_t)slot * Cfg::kStage + wdst;
        const uint8_t *wk = wg + (int64_t)it * kBlockK;
#pragma unroll
        for (int i = 0; i < NWW; ++i) dma_g2l_b128(sb + (uint32_t)i * 1024u, wk, woff[i]);
    };
    auto issue_x = [&](int slot, int it) {
        const uint32_t sb = lds0 + (uint32_t)slot * Cfg::kStage;
        const uint8_t *xk = xg + (int64_t)it * kBlockK;
#pragma unroll
        for (int i = 0; i < NXW; ++i) dma_g2l_b128(sb + xdst[i], xk, xoff[i]);
    };
    auto issue_scales = [&](int chunk) {
        const uint32_t st = (uint32_t)min(lane & 7, steps - 1 - 8 * chunk) * (uint32_t)p.xs_k;
        const float *base = p.Xs + (int64_t)(kb_begin + 8 * chunk) * p.xs_k;
#pragma unroll
        for (int i = 0; i < NXW; ++i)
            dma_g2l_b32(lds0 + chunk_off + (uint32_t)(chunk & 1) * Cfg::kChunkBytes + sdst[i], base, (sc_row[i] + st) * 4u);
    };

    // ---- per-lane LDS read offsets
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t xr0 = (uint32_t)r16 * 128u + c0 * 16u, xr1 = (uint32_t)r16 * 128u + c1 * 16u;
    const uint32_t wr0 = wdst + xr0, wr1 = wdst + xr1;
    const uint32_t sr8 = chunk_off + (uint32_t)r16 * 32u;

    // ---- first requests, in the order of the steady state: step j issues X(j+NS-1), its scale chunk, W(j+NS)
#pragma unroll
    for (int j = -NS; j < 0; ++j) {
        const int xi = j + NS - 1, wi = j + NS;
        if (xi >= 0 && xi < steps) {
            issue_x(xi % NS, xi);
            if (xi == 0) issue_scales(0);
        }
        if (wi < steps) issue_w(wi % NS, wi);
    }
    {
        const int NBk = (p.N + kBlockN - 1) / kBlockN;
        float *wl = (float *)(lds + Cfg::kWsOff);
        for (int i = tid; i < Cfg::NBLK * steps; i += Cfg::kThreads) {
            const int b = i / steps, it = i - b * steps;
            wl[i] = p.Ws[(int64_t)min(n0 / kBlockN + b, NBk - 1) * p.ws_n + (int64_t)(kb_begin + it) * p.ws_k];
        }
    }
    const float *wsl = (const float *)(lds + Cfg::kWsOff) + ((n0 + wave * WNS) / kBlockN - n0 / kBlockN) * steps;

    v4f acc[MT][TN];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    int slot = 0;
    for (int it = 0; it < steps; ++it) {
        // this wave's W rows and X groups of step `it` have landed; what was requested after them may be in flight:
        // W(it+1), and with three slots X(it+1) and W(it+2)
        if constexpr (NS == 2) {
            if (it + 1 < steps) wait_vmcnt<NWW>();
            else wait_vmcnt<0>();
        } else {
            if (it + 2 < steps) wait_vmcnt<2 * NWW + NXW>();
            else if (it + 1 < steps) wait_vmcnt<NWW + NXW>();
            else wait_vmcnt<0>();
        }
        lds_barrier();  // step `it` is visible to all; everyone has finished reading step it - 1
        {
            const int xi = it + NS - 1;
            if (xi < steps) {
                issue_x(slot == 0 ? NS - 1 : slot - 1, xi);
                if ((xi & 7) == 0) issue_scales(xi >> 3);
            }
        }
        const uint8_t *st = lds + slot * Cfg::kStage;
        const float ws_cur = wsl[it];
        const float *sp = (const float *)(lds + sr8 + ((it >> 3) & 1) * Cfg::kChunkBytes + (it & 7) * 4);
        v8i wf[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const v4i lo = *(const v4i *)(st + wr0 + j * 2048);
            const v4i hi = *(const v4i *)(st + wr1 + j * 2048);
            wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
        // the wave's own W rows of this slot have been read: request those of step it + NS into them.  (Only the
        // W reads are waited for here; the X reads below overlap the products.)
        __builtin_amdgcn_s_waitcnt(0xf | (0x3 << 14) | (0x7 << 4) | (0 << 8));  // lgkmcnt(0)
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if (it + NS < steps) issue_w(slot, it + NS);
#pragma unroll
        for (int h = 0; h < MT; h += XH) {  // at most 8 row blocks of X in registers at a time
            v8i xf[XH];
            float xs[XH];
#pragma unroll
            for (int i = 0; i < XH; ++i)
                if (h + i < MT) {
                    const v4i lo = *(const v4i *)(st + xr0 + (h + i) * 2048);
                    const v4i hi = *(const v4i *)(st + xr1 + (h + i) * 2048);
                    xf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    xs[i] = sp[(h + i) * 16 * 8] * ws_cur;
                }
#pragma unroll
            for (int i = 0; i < XH; ++i)
                if (h + i < MT) {
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const v4f part = mfma_16x16x128_fp8(wf[j], xf[i], v4f{0.f, 0.f, 0.f, 0.f});
                        acc[h + i][j] += part * xs[i];
                    }
                }
        }
        slot = slot + 1 == NS ? 0 : slot + 1;
    }

    // ---- shared K range: the partial sums go to the workspace in register order ([wave][block][lane] float4);
    // rows128_reduce_kernel adds them in split order and writes C
    if constexpr (SPLIT) {
        constexpr int F = MT * TN;
        float *part = p.partials + ((int64_t)tile_n * p.splits + split) * Cfg::kTileElems + (wave * F * 64 + lane) * 4;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) *(v4f *)(part + (i * TN + j) * 256) = acc[i][j];
        return;
    }

    // ---- epilogue: lane (r16, g4) holds row 16*i + r16 and the 4*TN columns n0 + 16*TN*wave + 4*TN*g4 + [0, 4*TN)
    const int nbase = n0 + wave * WNS;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int rl = m0 + 16 * i + r16;
        if (rl >= p.M) continue;
        float o[4 * TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) o[4 * j + vv] = acc[i][j][vv];
        rows128_store<TN>(p, rl, nbase, g4, o);
    }
}

// Second launch of a shared-K GEMM: thread (tile, wave, row block i, lane) adds its TN accumulator blocks over the
// splits in split order and stores 4*TN consecutive outputs of row 16*i + lane % 16.
template <int MT, int TN>
__global__ __launch_bounds__(256) void rows128_reduce_kernel(const GemmArgs p) {
    using Cfg = Rows128Cfg<MT, 2, TN, 8>;  // K is shared between 8-wave workgroups only
    constexpr int WNS = Cfg::WNS, F = MT * TN;
    const int lane = threadIdx.x & 63;
    const int item = blockIdx.x * 4 + (threadIdx.x >> 6);  // (tile, wave, i)
    const int tiles = (p.N + Cfg::BN - 1) / Cfg::BN;
    if (item >= tiles * Cfg::kWaves * MT) return;
    const int i = item % MT, wave = (item / MT) % Cfg::kWaves, tile_n = item / (MT * Cfg::kWaves);
    const int r16 = lane & 15, g4 = lane >> 4;
    const float *src = p.partials + (int64_t)tile_n * p.splits * Cfg::kTileElems + (wave * F * 64 + lane) * 4 + (i * TN) * 256;
    v4f a[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) a[j] = *(const v4f *)(src + j * 256);
    int sp = 1;
    for (; sp + 4 <= p.splits; sp += 4) {
        v4f b[4][TN];
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int j = 0; j < TN; ++j) b[d][j] = *(const v4f *)(src + (int64_t)(sp + d) * Cfg::kTileElems + j * 256);
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int j = 0; j < TN; ++j) a[j] += b[d][j];
    }
    for (; sp < p.splits; ++sp)
#pragma unroll
        for (int j = 0; j < TN; ++j) a[j] += *(const v4f *)(src + (int64_t)sp * Cfg::kTileElems + j * 256);
    const int rl = 16 * i + r16;
    if (rl >= p.M) return;
    float o[4 * TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) o[4 * j + vv] = a[j][vv];
    rows128_store<TN>(p, rl, tile_n * Cfg::BN + wave * WNS, g4, o);
}

}  // namespace mi355

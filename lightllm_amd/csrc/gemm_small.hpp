// Block-scaled FP8 grouped GEMM for gfx950: the tile for experts with few rows (at most 64 routed rows in the block).
//
// Such a tile is a stream over the expert's weights - 64 rows of activations against every weight row - and the
// 256x256 ping-pong tile spends it badly: three quarters of its activation area in LDS stay empty, half of its
// waves have no rows, and the 32 KiB of W per K step that its two ring slots keep in flight bound a compute unit
// to about 25 GB/s whatever the rest of the device does.  This tile turns the LDS around:
//
//   64 activation rows x 512 weight rows (two neighbouring 256-wide n tiles of the launch), K step 128.
//   8 waves, wave w owns weight rows [64w, 64w+64) and all 64 activation rows: 4 x 4 MFMA blocks per K step.
//   Two ring slots of { X 64 x 128 B, W 512 x 128 B } = 72 KiB each.  A wave fetches its own W rows (8 requests
//   of 1 KiB per step) into its own part of a slot and is the only one to read them, so the W stream needs no
//   barrier: the rows of step kb + 2 are requested as soon as the wave has read those of step kb, and up to two
//   steps - 128 KiB per compute unit - are in flight.  The X block (1 request per wave and step) is shared: one
//   barrier per step makes step kb visible and frees the slot of step kb - 1 for step kb + 1.
//   X scales come in [64 rows][8 steps] chunks by 4-byte requests (any scale layout), W scales of the tile's four
//   128-wide n blocks are copied to LDS once.
//
// A compute unit pulls about 30 to 40 GB/s from HBM through this tile when few of them stream, and the device
// about 5 TB/s when all do.  (A variant that kept operand fragments in registers one step ahead and refilled the
// W rows in 16-row pieces, so that LDS reads and products overlap, was no faster: the stream, not the step, is
// the bound.)
//
// Arithmetic, operand layouts in LDS and the epilogue are those of the other tiled kernels (gemm_tile.hpp).
#pragma once
#include "gemm_tile.hpp"

namespace mi355 {

struct SmallCfg {
    static constexpr int BM = 64, BN = 512, kWaves = 8, kThreads = 512;
    static constexpr int TM = 4, TN = 4, WNS = 64;
    static constexpr int kXBytes = BM * 128, kWBytes = BN * 128;
    static constexpr int kStage = kXBytes + kWBytes;
    static constexpr int kWsOff = 2 * kStage;                   // W scales [4 n blocks][KB]
    static constexpr int kChunkBytes = BM * 32;                 // one [64 rows][8 steps] chunk of X scales
    static constexpr int chunk_off(int KB) { return (kWsOff + 4 * KB * 4 + 127) & ~127; }
    static constexpr int lds_bytes(int KB) { return chunk_off(KB) + 2 * kChunkBytes; }
};

// One tile: expert `expert`, rows [m0, m0 + rows) of its list (rows <= 64), weight rows [n0, n0 + 512).
// Every wave of the workgroup calls this with the same arguments; on return all LDS reads are complete.
template <bool BIAS>
__device__ __forceinline__ void grouped_small_tile(const GemmArgs &p, uint8_t *lds, int expert, int m0, int rows, int n0) {
    using Cfg = SmallCfg;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, WNS = Cfg::WNS;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, g4 = lane >> 4, sub = lane >> 3;
    const uint32_t pch = (uint32_t)(lane & 7);
    const int KB = p.K / kBlockK;
    const uint32_t lds0 = lds_addr(lds);

    const int32_t *idx_list = p.e2t_index + (int64_t)expert * p.num_pairs + m0;
    const uint8_t *wg = p.W + (int64_t)expert * p.w_e + (int64_t)n0 * p.ldw;
    const float *ws_e = p.Ws + (int64_t)expert * p.ws_e;

    // ---- request offsets: X group `wave` (rows 8*wave + sub), the scale chunk rows of the same group, 8 W groups
    const int xr = 8 * wave + sub;
    const uint32_t src_row = (uint32_t)idx_list[min(xr, rows - 1)] / (uint32_t)p.topk;
    const uint32_t xoff = src_row * (uint32_t)p.ldx + (pch ^ swz((uint32_t)xr)) * 16u;
    const uint32_t xdst = (uint32_t)wave * 1024u;
    const uint32_t sc_row = src_row * (uint32_t)p.xs_m;
    uint32_t woff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int w = 8 * i + sub;  // LDS row inside the wave's 64-row span
        const int tn = w >> 4, gg = (w >> 2) & 3, vv = w & 3;
        const int nl = wave * WNS + lane_col<TN>(gg, tn) + vv;
        const int nc = min(n0 + nl, p.N - 1) - n0;
        woff[i] = (uint32_t)nc * (uint32_t)p.ldw + (pch ^ swz((uint32_t)w)) * 16u;
    }
    const uint32_t wdst = (uint32_t)Cfg::kXBytes + (uint32_t)wave * (WNS * 128u);
    const uint32_t chunk_off = (uint32_t)Cfg::chunk_off(KB);

    auto issue_w = [&](int slot, int kb) {
        const uint32_t sb = lds0 + (uint32_t)slot * Cfg::kStage + wdst;
        const uint8_t *wk = wg + (int64_t)kb * kBlockK;
#pragma unroll
        for (int i = 0; i < 8; ++i) dma_g2l_b128(sb + (uint32_t)i * 1024u, wk, woff[i]);
    };
    auto issue_x = [&](int slot, int kb) {
        dma_g2l_b128(lds0 + (uint32_t)slot * Cfg::kStage + xdst, p.X + (int64_t)kb * kBlockK, xoff);
    };
    auto issue_scales = [&](int chunk) {
        const uint32_t st = (uint32_t)min(lane & 7, KB - 1 - 8 * chunk) * (uint32_t)p.xs_k;
        dma_g2l_b32(lds0 + chunk_off + (uint32_t)(chunk & 1) * Cfg::kChunkBytes + (uint32_t)wave * 256u,
                    p.Xs + (int64_t)(8 * chunk) * p.xs_k, (sc_row + st) * 4u);
    };

    // ---- per-lane LDS read offsets
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t xr0 = (uint32_t)r16 * 128u + c0 * 16u, xr1 = (uint32_t)r16 * 128u + c1 * 16u;
    const uint32_t wr0 = wdst + xr0, wr1 = wdst + xr1;
    const uint32_t sr8 = chunk_off + (uint32_t)r16 * 32u;

    // ---- first requests, then the tile's W scales (plain loads: they are waited for before the loop starts)
    issue_w(0, 0);
    issue_x(0, 0);
    issue_scales(0);
    if (KB > 1) issue_w(1, 1);
    {
        const int NBk = (p.N + kBlockN - 1) / kBlockN;
        float *wl = (float *)(lds + Cfg::kWsOff);
        for (int i = tid; i < 4 * KB; i += Cfg::kThreads) {
            const int b = i / KB, kb = i - b * KB;
            wl[i] = ws_e[(int64_t)min(n0 / kBlockN + b, NBk - 1) * p.ws_n + (int64_t)kb * p.ws_k];
        }
    }
    const float *wsl = (const float *)(lds + Cfg::kWsOff) + ((wave * WNS) / kBlockN) * KB;

    v4f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    for (int kb = 0; kb < KB; ++kb) {
        const int slot = kb & 1;
        // this wave's W rows and X group of step kb have landed; only the W rows of step kb + 1 may be in flight
        if (kb + 1 < KB) wait_vmcnt<8>();
        else wait_vmcnt<0>();
        lds_barrier();  // step kb is visible to all; everyone has finished reading step kb - 1
        if (kb + 1 < KB) {
            issue_x(slot ^ 1, kb + 1);
            if (((kb + 1) & 7) == 0) issue_scales((kb + 1) >> 3);
        }
        const uint8_t *st = lds + slot * Cfg::kStage;
        const float ws_cur = wsl[kb];
        const float *sp = (const float *)(lds + sr8 + ((kb >> 3) & 1) * Cfg::kChunkBytes + (kb & 7) * 4);
        v8i wf[TN], xf[TM];
        float xs[TM];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const v4i lo = *(const v4i *)(st + wr0 + j * 2048);
            const v4i hi = *(const v4i *)(st + wr1 + j * 2048);
            wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const v4i lo = *(const v4i *)(st + xr0 + i * 2048);
            const v4i hi = *(const v4i *)(st + xr1 + i * 2048);
            xf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            xs[i] = sp[i * 16 * 8] * ws_cur;
        }
        // the wave's own W rows of this slot have been read: request those of step kb + 2 into them
        __builtin_amdgcn_s_waitcnt(0xf | (0x3 << 14) | (0x7 << 4) | (0 << 8));  // lgkmcnt(0)
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if (kb + 2 < KB) issue_w(slot, kb + 2);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4f part = mfma_16x16x128_fp8(wf[j], xf[i], v4f{0.f, 0.f, 0.f, 0.f});
                acc[i][j] += part * xs[i];
            }
    }
    lds_barrier();  // all reads of the last step are done: the caller may reuse the LDS

    // ---- epilogue: lane (r16, g4) holds row 16*i + r16 and, per block pair h, the 8 columns
    // n0 + 64*wave + lane_col(g4, 2h) + [0, 8)
    const int nbase = n0 + wave * WNS;
    const float *w_list = p.e2t_weight + (int64_t)expert * p.num_pairs + m0;
    float bias[BIAS ? 4 * TN : 1];
    if constexpr (BIAS) lane_bias<TN>(p, expert, nbase, g4, bias);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int rl = 16 * i + r16;
        if (rl >= rows) continue;
        const int64_t out_row = idx_list[rl];
        const float rw = p.mul_weight ? w_list[rl] : 1.0f;
        uint16_t *cp = p.C + out_row * p.ldc + nbase;
        float o[4 * TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) {
                if constexpr (BIAS) o[4 * j + vv] = (acc[i][j][vv] + bias[4 * j + vv]) * rw;
                else o[4 * j + vv] = acc[i][j][vv] * rw;
            }
        if (p.vec_store && nbase + WNS <= p.N) {
#pragma unroll
            for (int h = 0; h < TN / 2; ++h)
                *(v4i *)(cp + lane_col<TN>(g4, 2 * h)) =
                    v4i{(int)pack_out2(o[8 * h + 0], o[8 * h + 1], p.out_f16), (int)pack_out2(o[8 * h + 2], o[8 * h + 3], p.out_f16),
                        (int)pack_out2(o[8 * h + 4], o[8 * h + 5], p.out_f16), (int)pack_out2(o[8 * h + 6], o[8 * h + 7], p.out_f16)};
        } else {
#pragma unroll
            for (int e = 0; e < 4 * TN; ++e) {
                const int c = lane_col<TN>(g4, e >> 2) + (e & 3);
                if (nbase + c < p.N) cp[c] = (uint16_t)out_bits(o[e], p.out_f16);
            }
        }
    }
}

// Splits the rows of a 256-row schedule table by size for the launch with two kinds of workgroups (gemm_pp.hpp):
// lists[0] = number of blocks with more than 64 rows, lists[1] = number with 1..64 rows, then their table row
// indices in table order - the large ones from lists[2], the small ones from lists[2 + table_rows].
// One workgroup of 1024 lanes.
__global__ __launch_bounds__(1024) void grouped_split_kernel(const int32_t *__restrict__ table, int table_rows,
                                                             int32_t *__restrict__ lists) {
    __shared__ int wave_cnt[2][16];
    __shared__ int base[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < 2) base[tid] = 0;
    __syncthreads();
    for (int r0 = 0; r0 < table_rows; r0 += 1024) {
        const int r = r0 + tid;
        int kind = -1;
        if (r < table_rows) {
            const v4i row = *(const v4i *)(table + (int64_t)r * 4);
            if (row[0] >= 0 && row[3] > 0) kind = row[3] > SmallCfg::BM ? 0 : 1;
        }
        const uint64_t m0 = __ballot(kind == 0), m1 = __ballot(kind == 1);
        if (lane == 0) {
            wave_cnt[0][wave] = __popcll(m0);
            wave_cnt[1][wave] = __popcll(m1);
        }
        __syncthreads();
        if (kind >= 0) {
            int off = base[kind] + __popcll((kind == 0 ? m0 : m1) & ((1ull << lane) - 1ull));
            for (int w = 0; w < wave; ++w) off += wave_cnt[kind][w];
            lists[2 + (int64_t)kind * table_rows + off] = r;
        }
        __syncthreads();
        if (tid < 2) {
            int sum = 0;
            for (int w = 0; w < 16; ++w) sum += wave_cnt[tid][w];
            base[tid] += sum;
        }
        __syncthreads();
    }
    if (tid < 2) lists[tid] = base[tid];
}

}  // namespace mi355

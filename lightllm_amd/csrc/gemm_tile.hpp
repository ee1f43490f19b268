// Block-scaled FP8 GEMM for gfx950: the LDS-tiled MFMA kernel behind the dense, split-K and grouped launches.
//
//   C[m,n] = bf16( sum_kb ( sum_{k in kb} X[m,k] * W[n,k] ) * Xs[m,kb] * Ws[n/128,kb] )
//
// X is the activation matrix (A of the reference's w8a8_block_fp8_matmul), W the weight in its storage
// order [N,K]; both are K-contiguous fp8 bytes, so a 128-wide K step of one row is 128 contiguous bytes.
//
// Work decomposition
//   CTA tile BM x BN, K step 128 (one scale block).  WM x WN waves; a wave owns a (16*TM) x (16*TN)
//   sub-tile and runs v_mfma_f32_16x16x128_f8f6f4 once per 16x16 piece per K step: a single instruction
//   consumes the whole 128-wide scale block, so the partial product needs no second accumulator chain.
//   The MFMA is fed "transposed" (W rows as the A operand, X rows as the B operand): in the result each
//   lane then holds ONE token row m and 4 weight rows n, so the per-token scale is one register per lane
//   and the scale fold is 4 v_fmac per MFMA:   acc += partial * (Xs[m,kb] * Ws[nb,kb]).
//
// LDS (dynamic): NSTAGE stages of { X tile BM x 128 B, W tile BN x 128 B }, then NSTAGE x BM floats of X
//   scales (one column per stage), then the tile's weight scales for every K step (K/128 floats per 128-wide
//   n block), then - with chunked scales - two [BM rows][8 steps] buffers of X scales.
//   Rows are 128 B = 8 chunks of 16 B, chunk position XOR-swizzled with the row number (swz() in common.hpp)
//   so the ds_read_b128 operand fetches are conflict free.  W rows are stored in the order the MFMA wants
//   them: LDS row 16*tn + 4*g + v of a wave span holds weight row lane_col<TN>(g, tn) + v, which makes the
//   16-byte stores of the four lane groups of a token row adjacent (see lane_col).  Tiles are filled with
//   global_load_lds_dwordx4 (no register staging); each 8-lane group fetches one full 128-byte row segment.
//
// Pipelines
//   A ring of NSTAGE stages; the DMA for step kb+NSTAGE-1 is issued at the top of step kb, right after the one
//   barrier of the step (which also proves that the slot being refilled has been read by all).  The large
//   256x256 launches use the ping-pong kernel in gemm_pp.hpp instead.
//
// Launch modes
//   kDense     one CTA per output tile, whole K, ring.
//   kSplitK    grid = tiles x splits; each CTA accumulates a K range and stores its fp32 partial to the
//              workspace in register order; a second launch (tile_splitk_reduce_kernel) adds the partials in
//              split order (deterministic) and writes C.
//   kGrouped   rows are gathered through expert_to_token_index, the tile list is the moe_align2 table, the
//              weight and its scales are offset by the expert, rows are scattered back on store.
#pragma once
#include "common.hpp"

namespace mi355 {

enum { kDense = 0, kGrouped = 1, kSplitK = 2 };

struct GemmArgs {
    const uint8_t *X;    // [M,K] (dense) or [T,K] (grouped), row stride ldx bytes
    const uint8_t *W;    // [N,K] or [E,N,K], row stride ldw bytes
    const float *Xs;     // element (row,kb) at Xs[row*xs_m + kb*xs_k]
    const float *Ws;     // element (nb,kb) at Ws[nb*ws_n + kb*ws_k] (+ e*ws_e)
    uint16_t *C;         // bf16 [M,N] or [num_pairs,N], row stride ldc elements
    int32_t M, N, K;
    int32_t tiles_m, tiles_n, total_tiles, blocks_per_xcd;
    int64_t ldx, ldw, ldc;
    int64_t xs_m, xs_k, ws_n, ws_k;
    int32_t vec_store;   // 1: C rows are 16-byte aligned and N % 8 == 0
    int32_t out_f16;     // 0: C is bf16, 1: C is fp16
    // split-K launch only
    int32_t splits;
    uint32_t *counters;  // [total_tiles], zero before the launch, zero again after it
    float *partials;     // [total_tiles][splits][BM*BN]
    // grouped launch only
    const int32_t *table;        // [tiles_m,4] (expert, m_index, token_start, rows)
    const int32_t *e2t_index;    // [E,num_pairs]
    const float *e2t_weight;     // [E,num_pairs]
    const int32_t *e_num;        // [E]
    int64_t w_e, ws_e;           // expert strides of W (bytes) and Ws (elements)
    int32_t num_pairs, topk, mul_weight;
    const void *bias;            // [E,N] added to the fp32 accumulator before the routed weight, or nullptr
    int64_t bias_e;              // its expert stride (elements)
    int32_t bias_dtype;          // MI355_DTYPE_*
    // grouped launch with two kinds of workgroups (gemm_pp.hpp): row indices of the schedule table split by size
    const int32_t *lists;        // [0] = blocks with more than 64 rows, [1] = the others, then the two index lists
    int32_t small_first;         // workgroups per XCD that start on the small blocks
};

// Which of a wave's 16*TN output columns a lane holds.  The MFMA leaves lane group g (= lane / 16) with the four
// results v = 0..3 of A-operand rows 4*g + v of each of the TN 16-row blocks; which weight row sits in which
// A-operand row is free (it is fixed when the W tile is laid out in LDS).  The choice below makes the 8 values
// of a block pair (2h, 2h+1) eight consecutive columns, and the four lane groups of one token row adjacent
// 16-byte pieces: one store instruction then writes 64 contiguous bytes per row.  (With 16 consecutive columns
// per lane the pieces of one instruction were 32 bytes apart, and the L2 took four times as many write
// requests: 6 us per 256x256 tile.)
template <int TN>
__device__ __forceinline__ constexpr int lane_col(int g, int tn) {
    return TN == 1 ? 4 * g : 32 * (tn >> 1) + 8 * g + 4 * (tn & 1);
}

// The per-expert bias of the grouped launches: the values of the 4*TN output columns a lane holds (the same for
// every row of the tile), widened to fp32.  Columns past N repeat the last one (never stored).
__device__ __forceinline__ float bias_value(const void *bias, int dtype, int64_t i) {
    if (dtype == MI355_DTYPE_F32) return ((const float *)bias)[i];
    const uint16_t h = ((const uint16_t *)bias)[i];
    if (dtype == MI355_DTYPE_F16) return (float)__builtin_bit_cast(_Float16, h);
    return as_f32((uint32_t)h << 16);
}
template <int TN>
__device__ __forceinline__ void lane_bias(const GemmArgs &p, int expert, int nbase, int g4, float (&b)[4 * TN]) {
#pragma unroll
    for (int e = 0; e < 4 * TN; ++e) {
        const int c = min(nbase + lane_col<TN>(g4, e >> 2) + (e & 3), p.N - 1);
        b[e] = bias_value(p.bias, p.bias_dtype, (int64_t)expert * p.bias_e + c);
    }
}

template <int BM, int BN, int WM, int WN, int NSTAGE>
struct TileCfg {
    static constexpr int kThreads = WM * WN * 64;
    static constexpr int kWaves = WM * WN;
    static constexpr int WMS = BM / WM;  // rows of m per wave
    static constexpr int WNS = BN / WN;  // rows of n per wave
    static constexpr int TM = WMS / 16;
    static constexpr int TN = WNS / 16;
    static constexpr int XG = BM / 8;    // 8-row DMA groups in the X tile
    static constexpr int WG = BN / 8;
    static constexpr int XI = XG >= kWaves ? XG / kWaves : 1;  // DMA instructions per wave per stage
    static constexpr int WI = WG >= kWaves ? WG / kWaves : 1;
    static constexpr int SG = BM >= 64 ? BM / 64 : 1;          // 64-row groups of the scale vector
    static constexpr int kLoadsPerStage = XI + WI + 1;        // identical for every wave (one less with chunked scales)
    static constexpr int kStage = (BM + BN) * 128;
    static constexpr int kScaleOff = NSTAGE * kStage;
    static constexpr int kWsOff = kScaleOff + NSTAGE * BM * 4;  // weight scales of the whole K range
    static constexpr int NBC = BN >= 128 ? BN / 128 : 1;        // 128-wide scale blocks a tile spans
    static constexpr int lds_bytes(int KB) { return kWsOff + NBC * KB * 4 + 16; }  // + the split-K arrival word
    static_assert(XG % kWaves == 0 || kWaves % XG == 0, "X tile rows must split over the waves");
    static_assert(WG % kWaves == 0 || kWaves % WG == 0, "W tile rows must split over the waves");
    static_assert(WNS <= 128 && 128 % WNS == 0, "a wave's n span must sit inside one 128-wide scale block");
    static_assert(TN == 1 || TN == 2 || TN == 4, "TN");
    static_assert(SG <= kWaves, "scale DMA needs one wave per 64 rows");
    static_assert(NSTAGE >= 2 && (NSTAGE - 2) * kLoadsPerStage < 64, "vmcnt is a 6-bit counter");
};

// XS8: the X scales are row-major with 16-byte aligned rows and K/128 % 8 == 0, so they are fetched as
// [BM rows][8 steps] chunks (one request per 64 half-rows and chunk) instead of one column per step.
// BIAS (grouped launches only): p.bias is added to the accumulator before the routed weight.  A template parameter so
// that the launches without a bias keep their register allocation (sixteen more values live across the epilogue made
// the 256x256 kernel spill more and run 5 % slower with or without a bias).
template <int BM, int BN, int WM, int WN, int NSTAGE, int MODE, bool XS8, bool BIAS = false>
__global__ __launch_bounds__(WM *WN * 64) void block_fp8_gemm_tile_kernel(const GemmArgs p) {
    using Cfg = TileCfg<BM, BN, WM, WN, NSTAGE>;
    constexpr int kLoads = Cfg::XI + Cfg::WI + (XS8 ? 0 : 1);  // DMA requests per wave and stage
    constexpr int TM = Cfg::TM, TN = Cfg::TN, WMS = Cfg::WMS, WNS = Cfg::WNS;
    constexpr bool GROUPED = MODE == kGrouped;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    // ---- which tile (and which K range)
    uint32_t tile_m, tile_n, tile_id, split = 0;
    if constexpr (MODE == kSplitK) {
        // weight streaming: locality does not matter, keep the splits of a tile on neighbouring ids
        tile_id = blockIdx.x / (uint32_t)p.splits;
        split = blockIdx.x - tile_id * (uint32_t)p.splits;
        tile_m = tile_id % (uint32_t)p.tiles_m;
        tile_n = tile_id / (uint32_t)p.tiles_m;
    } else if constexpr (MODE == kGrouped) {
        // The schedule table is padded with empty rows at its end and tiles differ in cost, so tiles are dealt
        // out in launch order, n fastest: the n tiles of one m block land on different XCDs, and (tiles_n being
        // a multiple of 8 for the usual shapes) the same weight tile of consecutive m blocks on the same XCD.
        const uint32_t bid = blockIdx.x;
        if (bid >= (uint32_t)p.total_tiles) return;
        tile_m = bid / (uint32_t)p.tiles_n;
        tile_n = bid - tile_m * (uint32_t)p.tiles_n;
        tile_id = bid;
    } else {
        // XCD-aware order.  The hardware deals workgroup ids round-robin over the 8 XCDs; give every XCD a
        // contiguous run of logical tile ids so the tiles that share an L2 share X / W panels.
        const uint32_t bid = blockIdx.x;
        const uint32_t logical = (bid & 7u) * (uint32_t)p.blocks_per_xcd + (bid >> 3);
        if (logical >= (uint32_t)p.total_tiles) return;
        constexpr uint32_t GM = 8;
        const uint32_t width = GM * (uint32_t)p.tiles_n;
        const uint32_t grp = logical / width;
        const uint32_t first_m = grp * GM;
        const uint32_t gsz = min((uint32_t)p.tiles_m - first_m, GM);
        const uint32_t in_grp = logical - grp * width;
        tile_m = first_m + in_grp % gsz;
        tile_n = in_grp / gsz;
        tile_id = logical;
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WN, wave_n = wave % WN;
    const int r16 = lane & 15, g4 = lane >> 4;

    const int n0 = (int)tile_n * BN;
    int m0 = (int)tile_m * BM;  // dense: first row of the tile; grouped: first slot of the expert's list

    const int32_t *idx_list = nullptr;
    const float *w_list = nullptr;
    const uint8_t *Wbase = p.W;
    const float *Wsbase = p.Ws;
    int rows_valid;  // number of valid rows in this tile
    int expert = 0;
    if constexpr (GROUPED) {
        expert = p.table[tile_m * 4 + 0];
        if (expert < 0) return;
        const int mi = p.table[tile_m * 4 + 1];
        const int cnt = p.e_num[expert];
        m0 = mi * BM;
        idx_list = p.e2t_index + (int64_t)expert * p.num_pairs;
        w_list = p.e2t_weight + (int64_t)expert * p.num_pairs;
        Wbase += (int64_t)expert * p.w_e;
        Wsbase += (int64_t)expert * p.ws_e;
        rows_valid = min(cnt - m0, BM);
    } else {
        rows_valid = min(p.M - m0, BM);
    }

    // ---- per-lane DMA source offsets (bytes, relative to a wave-uniform base that advances with k)
    const int sub = lane >> 3;                  // row inside the 8-row DMA group
    const uint32_t pch = (uint32_t)(lane & 7);  // physical chunk this lane fills
    uint32_t xoff[Cfg::XI], woff[Cfg::WI];
    uint32_t xdst[Cfg::XI], wdst[Cfg::WI];
#pragma unroll
    for (int i = 0; i < Cfg::XI; ++i) {
        const int grpi = (wave + i * Cfg::kWaves) % Cfg::XG;  // waves beyond the tile repeat a group (same bytes)
        const int r = grpi * 8 + sub;
        const uint32_t c = pch ^ swz((uint32_t)r);
        const int rc = min(r, rows_valid - 1);
        uint32_t src_row;
        if constexpr (GROUPED) src_row = (uint32_t)idx_list[m0 + rc] / (uint32_t)p.topk;
        else src_row = (uint32_t)rc;
        xoff[i] = src_row * (uint32_t)p.ldx + c * 16u;
        xdst[i] = (uint32_t)grpi * 1024u;
    }
#pragma unroll
    for (int i = 0; i < Cfg::WI; ++i) {
        const int grpi = (wave + i * Cfg::kWaves) % Cfg::WG;
        const int rho = grpi * 8 + sub;  // LDS row
        const uint32_t c = pch ^ swz((uint32_t)rho);
        const int span = rho / WNS, w = rho % WNS;
        const int tn = w >> 4, gg = (w >> 2) & 3, v = w & 3;
        const int nl = span * WNS + lane_col<TN>(gg, tn) + v;
        const int nc = min(n0 + nl, p.N - 1) - n0;
        woff[i] = (uint32_t)nc * (uint32_t)p.ldw + c * 16u;
        wdst[i] = (uint32_t)BM * 128u + (uint32_t)grpi * 1024u;
    }
    // X-scale DMA: LDS slot j of a wave span holds row 16*(j % TM) + j / TM, so a lane's TM scales are contiguous
    uint32_t soff;
    const uint32_t sdst = (uint32_t)(wave % Cfg::SG) * 256u;
    const bool s_active = (wave % Cfg::SG) * 64 + lane < BM;
    {
        const int j = min((wave % Cfg::SG) * 64 + lane, BM - 1);
        const int span = j / WMS, w = j % WMS;
        const int row = span * WMS + 16 * (w % TM) + w / TM;
        const int rc = min(row, rows_valid - 1);
        uint32_t src_row;
        if constexpr (GROUPED) src_row = (uint32_t)idx_list[m0 + rc] / (uint32_t)p.topk;
        else src_row = (uint32_t)rc;
        soff = src_row * (uint32_t)(p.xs_m * 4);
    }

    const uint8_t *xg = p.X + (GROUPED ? (int64_t)0 : (int64_t)m0 * p.ldx);
    const uint8_t *wg = Wbase + (int64_t)n0 * p.ldw;
    const float *sg = p.Xs + (GROUPED ? (int64_t)0 : (int64_t)m0 * p.xs_m);
    const uint32_t lds0 = lds_addr(lds);

    // weight scales: the rows of the tile's 128-wide n blocks, all K steps, copied to LDS once
    const int KB = p.K / kBlockK;
    {
        const int NB = (p.N + kBlockN - 1) / kBlockN;
        float *wl = (float *)(lds + Cfg::kWsOff);
        for (int i = tid; i < Cfg::NBC * KB; i += Cfg::kThreads) {
            const int b = i / KB, kb = i - b * KB;
            const int nb = min(n0 / kBlockN + b, NB - 1);
            wl[i] = Wsbase[(int64_t)nb * p.ws_n + (int64_t)kb * p.ws_k];
        }
    }
    const float *wsl = (const float *)(lds + Cfg::kWsOff) + ((wave_n * WNS) / kBlockN) * KB;

    auto issue = [&](int stage, int kb) {
        const uint32_t sb = lds0 + (uint32_t)stage * Cfg::kStage;
        const uint8_t *xk = xg + (int64_t)kb * kBlockK;
        const uint8_t *wk = wg + (int64_t)kb * kBlockK;
#pragma unroll
        for (int i = 0; i < Cfg::XI; ++i) dma_g2l_b128(sb + xdst[i], xk, xoff[i]);
#pragma unroll
        for (int i = 0; i < Cfg::WI; ++i) dma_g2l_b128(sb + wdst[i], wk, woff[i]);
        // every wave issues this (waves beyond the tile repeat a group) so that all waves count the same
        // number of outstanding loads per stage; lanes past the tile's rows stay idle
        if constexpr (!XS8) {
            if (s_active)
                dma_g2l_b32(lds0 + Cfg::kScaleOff + (uint32_t)stage * (BM * 4) + sdst, sg + (int64_t)kb * p.xs_k, soff);
        }
    };

    // Chunked X scales (XS8).  Fetching one column of the row-major [M, K/128] scale matrix per step costs one
    // cache line per row and step - as many L2 requests as the X tile itself.  Instead a [BM rows][8 steps]
    // chunk is fetched at a time (32 useful bytes per line) into one of two LDS buffers behind the common
    // layout: lane l of wave w fetches steps 4*(l&1).. of row 32*w + l/2.  The scale of (row, step kb) then sits
    // at chunk[(kb/8) & 1][row][kb % 8].
    constexpr uint32_t kChunkBytes = BM * 32;
    const uint32_t chunk_off = (uint32_t)((Cfg::lds_bytes(KB) + 127) & ~127);
    uint32_t sc_off = 0;
    const bool sc_active = XS8 && wave * 64 + lane < 2 * BM;
    if (sc_active) {
        const int rc = min(wave * 32 + (lane >> 1), rows_valid - 1);
        uint32_t src_row;
        if constexpr (GROUPED) src_row = (uint32_t)idx_list[m0 + rc] / (uint32_t)p.topk;
        else src_row = (uint32_t)rc;
        sc_off = (src_row * (uint32_t)p.xs_m + 4u * (uint32_t)(lane & 1)) * 4u;
    }
    auto issue_scales = [&](int chunk) {
        if (wave * 64 < 2 * BM) {
            if (sc_active)
                dma_g2l_b128(lds0 + chunk_off + (uint32_t)(chunk & 1) * kChunkBytes + (uint32_t)wave * 1024u, sg + 8 * chunk, sc_off);
        }
    };
    const int nchunk = KB / 8;
    const uint32_t sr8 = chunk_off + (uint32_t)(wave_m * WMS + r16) * 32u;

    // ---- per-lane LDS read offsets
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t xrow = (uint32_t)(wave_m * WMS + r16) * 128u;
    const uint32_t wrow = (uint32_t)BM * 128u + (uint32_t)(wave_n * WNS + r16) * 128u;
    const uint32_t xr0 = xrow + c0 * 16u, xr1 = xrow + c1 * 16u;
    const uint32_t wr0 = wrow + c0 * 16u, wr1 = wrow + c1 * 16u;
    const uint32_t sr = Cfg::kScaleOff + (uint32_t)(wave_m * WMS + r16 * TM) * 4u;

    v4f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    // ---- K range of this CTA
    int kb_begin = 0, kb_end = KB;
    if constexpr (MODE == kSplitK) {
        const int per = KB / p.splits, rem = KB % p.splits;
        kb_begin = (int)split * per + min((int)split, rem);
        kb_end = kb_begin + per + ((int)split < rem ? 1 : 0);
    }
    const int nk = kb_end - kb_begin;

    // prologue: the scale chunk of the first step and the one after it, then NSTAGE-1 stages
    if constexpr (XS8) {
        issue_scales(kb_begin >> 3);
        if ((kb_begin >> 3) + 1 < nchunk) issue_scales((kb_begin >> 3) + 1);
    }
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s)
        if (s < nk) issue(s, kb_begin + s);

    int cur = 0;            // ring slot of step it
    int fill = NSTAGE - 1;  // ring slot the next DMA goes to
    for (int it = 0; it < nk; ++it) {
        // stage `it` must have landed; the NSTAGE-2 stages issued after it may still be in flight
        // (a scale-chunk request in between only makes the wait stricter: requests retire in order)
        if (it + NSTAGE - 2 < nk) wait_vmcnt<(NSTAGE - 2) * kLoads>();
        else wait_vmcnt<0>();
        __syncthreads();
        const int kb = kb_begin + it;
        if constexpr (XS8) {
            // the buffer of chunk kb/8 + 1 was last read in step kb - 1, before the barrier above
            if ((kb & 7) == 0 && it > 0 && (kb >> 3) + 1 < nchunk) issue_scales((kb >> 3) + 1);
        }
        if (it + NSTAGE - 1 < nk) issue(fill, kb_begin + it + NSTAGE - 1);
        const float ws_cur = wsl[kb_begin + it];

        const uint8_t *st = lds + cur * Cfg::kStage;
        float xs[TM];
        if constexpr (XS8) {
            const float *sp = (const float *)(lds + sr8 + ((kb >> 3) & 1) * kChunkBytes + (kb & 7) * 4);
#pragma unroll
            for (int i = 0; i < TM; ++i) xs[i] = sp[i * 16 * 8] * ws_cur;
        } else {
            const float *sp = (const float *)(lds + sr + cur * (BM * 4));
#pragma unroll
            for (int i = 0; i < TM; ++i) xs[i] = sp[i] * ws_cur;
        }
        v8i wf[TN];
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
            const v8i xf = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const v4f part = mfma_16x16x128_fp8(wf[j], xf, v4f{0.f, 0.f, 0.f, 0.f});
                acc[i][j] += part * xs[i];
            }
        }
        cur = cur + 1 == NSTAGE ? 0 : cur + 1;
        fill = fill + 1 == NSTAGE ? 0 : fill + 1;
    }


    // ---- split-K: the partial sums go to the workspace in register order ([split][block][thread] float4);
    // tile_splitk_reduce_kernel, a second launch, adds them in split order and writes C.  (The last workgroup of a
    // tile adding them alone - one compute unit reads about 40 GB/s - cost more than the launch: 128 KiB partials of
    // seven splits took 22 us.)
    if constexpr (MODE == kSplitK) {
        constexpr int kTileElems = BM * BN;
        float *mine = p.partials + ((int64_t)tile_id * p.splits + split) * kTileElems + tid * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) *(v4f *)(mine + (i * TN + j) * Cfg::kThreads * 4) = acc[i][j];
        return;
    }

    // ---- epilogue: lane (r16, g4) holds, for each tm, row m = wave_m*WMS + 16*tm + r16 and, for each MFMA block
    // tn, the 4 columns n0 + wave_n*WNS + lane_col(g4, tn) + [0, 4).
    const int nbase = n0 + wave_n * WNS;
    float bias[BIAS ? 4 * TN : 1];
    if constexpr (BIAS) lane_bias<TN>(p, expert, nbase, g4, bias);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int rl = wave_m * WMS + 16 * i + r16;
        if (rl >= rows_valid) continue;
        int64_t out_row;
        float rw = 1.0f;
        if constexpr (GROUPED) {
            out_row = idx_list[m0 + rl];
            if (p.mul_weight) rw = w_list[m0 + rl];
        } else {
            out_row = m0 + rl;
        }
        uint16_t *cp = p.C + out_row * p.ldc + nbase;
        float o[4 * TN];
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if constexpr (BIAS) o[4 * j + v] = (acc[i][j][v] + bias[4 * j + v]) * rw;
                else o[4 * j + v] = GROUPED ? acc[i][j][v] * rw : acc[i][j][v];
            }
        if (p.vec_store && nbase + WNS <= p.N) {
            if constexpr (TN == 1) {
                *(v2i *)(cp + lane_col<TN>(g4, 0)) = v2i{(int)pack_out2(o[0], o[1], p.out_f16), (int)pack_out2(o[2], o[3], p.out_f16)};
            } else {
#pragma unroll
                for (int h = 0; h < TN / 2; ++h)
                    *(v4i *)(cp + lane_col<TN>(g4, 2 * h)) =
                        v4i{(int)pack_out2(o[8 * h + 0], o[8 * h + 1], p.out_f16), (int)pack_out2(o[8 * h + 2], o[8 * h + 3], p.out_f16),
                            (int)pack_out2(o[8 * h + 4], o[8 * h + 5], p.out_f16), (int)pack_out2(o[8 * h + 6], o[8 * h + 7], p.out_f16)};
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4 * TN; ++e) {
                const int c = lane_col<TN>(g4, e >> 2) + (e & 3);
                if (nbase + c < p.N) cp[c] = (uint16_t)out_bits(o[e], p.out_f16);
            }
        }
    }
}

// Second launch of a split-K GEMM on the ring tiles: workgroup (tile, block b) - the thread layout of the GEMM's
// workgroup - adds block b of the tile's partial sums over the splits in split order and stores the 4 outputs of
// each thread.
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM *WN * 64) void tile_splitk_reduce_kernel(const GemmArgs p) {
    using Cfg = TileCfg<BM, BN, WM, WN, 2>;
    constexpr int TN = Cfg::TN, NB = Cfg::TM * Cfg::TN, kTileElems = BM * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WN, wave_n = wave % WN;
    const int r16 = lane & 15, g4 = lane >> 4;
    const uint32_t tile_id = blockIdx.x / NB, b = blockIdx.x - tile_id * NB;
    const uint32_t tile_m = tile_id % (uint32_t)p.tiles_m, tile_n = tile_id / (uint32_t)p.tiles_m;
    const int i = (int)b / TN, j = (int)b % TN;
    const float *src = p.partials + (int64_t)tile_id * p.splits * kTileElems + (int64_t)b * Cfg::kThreads * 4 + tid * 4;
    v4f a = *(const v4f *)src;
    int sp = 1;
    for (; sp + 4 <= p.splits; sp += 4) {
        v4f t[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) t[d] = *(const v4f *)(src + (int64_t)(sp + d) * kTileElems);
#pragma unroll
        for (int d = 0; d < 4; ++d) a += t[d];
    }
    for (; sp < p.splits; ++sp) a += *(const v4f *)(src + (int64_t)sp * kTileElems);
    const int row = (int)tile_m * BM + wave_m * Cfg::WMS + 16 * i + r16;
    const int col = (int)tile_n * BN + wave_n * Cfg::WNS + lane_col<TN>(g4, j);
    if (row >= p.M) return;
    uint16_t *cp = p.C + (int64_t)row * p.ldc + col;
    if (p.vec_store && col + 4 <= p.N) {
        *(v2i *)cp = v2i{(int)pack_out2(a[0], a[1], p.out_f16), (int)pack_out2(a[2], a[3], p.out_f16)};
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < p.N) cp[e] = (uint16_t)out_bits(a[e], p.out_f16);
    }
}

}  // namespace mi355

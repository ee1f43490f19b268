// Block-scaled FP8 GEMM for gfx950: the 256x256 ping-pong kernel behind the large dense and grouped launches.
//
// Same arithmetic, LDS tile layout and epilogue as the ring kernel in gemm_tile.hpp (see there for the operand
// layouts); what differs is the schedule:
//
//   * Two wave groups (waves 0-3 and 4-7: one wave of each per SIMD) run the phases of a K step
//         A0  read the W fragments and the first half of the X fragments (+ their scales)
//         B0  16 MFMA + scale folds of the first half
//         A1  read the second half of the X fragments (+ scales)
//         B1  16 MFMA + scale folds of the second half
//     one phase apart, a barrier after each, so the MFMA bursts of one group overlap the LDS / DMA traffic of the
//     other.  Group 1 passes one extra barrier before its first phase and group 0 one after its last.
//   * Two ring slots of { X 256 x 128 B, W 256 x 128 B }.  A region of a slot is requested again as soon as both
//     groups have read it: the W rows and first-half X rows of step it+2 at A1(it), the second-half X rows of
//     step it+1 at A0(it).  Every request is waited for one and a half steps later, by every wave, before the
//     barrier that lets the first group read it.  The loop body has no branches in the dense launch (steps past
//     the end re-fetch the last step, identical bytes) so the phases stay where they are written.
//   * X scales come in [256 rows][8 steps] chunks (one 16-byte request per half row and chunk, two buffers):
//     one column per step would cost as many cache-line requests as the X tile itself.
//   * The kernel is persistent: a workgroup keeps taking tiles, and between two tiles it issues the first
//     requests of the next tile before it stores the finished one, so the request latency, the stores and the
//     index gathers of the grouped launch overlap.  A fresh workgroup per tile costs about 9 us of such
//     serialized latencies per tile (10 % of a 56-step tile, 25 % of a 16-step one).
//     Tiles are numbered per XCD (workgroup ids go round-robin over the 8 XCDs): sequence number v on XCD x is
//     logical tile x*blocks_per_xcd + v of the dense order (runs of 8 m tiles x all n, so the tiles that share
//     an L2 share panels) or tile 8*v + x of the grouped launch order (n fastest: tiles differ in cost and the
//     schedule table is padded at its end, so they are dealt out).  The first two sequence numbers of a
//     workgroup are static (its index in the XCD, + workgroups per XCD), later ones come from one atomic counter
//     per XCD in the caller's workspace, fetched two tiles ahead; the schedule-table row of a tile is loaded one
//     tile ahead.  Counter words: [0..7] per-XCD, [8] workgroups that have finished; the last one to finish
//     zeroes them again.  Without a workspace (counters == nullptr) every workgroup runs one tile.
//     Dense launches with an even number of K steps let the ring run on across the boundary between two whole
//     tiles: the last two steps of a tile request W and X of the first two steps of the next one, in the slots
//     where its loop expects them, instead of repeating their own last step (M = 4096,
//     N = 32768, K = 512, eight tiles of four steps per workgroup: 129 us against 148; N = 36864, K = 7168: 1 %).
//   * Stream-K launch (SK, dense only): when the tiles do not fill whole rounds of the device, the K steps of all
//     tiles - tile-major, in the dense tile order - are cut into one contiguous run per workgroup, so every compute
//     unit does the same number of K steps.  A workgroup whose run covers only part of a tile's K range writes its
//     fp32 accumulators to its own slot of the workspace (two slots per workgroup: a run starts and ends inside at
//     most one tile each); a second launch (streamk_reduce_kernel) adds the parts of every shared tile in K order
//     and stores it.  (Adding them in the last workgroup to arrive at a tile was 3 to 8 % slower: one compute unit
//     reads the parts of a tile at a fraction of the rate the whole device does.)  Where the shape allows it the
//     host asks for a panel split instead (p.splits > 0): every tile's K range in the same p.splits runs and one
//     (m tile, run) pair per XCD across all n tiles, so that the workgroups of an XCD share their X rows in its L2
//     - cut as one sequence, neighbouring runs share nothing and the launch is bound by what they all pull.
//   * ROLES (grouped launch with a workspace): schedule blocks with at most 64 rows are weight streams, and this
//     tile streams badly (32 KiB of W in flight per step, three quarters of the X area and half of the waves
//     idle).  They go to the 64 x 512 tile of gemm_small.hpp instead, in the same launch: a split kernel has
//     listed the two kinds of blocks, each kind has its own tile queue, some workgroups start on the small blocks
//     and the others on the large ones, and a workgroup whose queue is empty moves to the other.  So at any time
//     part of the device streams weights while the rest computes, where one kind after the other would leave
//     the matrix cores idle during the streams and the memory idle during the computation.
//   * SC4: the X scales are row-major with 16-byte aligned rows and K/128 a multiple of 8, and a chunk is fetched
//     with one 16-byte request per half row.  Otherwise (any strides, any K/128) it is fetched with 4-byte
//     requests, one per (row, step), four instructions per wave and chunk; steps past the end of K repeat the
//     last one.
#pragma once
#include "gemm_small.hpp"
#include "gemm_tile.hpp"

namespace mi355 {

struct PPCfg {
    static constexpr int BM = 256, BN = 256, kWaves = 8, kThreads = 512;
    static constexpr int WMS = 128, WNS = 64;   // a wave's sub-tile: 2 x 4 waves
    static constexpr int TM = 8, TN = 4, HM = 4;
    static constexpr int XI = 4, WI = 4;         // 8-row DMA groups per wave: 32 of X and 32 of W over 8 waves
    static constexpr int kStage = (BM + BN) * 128;
    static constexpr int kDummyOff = 2 * kStage;     // 256-byte target of place-holder requests
    static constexpr int kWsOff = kDummyOff + 256;   // two buffers of the tile's weight scales [2 n blocks][KB]
    static constexpr int kChunkBytes = BM * 32;      // one [256 rows][8 steps] chunk of X scales
    static constexpr int ws_bytes(int KB) { return 2 * KB * 4; }
    static constexpr int chunk_off(int KB) { return (kWsOff + 2 * ws_bytes(KB) + 127) & ~127; }
    static constexpr int sched_off(int KB) { return chunk_off(KB) + 2 * kChunkBytes; }
    static constexpr int lds_bytes(int KB) { return sched_off(KB) + 16; }
    static constexpr int kCounterWords = 10;          // [0..7] per-XCD tile queues, [8] finished workgroups, [9] small-block queue
    // ROLES: the LDS word that hands sequence numbers to the waves sits behind both tiles' layouts
    static constexpr int roles_sched_off(int KB) {
        return sched_off(KB) > SmallCfg::lds_bytes(KB) ? sched_off(KB) : SmallCfg::lds_bytes(KB);
    }
    static constexpr int kPartialBytes = BM * BN * 4;  // one fp32 partial tile
};

template <bool GROUPED, bool SK, bool SC4, bool ROLES = false, bool BIAS = false>
__global__ __launch_bounds__(512) void block_fp8_gemm_pp_kernel(const GemmArgs p) {
    static_assert(!(GROUPED && SK), "stream-K is a dense launch");
    static_assert(!BIAS || GROUPED, "the per-expert bias belongs to the grouped launch");
    static_assert(!ROLES || GROUPED, "the small-block tile belongs to the grouped launch");
    using Cfg = PPCfg;
    constexpr int BM = Cfg::BM, TM = Cfg::TM, TN = Cfg::TN, HM = Cfg::HM, WMS = Cfg::WMS, WNS = Cfg::WNS;
    constexpr bool SKIP = GROUPED;  // ragged tiles skip empty halves; dense tiles keep the branch-free body
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int KB = p.K / kBlockK, nchunk = (KB + 7) >> 3;
    const uint32_t xcd = blockIdx.x & 7u, in_xcd = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
    const bool persistent = !SK && p.counters != nullptr;
    const bool xt_ok = !GROUPED && persistent && KB >= 2 && (KB & 1) == 0;
    volatile uint32_t *sched = (volatile uint32_t *)(lds + (ROLES ? Cfg::roles_sched_off(KB) : Cfg::sched_off(KB)));
    // ROLES: blocks with more than 64 rows (the tile loop below) and the others (small_blocks), listed by the
    // split kernel.  The first workgroups of every XCD start on the small blocks, the others on the large ones;
    // each moves on to the other queue when its own is empty.
    const int n_big = ROLES ? __builtin_amdgcn_readfirstlane(p.lists[0]) : 0;
    const int n_small = ROLES ? __builtin_amdgcn_readfirstlane(p.lists[1]) : 0;
    const int32_t *big_rows = ROLES ? p.lists + 2 : nullptr;
    const int32_t *small_rows = ROLES ? p.lists + 2 + p.tiles_m : nullptr;
    const bool small_first = ROLES && in_xcd < (uint32_t)p.small_first;
    auto small_blocks = [&]() {
        // one queue for the whole device: (block, pair of n tiles), n fastest
        const uint32_t pairs_n = (uint32_t)((p.N + SmallCfg::BN - 1) / SmallCfg::BN);
        const uint32_t total_small = (uint32_t)n_small * pairs_n;
        while (true) {
            if (threadIdx.x == 0)
                sched[0] = __hip_atomic_fetch_add(p.counters + 9, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            const uint32_t item = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[0]);
            __syncthreads();
            if (item >= total_small) break;
            const uint32_t blk = item / pairs_n;
            const v4i row = *(const v4i *)(p.table + (int64_t)small_rows[blk] * 4);
            grouped_small_tile<BIAS>(p, lds, __builtin_amdgcn_readfirstlane(row[0]), __builtin_amdgcn_readfirstlane(row[1]) * BM,
                               __builtin_amdgcn_readfirstlane(row[3]), (int)(item - blk * pairs_n) * SmallCfg::BN);
        }
    };
    if constexpr (ROLES) {
        if (small_first) small_blocks();
    }

    int tid = threadIdx.x;
    // ROLES: nothing that depends on the lane is to stay in registers while the other kind of tile runs
    if constexpr (ROLES) asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 2, wave_n = wave & 3;
    const int grp = wave >> 2;
    const int r16 = lane & 15, g4 = lane >> 4;
    const int sub = lane >> 3;
    const uint32_t pch = (uint32_t)(lane & 7);
    const uint32_t lds0 = lds_addr(lds);
    // stream-K: this workgroup's run of (tile, K step) units; workgroups are ranked XCD-major so that one XCD works
    // on neighbouring tiles
    uint32_t rank = xcd * per_xcd + in_xcd;
    const uint64_t units = (uint64_t)p.total_tiles * (uint64_t)KB;
    uint32_t u_end = SK ? (uint32_t)(((uint64_t)rank + 1u) * units / gridDim.x) : 0u;
    uint32_t u_first = SK ? (uint32_t)((uint64_t)rank * units / gridDim.x) : 0u;
    if constexpr (SK) {
        if (p.splits > 0) {
            // panel split: every tile's K range is cut into p.splits runs; XCD x takes the (m tile, run) pairs
            // 8*q + x and, of each, all n tiles - so the workgroups of an XCD read the same X rows and K steps at the
            // same time and its L2 serves all but the first of them.  rank becomes tile * splits + run.
            const uint32_t q = in_xcd / (uint32_t)p.tiles_n, tn = in_xcd - q * (uint32_t)p.tiles_n;
            const uint32_t pr = q * 8u + xcd, tm = pr / (uint32_t)p.splits, run = pr - tm * (uint32_t)p.splits;
            constexpr uint32_t GM = 8;
            const uint32_t g = tm / GM, first_m = g * GM, gsz = min((uint32_t)p.tiles_m - first_m, GM);
            const uint32_t id = g * GM * (uint32_t)p.tiles_n + tn * gsz + (tm - first_m);
            const uint32_t per = (uint32_t)KB / (uint32_t)p.splits, rem = (uint32_t)KB % (uint32_t)p.splits;
            u_first = id * (uint32_t)KB + run * per + min(run, rem);
            u_end = u_first + per + (run < rem ? 1u : 0u);
            rank = id * (uint32_t)p.splits + run;
        }
    }
    constexpr uint32_t kNone = 0xffffffffu;

    // ---- tile-independent LDS offsets
    uint32_t xdst[Cfg::XI], wdst[Cfg::WI];
#pragma unroll
    for (int i = 0; i < Cfg::XI; ++i) xdst[i] = (uint32_t)(wave + i * Cfg::kWaves) * 1024u;
#pragma unroll
    for (int i = 0; i < Cfg::WI; ++i) wdst[i] = (uint32_t)BM * 128u + (uint32_t)(wave + i * Cfg::kWaves) * 1024u;
    const uint32_t fr = swz((uint32_t)r16);
    const uint32_t c0 = ((uint32_t)(2 * g4)) ^ fr, c1 = c0 ^ 1u;
    const uint32_t xrow = (uint32_t)(wave_m * WMS + r16) * 128u;
    const uint32_t wrow = (uint32_t)BM * 128u + (uint32_t)(wave_n * WNS + r16) * 128u;
    const uint32_t xr0 = xrow + c0 * 16u, xr1 = xrow + c1 * 16u;
    const uint32_t wr0 = wrow + c0 * 16u, wr1 = wrow + c1 * 16u;
    const uint32_t chunk_off = (uint32_t)Cfg::chunk_off(KB);
    const uint32_t sr8 = chunk_off + (uint32_t)(wave_m * WMS + r16) * 32u;

    // ---- the tile a sequence number names
    struct Tile {
        int m0;      // dense: first row; grouped: first slot of the expert's list
        int n0;
        int rows;    // valid rows
        int expert;
        int k0, k1;  // K steps [k0, k1) of the tile that this workgroup computes (the whole range unless SK)
        uint32_t id; // stream-K: logical tile number
        bool valid;
    };
    auto dense_coords = [&](uint32_t logical, uint32_t &tile_m, uint32_t &tile_n) {
        constexpr uint32_t GM = 8;
        const uint32_t width = GM * (uint32_t)p.tiles_n;
        const uint32_t g = logical / width;
        const uint32_t first_m = g * GM;
        const uint32_t gsz = min((uint32_t)p.tiles_m - first_m, GM);
        const uint32_t in_grp = logical - g * width;
        tile_m = first_m + in_grp % gsz;
        tile_n = in_grp / gsz;
    };
    auto tile_coords = [&](uint32_t v, uint32_t &tile_m, uint32_t &tile_n) -> bool {
        if (v == kNone) return false;
        if constexpr (GROUPED) {
            const uint64_t bid = (uint64_t)v * 8u + xcd;
            if (bid >= (ROLES ? (uint64_t)n_big * (uint64_t)p.tiles_n : (uint64_t)p.total_tiles)) return false;
            tile_m = (uint32_t)bid / (uint32_t)p.tiles_n;
            tile_n = (uint32_t)bid - tile_m * (uint32_t)p.tiles_n;
            if constexpr (ROLES) tile_m = (uint32_t)big_rows[tile_m];
        } else {
            if (v >= (uint32_t)p.blocks_per_xcd) return false;
            const uint32_t logical = xcd * (uint32_t)p.blocks_per_xcd + v;
            if (logical >= (uint32_t)p.total_tiles) return false;
            dense_coords(logical, tile_m, tile_n);
        }
        return true;
    };
    // grouped: the schedule-table row (expert, m_index, token_start, rows) of sequence number v; expert < 0 = none
    auto load_row = [&](uint32_t v) -> v4i {
        uint32_t tm = 0, tn = 0;
        if (!GROUPED || !tile_coords(v, tm, tn)) return v4i{-1, 0, 0, 0};
        return *(const v4i *)(p.table + (int64_t)tm * 4);
    };
    // non-SK: v is a sequence number; SK: v is the first unit of the segment
    auto make_tile = [&](uint32_t v, v4i row) -> Tile {
        Tile t = {0, 0, 0, 0, 0, KB, 0u, false};
        uint32_t tm = 0, tn = 0;
        if constexpr (SK) {
            if (v >= u_end) return t;
            t.id = v / (uint32_t)KB;
            t.k0 = (int)(v - t.id * (uint32_t)KB);
            t.k1 = min(KB, t.k0 + (int)(u_end - v));
            t.k0 = __builtin_amdgcn_readfirstlane(t.k0);
            t.k1 = __builtin_amdgcn_readfirstlane(t.k1);
            dense_coords(t.id, tm, tn);
        } else {
            if (!tile_coords(v, tm, tn)) return t;
        }
        t.n0 = (int)tn * Cfg::BN;
        if constexpr (GROUPED) {
            t.expert = __builtin_amdgcn_readfirstlane(row[0]);
            if (t.expert < 0) return t;
            t.m0 = __builtin_amdgcn_readfirstlane(row[1]) * BM;
            t.rows = __builtin_amdgcn_readfirstlane(row[3]);
        } else {
            t.m0 = (int)tm * BM;
            t.rows = min(p.M - t.m0, BM);
        }
        t.m0 = __builtin_amdgcn_readfirstlane(t.m0);
        t.n0 = __builtin_amdgcn_readfirstlane(t.n0);
        t.rows = __builtin_amdgcn_readfirstlane(t.rows);
        t.valid = true;
        return t;
    };

    // ---- per-tile request state
    uint32_t xoff[Cfg::XI], woff[Cfg::WI], sc_off = 0;
    uint32_t sc_row[SC4 ? 1 : Cfg::XI];  // !SC4: scale-row offsets (elements) of the rows this lane fetches
    bool x_real[Cfg::XI];
    bool do_half0 = true, do_half1 = true;
    const uint8_t *xg = p.X, *wg = p.W;
    const float *sg = p.Xs;
    int wsbuf = 0;  // weight-scale buffer of the tile in the K loop

    // row gathers of a tile (grouped): slot -> token row.  Issued early, used by finish_setup.
    auto gather = [&](const Tile &t, uint32_t (&raw)[Cfg::XI + 1]) {
        if constexpr (GROUPED) {
            const int32_t *idx_list = p.e2t_index + (int64_t)t.expert * p.num_pairs + t.m0;
#pragma unroll
            for (int i = 0; i < Cfg::XI; ++i) raw[i] = (uint32_t)idx_list[min((wave + i * Cfg::kWaves) * 8 + sub, t.rows - 1)];
            raw[Cfg::XI] = (uint32_t)idx_list[min(wave * 32 + (lane >> 1), t.rows - 1)];
        } else {
#pragma unroll
            for (int i = 0; i < Cfg::XI; ++i) raw[i] = (uint32_t)min((wave + i * Cfg::kWaves) * 8 + sub, t.rows - 1);
            raw[Cfg::XI] = (uint32_t)min(wave * 32 + (lane >> 1), t.rows - 1);
        }
    };
    const uint8_t *w_tile = p.W;   // W rows of the tile (expert and n0 applied)
    const float *ws_tile = p.Ws;   // weight scales of the tile's expert
    auto setup_w = [&](const Tile &t) {
        w_tile = p.W + (GROUPED ? (int64_t)t.expert * p.w_e : (int64_t)0) + (int64_t)t.n0 * p.ldw;
        ws_tile = p.Ws + (GROUPED ? (int64_t)t.expert * p.ws_e : (int64_t)0);
        wg = w_tile;
#pragma unroll
        for (int i = 0; i < Cfg::WI; ++i) {
            const int rho = (wave + i * Cfg::kWaves) * 8 + sub;  // LDS row
            const uint32_t c = pch ^ swz((uint32_t)rho);
            const int span = rho / WNS, w = rho % WNS;
            const int tn = w >> 4, gg = (w >> 2) & 3, vv = w & 3;
            const int nl = span * WNS + lane_col<TN>(gg, tn) + vv;
            const int nc = min(t.n0 + nl, p.N - 1) - t.n0;
            woff[i] = (uint32_t)nc * (uint32_t)p.ldw + c * 16u;
        }
    };
    auto setup_x = [&](const Tile &t, const uint32_t (&raw)[Cfg::XI + 1]) {
        xg = p.X + (GROUPED ? (int64_t)0 : (int64_t)t.m0 * p.ldx);
        sg = p.Xs + (GROUPED ? (int64_t)0 : (int64_t)t.m0 * p.xs_m);
#pragma unroll
        for (int i = 0; i < Cfg::XI; ++i) {
            const int r = (wave + i * Cfg::kWaves) * 8 + sub;
            const uint32_t c = pch ^ swz((uint32_t)r);
            const uint32_t src_row = GROUPED ? raw[i] / (uint32_t)p.topk : raw[i];
            xoff[i] = src_row * (uint32_t)p.ldx + c * 16u;
            x_real[i] = !SKIP || (wave + i * Cfg::kWaves) * 8 < t.rows;
            if constexpr (!SC4) sc_row[i] = src_row * (uint32_t)p.xs_m;
        }
        const uint32_t srow = GROUPED ? raw[Cfg::XI] / (uint32_t)p.topk : raw[Cfg::XI];
        sc_off = (srow * (uint32_t)p.xs_m + 4u * (uint32_t)(lane & 1)) * 4u;
        do_half0 = !SKIP || wave_m * WMS < t.rows;
        do_half1 = !SKIP || wave_m * WMS + WMS / 2 < t.rows;
    };
    // the tile's weight scales (2 n blocks x all K steps) go to LDS buffer `buf` in two parts: the load is issued
    // with the tile's first requests, the LDS write waits until the stores of the previous tile are out (a
    // write right behind the load would wait for every request issued before it)
    auto ws_elem = [&](const Tile &t, int i) -> float {
        const int NB = (p.N + kBlockN - 1) / kBlockN;
        const int b = i / KB, kb = i - b * KB;
        const int nb = min(t.n0 / kBlockN + b, NB - 1);
        return ws_tile[(int64_t)nb * p.ws_n + (int64_t)kb * p.ws_k];
    };
    auto ws_load = [&](const Tile &t) -> float { return tid < 2 * KB ? ws_elem(t, tid) : 0.f; };
    auto ws_store = [&](const Tile &t, int buf, float first) {
        float *wl = (float *)(lds + Cfg::kWsOff + buf * Cfg::ws_bytes(KB));
        if (tid < 2 * KB) wl[tid] = first;
        for (int i = tid + Cfg::kThreads; i < 2 * KB; i += Cfg::kThreads) wl[i] = ws_elem(t, i);  // K > 32768 only
    };

    // ---- DMA requests.  An 8-row X group past the last valid row of a ragged tile is not fetched; a one-line
    // request takes its place so that every wave counts the same number of requests.
    auto issue_x = [&](int i, uint32_t sb, const uint8_t *xk) {
        if (x_real[i]) dma_g2l_b128(sb + xdst[i], xk, xoff[i]);
        else dma_g2l_b32(lds0 + Cfg::kDummyOff, p.X, 0u);
    };
    auto issue_w_at = [&](int stage, const uint8_t *wk) {
        const uint32_t sb = lds0 + (uint32_t)stage * Cfg::kStage;
#pragma unroll
        for (int i = 0; i < Cfg::WI; ++i) dma_g2l_b128(sb + wdst[i], wk, woff[i]);
    };
    auto issue_xlo_at = [&](int stage, const uint8_t *xk) {
        const uint32_t sb = lds0 + (uint32_t)stage * Cfg::kStage;
#pragma unroll
        for (int i = 0; i < Cfg::XI; i += 2) issue_x(i, sb, xk);
    };
    auto issue_xhi_at = [&](int stage, const uint8_t *xk) {
        const uint32_t sb = lds0 + (uint32_t)stage * Cfg::kStage;
#pragma unroll
        for (int i = 1; i < Cfg::XI; i += 2) issue_x(i, sb, xk);
    };
    auto issue_w = [&](int stage, int kb) { issue_w_at(stage, wg + (int64_t)kb * kBlockK); };
    auto issue_xlo = [&](int stage, int kb) { issue_xlo_at(stage, xg + (int64_t)kb * kBlockK); };
    auto issue_xhi = [&](int stage, int kb) { issue_xhi_at(stage, xg + (int64_t)kb * kBlockK); };
    // Scale (row, kb) sits at chunk[(kb/8) & 1][row][kb % 8].  SC4: lane l of wave w fetches steps 4*(l&1).. of row
    // 32*w + l/2.  Otherwise lane l fetches step l%8 of row l/8 of the same four 8-row groups it fetches X rows
    // for; steps past the end of K repeat the last step (never read).
    auto issue_scales = [&](int chunk) {
        const uint32_t dst = lds0 + chunk_off + (uint32_t)(chunk & 1) * Cfg::kChunkBytes;
        if constexpr (SC4) {
            dma_g2l_b128(dst + (uint32_t)wave * 1024u, sg + 8 * chunk, sc_off);
        } else {
            const uint32_t st = (uint32_t)min(lane & 7, KB - 1 - 8 * chunk) * (uint32_t)p.xs_k;
            const float *sk = sg + (int64_t)(8 * chunk) * p.xs_k;
#pragma unroll
            for (int i = 0; i < Cfg::XI; ++i)
                dma_g2l_b32(dst + (uint32_t)(wave + i * Cfg::kWaves) * 256u, sk, (sc_row[i] + st) * 4u);
        }
    };
    constexpr int kXhi = Cfg::XI / 2;             // requests per wave in A0
    constexpr int kWXlo = Cfg::XI / 2 + Cfg::WI;  // requests per wave in A1

    auto phase_end = [&]() {
        __atomic_signal_fence(__ATOMIC_SEQ_CST);  // compiler only: no LDS access may move across the barrier
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
    };
    auto wait_lds = [&]() { __builtin_amdgcn_s_waitcnt(0xf | (0x3 << 14) | (0x7 << 4) | (0 << 8)); };

    // ---- start: the first tile and the row of the second
    uint32_t v_next = persistent ? per_xcd + in_xcd : kNone;  // sequence number of the tile after the current one
    uint32_t v_after = kNone;                                 // and of the one after that (fetched)
    uint32_t fetched = 0;
    uint32_t v_first = SK ? u_first : in_xcd;
    if constexpr (ROLES) {
        // a workgroup may enter this loop at any time: all its sequence numbers come from the XCD's queue
        if (tid == 0)
            for (int i = 0; i < 3; ++i)
                sched[i] = __hip_atomic_fetch_add(p.counters + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        v_first = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[0]);
        v_next = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[1]);
        v_after = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[2]);
        __syncthreads();
        wsbuf = 0;
    }
    Tile cur = make_tile(v_first, load_row(v_first));
    v4i row_next = load_row(v_next);
    if (!ROLES && persistent && tid == 0)
        fetched = __hip_atomic_fetch_add(p.counters + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the first requests of a tile: both W slots, the scale chunk(s) of the first steps, X of the first step and
    // the first half of the second
    auto first_requests = [&](const Tile &t, const uint32_t (&raw)[Cfg::XI + 1]) {
        const int k1 = t.k0 + min(1, t.k1 - t.k0 - 1);  // second step (the first again for a one-step range)
        setup_w(t);
        issue_w(0, t.k0);
        issue_w(1, k1);
        setup_x(t, raw);
        issue_scales(t.k0 >> 3);
        if (SK && (t.k0 & 7) != 0 && (t.k0 >> 3) + 1 < nchunk) issue_scales((t.k0 >> 3) + 1);
        issue_xlo(0, t.k0);
        issue_xhi(0, t.k0);
        issue_xlo(1, k1);
    };
    if (cur.valid) {
        uint32_t raw[Cfg::XI + 1];
        gather(cur, raw);
        first_requests(cur, raw);
        ws_store(cur, 0, ws_load(cur));
    }
    wait_vmcnt<0>();
    if (!ROLES && persistent && tid == 0) sched[0] = 2u * per_xcd + fetched;
    __syncthreads();
    if (!ROLES && persistent) v_after = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[0]);

    uint32_t u_pos = v_first;  // stream-K: first unit of the current segment
    v4f acc[TM][TN];
    while (cur.valid) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
        const float *wsl = (const float *)(lds + Cfg::kWsOff + wsbuf * Cfg::ws_bytes(KB)) + ((wave_n * WNS) / kBlockN) * KB;

        // ---- the K loop
        if (grp == 1) phase_end();
        int slot = 0;
        const int kfirst = cur.k0, klast = cur.k1 - 1;
        // Dense persistent launches with an even number of K steps (the ring slots come out right), from one whole
        // tile to the next whole tile (the request offsets are the same): the last two steps of a tile, which have
        // nothing of their own left to request, request the first two steps of the next tile instead of repeating
        // the last step - the ring runs on across the tile boundary.
        bool prefetch = false;
        const uint8_t *xg_n = p.X, *wg_n = p.W;
        if constexpr (!GROUPED && !SK) {
            if (xt_ok) {
                const Tile nt = make_tile(v_next, row_next);
                prefetch = nt.valid && nt.rows == BM && nt.n0 + Cfg::BN <= p.N && cur.rows == BM && cur.n0 + Cfg::BN <= p.N;
                if (prefetch) {
                    xg_n = p.X + (int64_t)nt.m0 * p.ldx;
                    wg_n = p.W + (int64_t)nt.n0 * p.ldw;
                }
            }
        }
        for (int kb = kfirst; kb <= klast; ++kb) {
            const uint8_t *st = lds + slot * Cfg::kStage;
            const int cbuf = (kb >> 3) & 1;
            // A0 (LDS reads first: a DMA request can stall the wave's issue, the reads behind it would wait)
            const float ws_cur = wsl[kb];
            const float *sp = (const float *)(lds + sr8 + cbuf * Cfg::kChunkBytes + (kb & 7) * 4);
            v8i wf[TN], xf[HM];
            if (do_half0) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const v4i lo = *(const v4i *)(st + wr0 + j * 2048);
                    const v4i hi = *(const v4i *)(st + wr1 + j * 2048);
                    wf[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const bool do_half = h == 0 ? do_half0 : do_half1;
                float xs[HM];
                if (do_half) {
#pragma unroll
                    for (int i = 0; i < HM; ++i) {
                        const v4i lo = *(const v4i *)(st + xr0 + (h * HM + i) * 2048);
                        const v4i hi = *(const v4i *)(st + xr1 + (h * HM + i) * 2048);
                        xf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                        xs[i] = sp[(h * HM + i) * 16 * 8] * ws_cur;
                    }
                }
                if (h == 0) {
                    if ((kb & 7) == 0 && (kb >> 3) + 1 < nchunk) issue_scales((kb >> 3) + 1);
                    // (scalar selects, no branch: the body keeps its instruction order)
                    const bool nx = prefetch && kb + 1 > klast;
                    issue_xhi_at(slot ^ 1, (nx ? xg_n : xg) + (int64_t)(nx ? 0 : min(kb + 1, klast)) * kBlockK);
                } else {
                    const bool nx = prefetch && kb + 2 > klast;
                    const int64_t ko = (int64_t)(nx ? kb + 1 - klast : min(kb + 2, klast)) * kBlockK;  // next tile: step 0 or 1
                    issue_xlo_at(slot, (nx ? xg_n : xg) + ko);
                    issue_w_at(slot, (nx ? wg_n : wg) + ko);
                }
                // everything but the last two request groups has landed: at the end of A0 that covers the second
                // X half of this step, at the end of A1 the W rows and first X half of the next one (the scale
                // request of every eighth step only makes the wait one request stricter)
                wait_vmcnt<kXhi + kWXlo>();
                wait_lds();
                phase_end();
                // B0 / B1: the scale fold of a product is issued kLag MFMAs after its own MFMA, when the result
                // has long left the matrix pipe (a fold right behind the next MFMA would cost 7 idle issue
                // slots every other product)
                if (do_half) {
                    constexpr int E = HM * TN, kLag = 2;
                    v4f parts[kLag + 1];
#pragma unroll
                    for (int e = 0; e < E + kLag; ++e) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (e < E) parts[e % (kLag + 1)] = mfma_16x16x128_fp8(wf[e % TN], xf[e / TN], v4f{0.f, 0.f, 0.f, 0.f});
                        if (e >= kLag) {
                            const int f = e - kLag;
                            acc[h * HM + f / TN][f % TN] += parts[f % (kLag + 1)] * xs[f / TN];
                        }
                        if (e < E && e >= kLag) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // the MFMA first,
                            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // an older product's fold behind it
                        }
                    }
                }
                phase_end();
            }
            slot ^= 1;
        }
        if (grp == 0) phase_end();
        wait_vmcnt<0>();  // the re-fetches of the last steps have landed: the slots are free

        // ---- between two tiles: first requests of the next tile, then the stores of this one
        const Tile done = cur;
        float ws_first = 0.f;
        if constexpr (SK) {
            u_pos += (uint32_t)(done.k1 - done.k0);
            cur = make_tile(u_pos, v4i{-1, 0, 0, 0});
        } else {
            cur = make_tile(v_next, row_next);
        }
        if (cur.valid) {
            uint32_t raw[Cfg::XI + 1];
            gather(cur, raw);
            if (prefetch) {  // W and X of the first two steps were requested by the last two steps above
                setup_w(cur);
                setup_x(cur, raw);
                issue_scales(cur.k0 >> 3);
            } else {
                first_requests(cur, raw);
            }
            // sequence number and table row for later tiles (used one and two tiles from now)
            v_next = v_after;
            row_next = load_row(v_next);
            if (persistent && tid == 0)
                fetched = __hip_atomic_fetch_add(p.counters + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            wsbuf ^= 1;
            ws_first = ws_load(cur);
        }

        // ---- stream-K: a part of a tile goes to the workspace
        bool store_tile = true;
        if constexpr (SK) {
            if (done.k0 != 0 || done.k1 != KB) {  // the same for the whole workgroup
                constexpr uint32_t kBlockStride = Cfg::kThreads * 16;  // bytes between a lane's 16x16 blocks
                const Sc1Buffer xch(p.partials);
                const uint32_t lane_off = (uint32_t)tid * 16u;
                const uint32_t mine = (p.splits > 0 ? rank : 2u * rank + (done.k0 == 0 ? 1u : 0u)) * (uint32_t)Cfg::kPartialBytes + lane_off;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) xch.store(mine + (uint32_t)(i * TN + j) * kBlockStride, acc[i][j]);
                store_tile = false;  // the second launch (streamk_reduce_kernel) adds the parts and stores the tile
            }
        }

        // epilogue of the finished tile: lane (r16, g4) holds, for each tm, row wave_m*WMS + 16*tm + r16 and, for
        // each block pair h, the 8 columns n0 + wave_n*WNS + lane_col(g4, 2h) + [0, 8)
        if (store_tile) {
            const int nbase = done.n0 + wave_n * WNS;
            const int32_t *idx_list = GROUPED ? p.e2t_index + (int64_t)done.expert * p.num_pairs + done.m0 : nullptr;
            const float *w_list = GROUPED ? p.e2t_weight + (int64_t)done.expert * p.num_pairs + done.m0 : nullptr;
            float bias[BIAS ? 4 * TN : 1];
            if constexpr (BIAS) lane_bias<TN>(p, done.expert, nbase, g4, bias);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int rl = wave_m * WMS + 16 * i + r16;
                if (rl >= done.rows) continue;
                int64_t out_row;
                float rw = 1.0f;
                if constexpr (GROUPED) {
                    out_row = idx_list[rl];
                    if (p.mul_weight) rw = w_list[rl];
                } else {
                    out_row = done.m0 + rl;
                }
                uint16_t *cp = p.C + out_row * p.ldc + nbase;
                float o[4 * TN];
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int vv = 0; vv < 4; ++vv) {
                        if constexpr (BIAS) o[4 * j + vv] = (acc[i][j][vv] + bias[4 * j + vv]) * rw;
                        else o[4 * j + vv] = GROUPED ? acc[i][j][vv] * rw : acc[i][j][vv];
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
        wait_vmcnt<0>();
        if (cur.valid) {
            ws_store(cur, wsbuf, ws_first);
            if (persistent && tid == 0) sched[0] = ROLES ? fetched : 2u * per_xcd + fetched;
            __syncthreads();
            if (persistent) v_after = (uint32_t)__builtin_amdgcn_readfirstlane((int)sched[0]);
        }
    }
    if constexpr (ROLES) {
        __syncthreads();  // the other kind of tile lays the LDS out differently
        if (!small_first) small_blocks();
    }

    // ---- the last workgroup to finish leaves the counters zero for the next launch
    if (persistent && tid == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(p.counters + 8, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev == gridDim.x - 1) {
#pragma unroll
            for (int i = 0; i < Cfg::kCounterWords; ++i)
                __hip_atomic_store(p.counters + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Second launch of a stream-K GEMM: workgroup (tile, row block i) adds the parts of the tile that
// the first launch left in the workspace - in K order, so the result does not depend on the schedule - and stores
// the 16-row slices 16*i + [0, 16) of both wave rows.  Tiles that one workgroup computed whole were stored by it.
// `groups` is the grid size of the first launch.
__global__ __launch_bounds__(512) void streamk_reduce_kernel(const GemmArgs p, uint32_t groups) {
    using Cfg = PPCfg;
    constexpr int TN = Cfg::TN, WMS = Cfg::WMS, WNS = Cfg::WNS;
    constexpr uint32_t kBlockStride = Cfg::kThreads * 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 2, wave_n = wave & 3, r16 = lane & 15, g4 = lane >> 4;
    const uint32_t id = blockIdx.x / Cfg::TM, i = blockIdx.x % Cfg::TM;
    const uint32_t KB = (uint32_t)(p.K / kBlockK);
    const uint64_t units = (uint64_t)p.total_tiles * KB, t0 = (uint64_t)id * KB;
    // slots of the tile's parts in K order.  Runs cut from the unit sequence: the first rank's run ends inside the
    // tile (its second slot), every later one starts inside it (its first slot).  Panel split: slots
    // tile * splits + run.
    uint32_t r_lo, r_hi, first_slot, step;
    if (p.splits > 0) {
        r_lo = id * (uint32_t)p.splits;
        r_hi = r_lo + (uint32_t)p.splits - 1u;
        first_slot = r_lo;
        step = 1u;
    } else {
        r_lo = (uint32_t)(((t0 + 1u) * groups - 1u) / units);
        r_hi = (uint32_t)(((t0 + (uint64_t)KB) * groups - 1u) / units);
        if (r_lo == r_hi) return;
        first_slot = 2u * r_lo + 1u;
        step = 2u;
    }
    const uint8_t *base = (const uint8_t *)p.partials + (uint32_t)tid * 16u + i * TN * kBlockStride;
    v4f acc[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
        acc[j] = *(const v4f *)(base + (uint64_t)first_slot * Cfg::kPartialBytes + (uint32_t)j * kBlockStride);
    for (uint32_t r = r_lo + 1; r <= r_hi; ++r) {
        v4f part[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) part[j] = *(const v4f *)(base + (uint64_t)(step * r) * Cfg::kPartialBytes + (uint32_t)j * kBlockStride);
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[j] += part[j];
    }
    constexpr uint32_t GM = 8;
    const uint32_t width = GM * (uint32_t)p.tiles_n, g = id / width, first_m = g * GM;
    const uint32_t gsz = min((uint32_t)p.tiles_m - first_m, GM), in_grp = id - g * width;
    const int m0 = (int)(first_m + in_grp % gsz) * Cfg::BM, n0 = (int)(in_grp / gsz) * Cfg::BN;
    const int rl = wave_m * WMS + 16 * (int)i + r16;
    if (m0 + rl >= p.M) return;
    const int nbase = n0 + wave_n * WNS;
    uint16_t *cp = p.C + (int64_t)(m0 + rl) * p.ldc + nbase;
    float o[4 * TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) o[4 * j + vv] = acc[j][vv];
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

}  // namespace mi355

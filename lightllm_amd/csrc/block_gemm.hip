// Host side of the block-scaled FP8 GEMM entry points: argument checks, kernel choice, launches.
#include <cstdlib>

#include "gemm_pp.hpp"
#include "gemm_small.hpp"
#include "gemm_stream.hpp"
#include "gemm_streamcu.hpp"
#include "gemm_xshare.hpp"
#include "gemm_rows128.hpp"
#include "gemm_tile.hpp"

namespace mi355 {

// Correctness fallback for layouts the MFMA kernels do not take (B not K-contiguous, K not a multiple of
// 128, unaligned leading dimensions).  One thread per output element, same per-block arithmetic.
__device__ __forceinline__ float e4m3_to_f32(uint8_t b) {
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    const uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float v;
    if (e == 0) v = (float)m * 0.001953125f;  // m * 2^-9
    else v = as_f32(((e + 120u) << 23) | (m << 20));
    return as_f32(as_u32(v) | sign);
}

__global__ __launch_bounds__(256) void block_fp8_gemm_generic_kernel(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ As,
    const float *__restrict__ Bs, uint16_t *__restrict__ C, int M, int N, int K, int64_t lda, int64_t ldb_k,
    int64_t ldb_n, int64_t ldc, int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n, int block_n, int block_k,
    int out_f16) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)M * N) return;
    const int m = (int)(idx / N), n = (int)(idx % N);
    float acc = 0.f;
    int kb = 0;
    for (int k0 = 0; k0 < K; k0 += block_k, ++kb) {
        const int k1 = min(k0 + block_k, K);
        float d = 0.f;
        for (int k = k0; k < k1; ++k) d += e4m3_to_f32(A[m * lda + k]) * e4m3_to_f32(B[k * ldb_k + n * ldb_n]);
        acc += d * As[m * as_m + kb * as_k] * Bs[kb * bs_k + (n / block_n) * bs_n];
    }
    C[m * ldc + n] = (uint16_t)out_bits(acc, out_f16);
}

constexpr int kMaxLds = 160 * 1024;  // LDS per workgroup on gfx950

// X scales that can be fetched eight K steps at a time: row-major, 16-byte aligned rows, K/128 % 8 == 0.
static bool chunked_scales_ok(const GemmArgs &a) {
    return a.xs_k == 1 && (a.K / kBlockK) % 8 == 0 && a.xs_m % 4 == 0 && ((uintptr_t)a.Xs & 15) == 0;
}

template <int BM, int BN, int WM, int WN, int NSTAGE, int MODE, bool XS8, bool BIAS = false>
static int launch_tile_as(GemmArgs &a, int grid, hipStream_t st) {
    using Cfg = TileCfg<BM, BN, WM, WN, NSTAGE>;
    constexpr auto kernel = block_fp8_gemm_tile_kernel<BM, BN, WM, WN, NSTAGE, MODE, XS8, BIAS>;
    const int KB = a.K / kBlockK;
    // chunked scales keep two [BM rows][8 steps] buffers behind the common layout
    const int lds_bytes = XS8 ? ((Cfg::lds_bytes(KB) + 127) & ~127) + 2 * BM * 32 : Cfg::lds_bytes(KB);
    if (lds_bytes > kMaxLds) return MI355_EUNSUPPORTED;
    if (!allow_lds<kernel>(kMaxLds)) return MI355_ELAUNCH;
    return launch(kernel, dim3(grid), dim3(Cfg::kThreads), lds_bytes, st, a);
}

template <int BM, int BN, int WM, int WN, int NSTAGE, int MODE, bool BIAS = false>
static int launch_tile(GemmArgs &a, int grid, hipStream_t st) {
    using Cfg = TileCfg<BM, BN, WM, WN, NSTAGE>;
    constexpr bool kFits = ((Cfg::lds_bytes(144) + 127) & ~127) + 2 * BM * 32 <= kMaxLds;  // up to K = 18432
    if constexpr (kFits) {
        if (chunked_scales_ok(a)) {
            const int r = launch_tile_as<BM, BN, WM, WN, NSTAGE, MODE, true, BIAS>(a, grid, st);
            if (r != MI355_EUNSUPPORTED) return r;
        }
    }
    return launch_tile_as<BM, BN, WM, WN, NSTAGE, MODE, false, BIAS>(a, grid, st);
}

// A grouped launch of ring tiles, with or without the per-expert bias.
template <int BM, int BN, int WM, int WN, int NSTAGE>
static int launch_grouped_tile(GemmArgs &a, int grid, hipStream_t st) {
    if (a.bias) return launch_tile<BM, BN, WM, WN, NSTAGE, kGrouped, true>(a, grid, st);
    return launch_tile<BM, BN, WM, WN, NSTAGE, kGrouped, false>(a, grid, st);
}

#ifndef MI355_SK_PANEL
#define MI355_SK_PANEL 1
#endif
// Runs per tile of the panel split (0 = none): the most that keep tiles * runs within the compute units, with
// (m tiles * runs) a multiple of the 8 XCDs and at least 12 K steps in a run.
static int sk_panel_splits(int tiles_m, int tiles_n, int KB, int cus) {
    int best = 0;
    for (int s = 2; s <= 32; ++s) {
        if ((int64_t)tiles_m * tiles_n * s > cus || KB / s < 12) break;
        if ((tiles_m * s) % 8 == 0) best = s;
    }
    return best;
}

// Stream-K plan of the 256x256 kernel: the number of workgroups (one per compute unit, a multiple of 8), or 0 when
// the tiles fill whole rounds anyway or there is too little work to give every unit 16 K steps (the 128x128
// split-K tiles take those shapes).
static int stream_k_groups(int64_t tiles, int64_t KB, int cus, int64_t tiles_m = 0) {
    if (cus < 8 || tiles <= 0) return 0;
    // a panel split (see launch_pp) stands in for the cut of the unit sequence wherever the shape has one
    if (MI355_SK_PANEL && tiles_m > 0 && tiles % tiles_m == 0 &&
        sk_panel_splits((int)tiles_m, (int)(tiles / tiles_m), (int)KB, cus) > 0)
        return cus / 8 * 8;
    const int64_t units = tiles * KB;
    if (units >= (1ll << 31)) return 0;
    const int64_t groups = cus / 8 * 8;
    if (units / 16 < groups || tiles % groups == 0) return 0;
    return (int)groups;
}

// Whether the shape table should take that plan.  A workgroup that shares tiles no longer runs in step with the
// ones that read the same X and W panels, so its K steps are served by the memory side instead of the L2 and take
// about 2.5 times as long: sharing pays only where the plain loop leaves most of the device idle.
static bool stream_k_pays(int64_t tiles, int64_t KB, int cus, int64_t tiles_m) {
    // a panel split that fills three eighths of the device with runs of a long K: measured ahead of every other
    // kernel from 385 rows on (DeepSeek-V3 down, M = 1024: 128 us against 164 for one workgroup per tile; q_a+kv_a,
    // M = 2048: 49.6 against 67.9; Llama-3 down, M = 512: 48.8 against 67.8; N = 4096, K = 7168, M = 512, 128
    // workgroups: 34.5 against 39.8; N = 5120, K = 5120, M = 1024: 47.0 against 53.8), behind them with K = 4096
    const int panel = tiles % tiles_m == 0 ? sk_panel_splits((int)tiles_m, (int)(tiles / tiles_m), (int)KB, cus) : 0;
    if (MI355_SK_PANEL && panel > 0 && KB >= 40 && tiles * panel * 8 >= (int64_t)cus * 3) return true;
    const int groups = stream_k_groups(tiles, KB, cus);
    if (groups == 0) return false;
    const int64_t plain = (tiles + groups - 1) / groups * KB, shared = (tiles * KB + groups - 1) / groups;
    if (shared * 5 <= plain * 2) return true;
    // every tile shared by the same whole number of workgroups, none of which straddles two tiles, is a plain split
    // of K with half the partial tiles: it still pays at two workgroups per tile when their runs are long
    // (N = 4096, K = 14336, M = 2048: 128 tiles, 111 us against 130; N = 16384, K = 7168, M = 512, 28 steps each: 70.0
    // against 77.8; with K = 4096, 16 steps each, 51.6 against 43.7)
    return groups % tiles == 0 && shared * 2 <= plain && shared >= 28;
}

static size_t stream_k_workspace(int groups) {
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)2 * groups * PPCfg::kPartialBytes;
}

// The 256x256 ping-pong kernel.  a.tiles_m / a.tiles_n / a.total_tiles are set by the caller.  With a workspace
// whose counter words are zero the launch is persistent (one workgroup per CU, tiles handed out per XCD);
// without one every workgroup runs a single tile.  `sk_groups` > 0 asks for the stream-K launch with that many
// workgroups (dense only; the workspace must hold stream_k_workspace(sk_groups)).  Returns MI355_EUNSUPPORTED
// when the K range does not fit the kernel's LDS layout.
template <bool GROUPED, bool SK, bool SC4, bool BIAS = false>
static int launch_pp_as(GemmArgs &a, int grid, int lds_bytes, hipStream_t st) {
    constexpr auto kernel = block_fp8_gemm_pp_kernel<GROUPED, SK, SC4, false, BIAS>;
    if (!allow_lds<kernel>(kMaxLds)) return MI355_ELAUNCH;
    return launch(kernel, dim3(grid), dim3(PPCfg::kThreads), lds_bytes, st, a);
}

template <bool GROUPED>
static int launch_pp(GemmArgs &a, void *ws, size_t ws_bytes, int cus, int sk_groups, hipStream_t st) {
    const int lds_bytes = PPCfg::lds_bytes(a.K / kBlockK);
    if (lds_bytes > kMaxLds) return MI355_EUNSUPPORTED;
    if (a.xs_m < 0 || a.xs_k < 0) return MI355_EUNSUPPORTED;
    const bool sc4 = chunked_scales_ok(a);
    a.blocks_per_xcd = (a.total_tiles + 7) / 8;
    int per_xcd = a.blocks_per_xcd;
    a.counters = nullptr;
    const bool ws_ok = ws && ((uintptr_t)ws & 15) == 0;
    if constexpr (!GROUPED) {
        if (sk_groups > 0) {
            if (!ws_ok || ws_bytes < stream_k_workspace(sk_groups)) return MI355_EWORKSPACE;
            a.counters = (uint32_t *)ws;
            a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);
            // panel split where the shape allows it: every tile's K range in the same few runs, an XCD working on
            // one (m tile, run) pair across all n tiles, so that its L2 holds the X rows its workgroups share
            a.splits = MI355_SK_PANEL ? sk_panel_splits(a.tiles_m, a.tiles_n, a.K / kBlockK, cus) : 0;
            if (a.splits > 0) sk_groups = a.total_tiles * a.splits;
            const int r = sc4 ? launch_pp_as<false, true, true>(a, sk_groups, lds_bytes, st)
                              : launch_pp_as<false, true, false>(a, sk_groups, lds_bytes, st);
            if (r != MI355_OK) return r;
            return launch(streamk_reduce_kernel, dim3(a.total_tiles * PPCfg::TM), dim3(PPCfg::kThreads), 0, st, a,
                          (uint32_t)sk_groups);
        }
    }
    // persistent only when there is more than one tile per CU (a single round gains nothing from the tile queue)
    if (ws_ok && ws_bytes >= (size_t)MI355_WS_COUNTER_BYTES && per_xcd > cus / 8 && cus >= 8) {
        a.counters = (uint32_t *)ws;
        per_xcd = cus / 8;
    }
    if constexpr (GROUPED) {
        if (a.bias)
            return sc4 ? launch_pp_as<true, false, true, true>(a, per_xcd * 8, lds_bytes, st)
                       : launch_pp_as<true, false, false, true>(a, per_xcd * 8, lds_bytes, st);
    }
    return sc4 ? launch_pp_as<GROUPED, false, true>(a, per_xcd * 8, lds_bytes, st)
               : launch_pp_as<GROUPED, false, false>(a, per_xcd * 8, lds_bytes, st);
}

// Grouped launch over a 256-row schedule.  With a workspace that also holds the two block lists
// (grouped_workspace) the blocks of at most 64 rows go to the 64x512 streaming tile inside the same persistent
// launch: some workgroups of every XCD start on them, the others on the large blocks, and each moves on to the
// other queue when its own is empty.
static size_t grouped_workspace(int64_t table_rows) {
    return (size_t)MI355_WS_COUNTER_BYTES + (((size_t)(2 + 2 * table_rows) * 4 + 255) & ~(size_t)255);
}

template <auto Kernel>
struct KernelTag {
    static constexpr auto value = Kernel;
};

static int launch_grouped_pp(GemmArgs &a, void *ws, size_t ws_bytes, int cus, hipStream_t st) {
    const int KB = a.K / kBlockK;
    const int lds_roles = PPCfg::roles_sched_off(KB) + 16;
    const bool ws_ok = ws && ((uintptr_t)ws & 15) == 0 && ws_bytes >= grouped_workspace(a.tiles_m);
    if (!ws_ok || cus < 8 || a.total_tiles <= cus || lds_roles > kMaxLds || a.xs_m < 0 || a.xs_k < 0)
        return launch_pp<true>(a, ws, ws_bytes, cus, 0, st);
    int32_t *lists = (int32_t *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);
    const int r = launch(grouped_split_kernel, dim3(1), dim3(1024), 0, st, a.table, a.tiles_m, lists);
    if (r != MI355_OK) return r;
    a.lists = lists;
    a.counters = (uint32_t *)ws;
    a.blocks_per_xcd = (a.total_tiles + 7) / 8;
    const int per_xcd = cus / 8;
    a.small_first = per_xcd * 3 / 8;  // measured on the 256-expert routed batch: 8..14 of 32 are within 3 %
    auto go = [&](auto kernel_tag) {
        constexpr auto kernel = decltype(kernel_tag)::value;
        if (!allow_lds<kernel>(kMaxLds)) return (int)MI355_ELAUNCH;
        return launch(kernel, dim3(per_xcd * 8), dim3(PPCfg::kThreads), lds_roles, st, a);
    };
    const bool sc4 = chunked_scales_ok(a);
    if (a.bias)
        return sc4 ? go(KernelTag<block_fp8_gemm_pp_kernel<true, false, true, true, true>>{})
                   : go(KernelTag<block_fp8_gemm_pp_kernel<true, false, false, true, true>>{});
    return sc4 ? go(KernelTag<block_fp8_gemm_pp_kernel<true, false, true, true>>{})
               : go(KernelTag<block_fp8_gemm_pp_kernel<true, false, false, true>>{});
}

template <int BM, int BN, int WM, int WN, int NSTAGE, int MODE = kDense>
static int launch_dense(GemmArgs &a, hipStream_t st) {
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.N + BN - 1) / BN;
    a.total_tiles = a.tiles_m * a.tiles_n;
    a.blocks_per_xcd = (a.total_tiles + 7) / 8;
    return launch_tile<BM, BN, WM, WN, NSTAGE, MODE>(a, a.blocks_per_xcd * 8, st);
}

// Weight-streaming launches for M <= 64.
static int skinny_mt(int64_t M) { return M <= 16 ? 1 : (M <= 32 ? 2 : 4); }

struct SkinnyPlan {
    int tnw, splits, tiles;
};

static SkinnyPlan skinny_plan(int64_t M, int64_t N, int64_t K, int cus) {
    SkinnyPlan pl;
    pl.splits = 1;
    const int64_t t64 = (N + 63) / 64;
    // 64-row tiles that come to just over one per unit leave half the units with twice the work of the others:
    // narrower tiles then (N = 18432, K = 7168, 288 tiles of 64 rows, M = 1 / 16: 22.6 / 26.8 us against 27.9 /
    // 29.9; N = 18944, K = 3584: 13.2 / 15.2 against 16.4 / 17.3); up to 1.5 per unit for M > 16, where the narrower
    // tiles have 32 rows (N = 24576, K = 1536, M = 32 / 64: 10.3 / 15.3 against 12.2 / 18.7)
    bool unbalanced = t64 > cus && t64 * 4 <= (int64_t)cus * (M <= 16 ? 5 : 6);
    // up to 8 rows under a long K the 16-row tiles also win wherever the 64-row ones fill less than 84 % of their
    // last round (N = 36864, K = 7168, 2.25 per unit, M = 1 / 8: 39.6 / 41.5 us against 45.4 / 46.2; N = 22016,
    // K = 5120, 1.34 per unit: 19.9 / 21.4 against 22.7 / 23.4); with whole rounds they lose (N = 49152, M = 8: 41.6
    // against 38.5), and so they do on K = 4096
    if (M <= 8 && K >= 5120 && t64 > cus) {
        const int64_t rounds = (t64 + cus - 1) / cus;
        if (t64 * 25 < rounds * cus * 21) unbalanced = true;
    }
    if (t64 >= cus && !unbalanced) {
        // N alone gives every compute unit a workgroup: 64-row tiles, whole K
        pl.tnw = 4;
        pl.tiles = (int)((N + 63) / 64);
        return pl;
    }
    // Otherwise narrow tiles first, then K splits, until there are about two workgroups per compute unit (measured
    // on N=4096, K=14336: 16-row tiles x 2 splits 13.1 us at M <= 8 against 14.1 for 64-row tiles x 4 splits;
    // at M > 16, 32-row tiles x 4 splits 16.1 / 20.0 us at M = 32 / 64, 16-row tiles 18.3 / 25.8), never below 16 K
    // steps per workgroup (4 per wave).
    pl.tnw = M <= 16 ? 1 : 2;
    pl.tiles = (int)((N + 16 * pl.tnw - 1) / (16 * pl.tnw));
    const int KB = (int)(K / kBlockK);
    pl.splits = (2 * cus + pl.tiles - 1) / pl.tiles;
    // from 1.5 tiles per unit on K stays whole: two splits would make 3 to 4 workgroups per unit and an exchange
    // (N = 7168, K = 8192, 448 tiles, M = 1 / 16: 12.8 / 13.7 us against 16.7 / 17.9; 14336 x 4096, M = 32: 15.1
    // against 18.8; 6912 x 6912, M = 1: 10.2 against 12.3)
    if (pl.tiles * 2 >= 3 * cus) pl.splits = 1;
    const int max_splits = KB / 16 > 0 ? KB / 16 : 1;
    if (pl.splits > max_splits) pl.splits = max_splits;
    if (pl.splits < 1) pl.splits = 1;
    // a workgroup stages the activation scales of its K range in LDS if the range is short enough; one more split
    // that gets it there pays (N=7168, K=18432, M=16: 72 steps unstaged 37.5 us, 48 steps staged 30.7)
    const int cap = skinny_mt(M) == 4 ? StreamCfg<4, 2>::kMaxScaleSteps : StreamCfg<1, 1>::kMaxScaleSteps;
    const int need = (KB + cap - 1) / cap;
    if (pl.splits < need && need <= max_splits) pl.splits = need;
    return pl;
}

static size_t skinny_workspace(int64_t M, const SkinnyPlan &pl) {
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)pl.tiles * pl.splits * 16 * skinny_mt(M) * 16 * pl.tnw * 4;
}

// Preconditions of the stream kernel beyond the fast layout.
static int skinny_check(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t as_m, int cus,
                        bool ws_usable, size_t ws_bytes) {
    if (M > 64) return MI355_EUNSUPPORTED;
    // rows are addressed from the matrix bases with 32-bit byte offsets
    if (N * ldw >= (1ll << 32) || M * lda >= (1ll << 32) || M * as_m >= (1ll << 32)) return MI355_EUNSUPPORTED;
    const SkinnyPlan pl = skinny_plan(M, N, K, cus);
    if ((int64_t)pl.tiles * 4 > MI355_WS_COUNTER_BYTES) return MI355_EUNSUPPORTED;
    if (pl.splits > 1 && (!ws_usable || ws_bytes < skinny_workspace(M, pl))) return MI355_EWORKSPACE;
    return MI355_OK;
}

template <int MT, int TNW, bool XSL>
static int launch_stream_as(GemmArgs &a, const SkinnyPlan &pl, void *ws, int lds_bytes, hipStream_t st) {
    using Cfg = StreamCfg<MT, TNW>;
    constexpr int max_lds = Cfg::kLds + (XSL ? Cfg::scale_lds_bytes(Cfg::kMaxScaleSteps) : 0);
    constexpr auto whole_k = block_fp8_gemm_stream_kernel<MT, TNW, false, XSL>;
    constexpr auto split_k = block_fp8_gemm_stream_kernel<MT, TNW, true, XSL>;
    if (pl.splits <= 1) {
        if (!allow_lds<whole_k>(max_lds)) return MI355_ELAUNCH;
        return launch(whole_k, dim3(pl.tiles), dim3(256), lds_bytes, st, a);
    }
    if (!allow_lds<split_k>(max_lds)) return MI355_ELAUNCH;
    a.splits = pl.splits;
    a.counters = (uint32_t *)ws;
    a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);
    return launch(split_k, dim3(pl.tiles * pl.splits), dim3(256), lds_bytes, st, a);
}

// The activation scales of a CTA's K range are staged in LDS when the range is short enough for the staging area.
template <int MT, int TNW>
static int launch_stream(GemmArgs &a, const SkinnyPlan &pl, void *ws, hipStream_t st) {
    using Cfg = StreamCfg<MT, TNW>;
    const int KB = a.K / kBlockK;
    const int steps = (KB + pl.splits - 1) / pl.splits;
    if (steps <= Cfg::kMaxScaleSteps)
        return launch_stream_as<MT, TNW, true>(a, pl, ws, Cfg::kLds + Cfg::scale_lds_bytes(steps), st);
    return launch_stream_as<MT, TNW, false>(a, pl, ws, Cfg::kLds, st);
}

template <int MT>
static int launch_stream_mt(GemmArgs &a, const SkinnyPlan &pl, void *ws, hipStream_t st) {
    switch (pl.tnw) {
        case 4: return launch_stream<MT, 4>(a, pl, ws, st);
        case 2: return launch_stream<MT, 2>(a, pl, ws, st);
        case 1:
            if constexpr (MT == 1) return launch_stream<1, 1>(a, pl, ws, st);
            return MI355_EINVAL;
        default: return MI355_EINVAL;
    }
}

// ---- the weight stream cut into one equal share per compute unit (gemm_streamcu.hpp): TNW 16-row blocks per
// workgroup with TNW = ceil(N / 16 / cus), one workgroup of 8 waves per tile, whole K.  Returns TNW, or 0 where the
// kernel does not apply: more than 16 rows, more than 5 blocks per unit, tiles that fill under 85 % of the units,
// fewer than two K steps per wave, offsets past 32 bits or scales that do not fit the LDS.
static int streamcu_tnw(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t as_m, int cus) {
    if (M > 16 || cus <= 0) return 0;
    const int64_t blocks = (N + 15) / 16, KB = K / kBlockK;
    const int64_t tnw = (blocks + cus - 1) / cus;
    if (tnw > 5 || KB < 16 || KB > CuStreamCfg<1, 1>::max_steps()) return 0;
    const int64_t tiles = (blocks + tnw - 1) / tnw;
    if (tiles * 20 < (int64_t)cus * 17) return 0;
    if (N * ldw >= (1ll << 32) || M * lda >= (1ll << 32) || M * as_m >= (1ll << 32)) return 0;
    if (8 * ((16 * tnw + 16) * 128) + KB * (17 + 2) * 4 > kMaxLds) return 0;
    return (int)tnw;
}

// Where it is ahead of the streaming kernel (M = 1 / 8 / 16, weights rotated past the memory-side cache): wherever
// that kernel has to share K between workgroups (N = 4096, K = 14336: 12.3 - 13.0 / 12.6 - 13.4 / 13.6 - 14.4 us
// against 13.4 / 13.7 / 14.9; N = 7168, K = 18432: 23.1 / 23.9 / 25.4 against 26.6 / 28.8 / 30.9), and from three
// row blocks per unit on, where the 64-row tiles fill their last round badly (N = 14336, K = 4096: 13.4 / 13.5 / 14.0
// against 14.5 / 15.0 / 16.0; N = 18432, K = 7168: 23.4 / 23.3 / 23.6 against 23.0 / 24.0 / 27.1).  With one or two
// blocks per unit and K unshared the 16-row tiles of the streaming kernel are ahead (N = 7168, K = 8192: 16.6
// against 12.9).
static bool streamcu_pays(int64_t M, int64_t N, int64_t K, int cus) {
    const int tnw = streamcu_tnw(M, N, K, K, K, K / kBlockK, cus);
    if (tnw == 0) return false;
    return skinny_plan(M, N, K, cus).splits > 1 || tnw >= 3;
}

template <int TNW>
static int launch_streamcu_as(GemmArgs &a, hipStream_t st) {
    using Cfg = CuStreamCfg<1, TNW>;
    constexpr auto kernel_lo = block_fp8_gemm_streamcu_kernel<1, TNW, false>;
    constexpr auto kernel_hi = block_fp8_gemm_streamcu_kernel<1, TNW, true>;
    const int lds_bytes = Cfg::lds_bytes(a.K / kBlockK);
    if (lds_bytes > kMaxLds) return MI355_EUNSUPPORTED;
    const int tiles = (a.N + Cfg::BN - 1) / Cfg::BN;
    if (a.M <= 8) {
        if (!allow_lds<kernel_lo>(kMaxLds)) return MI355_ELAUNCH;
        return launch(kernel_lo, dim3(tiles), dim3(Cfg::kThreads), lds_bytes, st, a);
    }
    if (!allow_lds<kernel_hi>(kMaxLds)) return MI355_ELAUNCH;
    return launch(kernel_hi, dim3(tiles), dim3(Cfg::kThreads), lds_bytes, st, a);
}

static int launch_streamcu(GemmArgs &a, int tnw, hipStream_t st) {
    switch (tnw) {
        case 1: return launch_streamcu_as<1>(a, st);
        case 2: return launch_streamcu_as<2>(a, st);
        case 3: return launch_streamcu_as<3>(a, st);
        case 4: return launch_streamcu_as<4>(a, st);
        case 5: return launch_streamcu_as<5>(a, st);
        default: return MI355_EUNSUPPORTED;
    }
}

// ---- the second streaming kernel (activation block shared by the workgroup).  Measured against the first one on
// the Llama decode shapes it wins only where the first is shortest of registers and N alone fills the device:
// M = 33..64 with 128-row workgroup tiles (N=28672, K=4096, M=64: 29.7 us against 34.4); with 64-row tiles, few
// tiles or smaller M its barrier per K step costs more than the shared activation block saves
// (N=4096, K=14336: 21.5-25.2 us against 13.9-19.8).  Only that configuration is built.
constexpr int kXshareDepth = 4;
using XshareCfg = ShareCfg<4, 2, kXshareDepth>;

static bool xshare_pays(int64_t M, int64_t N, int64_t K, int cus) {
    return M > 32 && M <= 64 && (N + 127) / 128 >= (int64_t)cus * 3 / 4 && K / kBlockK <= XshareCfg::kMaxScaleSteps;
}

// 128-row workgroup tiles; the K range is split in two while that leaves fewer than two workgroups per compute unit
// (224 tiles unsplit take 34.7 us on N=28672, K=4096, M=64; split in two, 29.7), never below 8 K steps each.
static int xshare_splits(int64_t N, int64_t K, int cus) {
    const int64_t tiles = (N + XshareCfg::BN - 1) / XshareCfg::BN, KB = K / kBlockK;
    return tiles < 2 * (int64_t)cus && KB >= 16 ? 2 : 1;
}

static size_t xshare_workspace(int64_t N, int splits) {
    const int64_t tiles = (N + XshareCfg::BN - 1) / XshareCfg::BN;
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)tiles * splits * XshareCfg::kTileElems * 4;
}

static int launch_xshare(GemmArgs &a, int splits, void *ws, hipStream_t st) {
    const int KB = a.K / kBlockK;
    const int steps = (KB + splits - 1) / splits;
    if (steps > XshareCfg::kMaxScaleSteps) return MI355_EUNSUPPORTED;
    constexpr int max_lds = XshareCfg::kLds + XshareCfg::scale_lds_bytes(XshareCfg::kMaxScaleSteps);
    const int lds_bytes = XshareCfg::kLds + XshareCfg::scale_lds_bytes(steps);
    const int tiles = (a.N + XshareCfg::BN - 1) / XshareCfg::BN;
    if (splits <= 1) {
        constexpr auto kernel = block_fp8_gemm_xshare_kernel<4, 2, kXshareDepth, false>;
        if (!allow_lds<kernel>(max_lds)) return MI355_ELAUNCH;
        return launch(kernel, dim3(tiles), dim3(256), lds_bytes, st, a);
    }
    constexpr auto kernel = block_fp8_gemm_xshare_kernel<4, 2, kXshareDepth, true>;
    if (!allow_lds<kernel>(max_lds)) return MI355_ELAUNCH;
    a.splits = splits;
    a.counters = (uint32_t *)ws;
    a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);
    return launch(kernel, dim3(tiles * splits), dim3(256), lds_bytes, st, a);
}

// ---- at most 384 rows: the weight stream with the activation block in LDS (gemm_rows128.hpp).  Up to 128 rows a
// workgroup takes 256 weight rows on three ring slots, beyond that 128 weight rows on two (the activation block of a
// step is two to three times as large).
constexpr int kRows128MinSteps = 6;

static int rows128_mt(int64_t M) { return (int)((M + 15) / 16); }
constexpr int64_t kRows128NarrowMaxM = 208;  // the last row count with narrow workgroups above 128 rows

// Workgroup width, K sharing and tile count of a launch.  Up to 128 rows a workgroup is 8 waves x 32 weight rows;
// beyond, 8 waves x 16.  While the tiles leave compute units idle the K range is shared, never below
// kRows128MinSteps K steps for a workgroup.  Up to 128 rows there is a second way to occupy the idle units: narrower
// workgroups (5 or 6 waves) with K unshared - a unit's pull covers the X block and the W rows of a step alike, so
// more, narrower workgroups mean fewer bytes per unit.  It is taken when such a width gives between 0.55 cus and cus
// tiles (DeepSeek-V3 gate_up, N = 36864: 231 tiles of 160 rows, M = 64 / 128: 50.3 / 62.8 us against 59.4 / 68.8
// for 144 tiles of 256; q_b, N = 24576, K = 1536: 16.6 against 21.4 with K shared by two).
struct Rows128Plan {
    int wv, bn, splits, tiles, tn;
};

static Rows128Plan rows128_plan(int64_t M, int64_t N, int64_t K, int cus) {
    Rows128Plan pl;
    const int64_t KB = K / kBlockK;
    pl.wv = 8;
    pl.bn = M <= 128 ? 256 : 128;
    pl.tn = M <= 128 ? 2 : 1;
    if (M <= 128) {
        for (int wv = 5; wv <= 6; ++wv) {
            const int64_t tiles = (N + 32 * wv - 1) / (32 * wv);
            if (tiles <= cus && tiles * 20 >= (int64_t)cus * 11) {
                pl.wv = wv;
                pl.bn = 32 * wv;
                pl.splits = 1;
                pl.tiles = (int)tiles;
                return pl;
            }
        }
    }
    if (M > 128 && M <= kRows128NarrowMaxM) {
        // one round of workgroups of just the width that fits it: two 16-row blocks per wave (5..8 waves, 160..256
        // weight rows) where N is wide enough for that, else one (4..7 waves, 64..112 weight rows)
        const int64_t wv2 = (N + 32 * (int64_t)cus - 1) / (32 * (int64_t)cus);
        int64_t wv1 = (N + 16 * (int64_t)cus - 1) / (16 * (int64_t)cus);
        if (wv1 < 4) wv1 = 4;
        const int tn = wv2 >= 5 ? 2 : 1;
        const int64_t wv = tn == 2 ? wv2 : wv1, bn = 16 * tn * wv;
        const int64_t tiles = (N + bn - 1) / bn;
        // (four-wave workgroups fall behind the 128x128 tiles a little earlier: N = 16384, K = 7168, M = 208: 63.6 us
        // against 60.9)
        if (wv <= (tn == 2 ? 8 : 7) && (wv > 4 || M <= 192) && tiles <= cus && tiles * 20 >= (int64_t)cus * 11) {
            pl.wv = (int)wv;
            pl.bn = (int)bn;
            pl.splits = 1;
            pl.tiles = (int)tiles;
            pl.tn = tn;
            return pl;
        }
    }
    const int64_t tiles = (N + pl.bn - 1) / pl.bn;
    int64_t splits = cus / tiles;
    if (splits > KB / kRows128MinSteps) splits = KB / kRows128MinSteps;
    pl.splits = (int)(splits < 1 ? 1 : splits);
    pl.tiles = (int)tiles;
    return pl;
}

static int rows128_splits(int64_t M, int64_t N, int64_t K, int cus) { return rows128_plan(M, N, K, cus).splits; }

static size_t rows128_workspace(int64_t M, int64_t N, int64_t K, int cus) {
    const Rows128Plan pl = rows128_plan(M, N, K, cus);
    if (pl.splits <= 1) return 0;
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)pl.tiles * pl.splits * 16 * rows128_mt(M) * pl.bn * 4;
}

// Where the kernel pays (Llama-3-8B and DeepSeek-V3 linears, weights rotated so that none is found in the
// memory-side cache).  At 65..128 rows it beats the 128x128 tiles by 10 to 30 % (DeepSeek-V3 down, M = 128: 39.5 us
// against 50.0; Llama-3 down: 27.9 against 30.3) unless K is short (q_b, K = 1536: 21.7 against 17.0).  At 33..64
// rows it beats the streaming kernels on the large weights (DeepSeek-V3 gate_up, down, o at M = 64: 58.4, 31.7,
// 31.9 us against 72.3, 42.5, 43.1) and loses on the small ones, where its second launch shows (Llama-3 qkv: 15.0
// against 13.1); at 32 rows and fewer the streaming kernels are the faster ones but for one case (below).
static bool rows128_pays(int64_t M, int64_t N, int64_t K, int cus) {
    if (M > 384 || M < 16) return false;
    if (M <= 32) {
        // 16..32 rows: only where the streaming kernel's 64-row workgroups (two fit a unit) spill into a second,
        // mostly empty round and this kernel has a well-filled single launch (N = 36864, K = 7168: 576 workgroups on
        // 512 slots, M = 24 / 32 51.1 / 52.5 us against 46.6 / 46.8 here; on N = 28672, 448 workgroups, the
        // streaming kernel keeps its lead, 23.8 against 27.4)
        const int64_t t64 = (N + 63) / 64;
        const Rows128Plan pl = rows128_plan(M, N, K, cus);
        // likewise on large weights whose 64-row workgroups come to just over one per unit (N = 18432, K = 7168,
        // 288 of them, M = 16 / 32: 27.5 / 28.4 us against 30.3 / 34.4), and under a very long K (N = 8192,
        // K = 28672: 45.3 / 47.0 against 50.7 / 54.6; N = 7168, K = 18432: 27.2 / 28.5 against 30.9 / 31.4)
        if (N * K >= 100000000ll && pl.tiles <= cus &&
            ((t64 > cus && t64 * 4 <= 5 * (int64_t)cus) || K >= 18432))
            return true;
        return t64 > 2 * (int64_t)cus && t64 <= 3 * (int64_t)cus && pl.splits == 1 && pl.tiles <= cus &&
               pl.tiles * 20 >= (int64_t)cus * 11;
    }
    if (M > 256) {
        // 257..384 rows (the activation block of a step is 48 KiB): still ahead where the 128-row tiles are few, K is
        // long and the weights are not small (Llama-3 down at M = 257 / 384: 38.0 / 46.8 us against 66.3 / 66.5;
        // DeepSeek-V3 down 70.6 / 86.6 against 97.7 / 106.4; Llama-3 qkv 26.0 / 32.0 against 36.3); on 15 MB of
        // weights (q_a+kv_a) it is not (24.1 against 23.5 at M = 320)
        const int64_t tiles = (N + 127) / 128;
        // from about 340 rows on the 256x256 tiles with a panel split of K overtake it on the large weights
        // (DeepSeek-V3 down, M = 352 / 384: 79.4 / 78.3 us against 82.9 / 87.5; Llama-3 down stays: 49.7 against 44.8)
        if (M > 336 && N * K >= 100000000ll &&
            stream_k_pays(((M + 255) / 256) * ((N + 255) / 256), K / kBlockK, cus, (M + 255) / 256))
            return false;
        // (with more than cus/4 tiles of 128 weight rows only up to 320 rows: N = 10240, K = 8192, M = 257 / 300:
        // 49.4 / 53.4 us against 68.8 / 68.9; N = 14336, K = 5120: 48.3 / 49.7 against 54.3 / 54.0; at M = 384 the
        // 128x128 tiles are ahead there - N = 16384, K = 4096: 44.7 against 56.6; N = 12288: 43.3 against 48.9)
        return K / kBlockK >= 16 && N * K >= 20000000ll && tiles * 2 <= cus && (tiles * 4 <= cus || M <= 320) &&
               tiles * rows128_splits(M, N, K, cus) * 2 >= cus;
    }
    if (M > 128) {
        // 129..256 rows, 128-row tiles.  Against the 128x128 tiles it wins where those are few and K is long
        // (DeepSeek-V3 down at M = 129 / 256: 44.8 / 62.4 us against 83.9 / 84.6; Llama-3 down 25.3 / 34.7 against
        // 42.5), and up to 160 rows also where the tiles about fill the device (Llama-3 gate_up, 224 tiles, M = 160:
        // 40.1 against 46.7; M = 192: 49.2 against 46.8).  With more tiles than units it loses (DeepSeek-V3 gate_up).
        const int64_t tiles = (N + 127) / 128;
        // up to 208 rows a single round of narrower workgroups (160..256 weight rows at two blocks per wave, 64..112
        // at one) beats the square tiles (N = 36864, K = 7168, M = 144 / 192: 69.1 / 80.5 us against 82.7 / 85.9;
        // N = 28672, K = 4096: 35.8 / 42.0 against 43.3 / 48.4; q_b, K = 1536: 15.3 / 18.3 against 19.6 / 21.3);
        // its time grows with M (every wave reads the whole X block from LDS) and the square tiles are level or
        // ahead from about 220 rows
        {
            const Rows128Plan pl = rows128_plan(M, N, K, cus);
            if (pl.tn == 2 || pl.wv != 8) return true;
        }
        if (K / kBlockK < 16) return false;
        // from about 200 rows the panel split of the 256x256 tiles is level or ahead on the large weights, its time
        // flat in M (DeepSeek-V3 down, M = 208 / 240 / 256: 55.1 / 54.9 / 56.9 us against 58.4 / 60.4 / 63.3;
        // o_proj 53.1 / 52.8 / 58.1 against 54.9 / 57.5 / 57.6)
        if (M > 200 && N * K >= 100000000ll && stream_k_pays((N + 255) / 256, K / kBlockK, cus, 1)) return false;
        // and on small weights the 128x128 tiles with K shared (N = 4096, K = 4096, M = 224 / 256: 18.9 / 19.0 us
        // against 20.9 / 21.3; N = 7168, K = 2304, M = 256: 19.7 against 23.0)
        if (M > 192 && N * K < 20000000ll) return false;
        if (tiles * 2 <= cus) return tiles * rows128_splits(M, N, K, cus) * 2 >= cus;
        return tiles <= cus && (M <= 160 || (M <= kRows128NarrowMaxM && tiles * 8 >= (int64_t)cus * 7));
    }
    // up to 128 rows: a single well-filled launch always pays (narrow or full-width workgroups on 0.55 cus .. cus
    // tiles with K unshared: DeepSeek-V3 gate_up at M = 64: 49.7 us against 69.9 - 72.5 for the streaming kernels,
    // q_b 12.5 against 15.0, Llama-3 gate_up 29.5 against 29.8)
    const Rows128Plan pl = rows128_plan(M, N, K, cus);
    if (pl.splits == 1 && pl.tiles <= cus && pl.tiles * 20 >= (int64_t)cus * 11) return true;
    if (M > 64) return K / kBlockK >= 16;
    // 33..64 rows with K shared or more tiles than units: on the large weights, and not where the
    // shared-activation streaming kernel runs (lm_head, N = 128256, K = 4096, M = 64: 116 us against 110 - its small
    // workgroups fill the second round better)
    if (pl.tiles > cus || xshare_pays(M, N, K, cus)) return false;
    // ... unless the streaming kernel's workgroups come out as one per unit with K whole (N = 16384, K = 7168,
    // M = 64: 25.9 us against 29.9) ...
    const SkinnyPlan sp = skinny_plan(M, N, K, cus);
    const int64_t wgs = (int64_t)sp.tiles * sp.splits;
    if (N * K >= 100000000ll) return !(sp.splits == 1 && wgs == cus);
    // ... and on the mid-size ones (from 35 MB) where they come out as neither one nor two per unit: N = 10240,
    // K = 8192 (640 of them), M = 64: 24.5 us against 33.6; 14336 x 4096 (896): 19.6 against 24.0; 12288 x 4096 (768):
    // 18.0 against 22.4; 5120 x 13824 (640): 21.4 against 28.8.  With 512 or 256 of them it keeps its lead (8192 x
    // 8192: 21.3 against 22.9; 16384 x 4096: 18.7 against 21.3), and on smaller weights the second launch shows
    // (6144 x 4096: 12.8 against 14.6).
    return N * K >= 35000000ll && wgs != cus && wgs != 2 * (int64_t)cus;
}

static bool rows128_limits_ok(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t as_m, int64_t as_k, int cus) {
    if (M > 384) return false;
    if (M * lda >= (1ll << 32) || M * as_m * 4 >= (1ll << 32) || as_k * 32 >= (1ll << 32)) return false;
    const Rows128Plan pl = rows128_plan(M, N, K, cus);
    const int64_t steps = (K / kBlockK + pl.splits - 1) / pl.splits;
    // Rows128Cfg::lds_bytes for the plan's tile: the ring, the W scales of the tile's n blocks, two X scale chunks
    const int64_t mt = rows128_mt(M), ns = mt <= 8 ? 3 : 2, nblk = (pl.bn + 2 * kBlockN - 2) / kBlockN;
    const int64_t ring = ns * (16 * mt * 128 + (int64_t)pl.bn * 128);
    return ((ring + nblk * steps * 4 + 127) & ~127ll) + 2 * 16 * mt * 32 <= 160 * 1024;
}

template <int MT, int WV, int TN = (MT <= 8 ? 2 : 1)>
static int launch_rows128_as(GemmArgs &a, const Rows128Plan &pl, void *ws, hipStream_t st) {
    constexpr int NS = MT <= 8 ? 3 : 2;
    using Cfg = Rows128Cfg<MT, NS, TN, WV>;
    const int KB = a.K / kBlockK;
    const int steps = (KB + pl.splits - 1) / pl.splits;
    const int lds_bytes = Cfg::lds_bytes(steps);
    if (lds_bytes > 160 * 1024) return MI355_EUNSUPPORTED;
    if (pl.splits <= 1) {
        constexpr auto kernel = block_fp8_gemm_rows128_kernel<MT, NS, TN, WV, false>;
        if (!allow_lds<kernel>(160 * 1024)) return MI355_ELAUNCH;
        return launch(kernel, dim3(pl.tiles), dim3(Cfg::kThreads), lds_bytes, st, a);
    }
    if constexpr (WV == 8 && TN == (MT <= 8 ? 2 : 1)) {
        constexpr auto kernel = block_fp8_gemm_rows128_kernel<MT, NS, TN, 8, true>;
        if (!allow_lds<kernel>(160 * 1024)) return MI355_ELAUNCH;
        a.splits = pl.splits;
        a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);  // the counter words stay untouched
        const int r = launch(kernel, dim3(pl.tiles * pl.splits), dim3(Cfg::kThreads), lds_bytes, st, a);
        if (r != MI355_OK) return r;
        return launch(rows128_reduce_kernel<MT, TN>, dim3((pl.tiles * Cfg::kWaves * MT + 3) / 4), dim3(256), 0, st, a);
    }
    return MI355_EINVAL;  // narrow workgroups never share K
}

template <int MT>
static int launch_rows128(GemmArgs &a, const Rows128Plan &pl, void *ws, hipStream_t st) {
    if constexpr (MT <= 8) {
        if (pl.wv == 5) return launch_rows128_as<MT, 5>(a, pl, ws, st);
        if (pl.wv == 6) return launch_rows128_as<MT, 6>(a, pl, ws, st);
    } else if constexpr (MT <= (kRows128NarrowMaxM + 15) / 16) {
        if (pl.tn == 2) {
            switch (pl.wv) {
            case 5: return launch_rows128_as<MT, 5, 2>(a, pl, ws, st);
            case 6: return launch_rows128_as<MT, 6, 2>(a, pl, ws, st);
            case 7: return launch_rows128_as<MT, 7, 2>(a, pl, ws, st);
            case 8: return launch_rows128_as<MT, 8, 2>(a, pl, ws, st);
            default: return MI355_EINVAL;
            }
        }
        switch (pl.wv) {
        case 4: return launch_rows128_as<MT, 4>(a, pl, ws, st);
        case 5: return launch_rows128_as<MT, 5>(a, pl, ws, st);
        case 6: return launch_rows128_as<MT, 6>(a, pl, ws, st);
        case 7: return launch_rows128_as<MT, 7>(a, pl, ws, st);
        default: break;
        }
    }
    return launch_rows128_as<MT, 8>(a, pl, ws, st);
}

// ---- more rows than that on a narrow N: the same kernel tiled over M as well (tiles_m x tiles_n workgroups in one
// round, K unshared).  Where N gives few 256-wide tiles the 256x256 launch leaves most units idle (N = 2112: 9 tile
// columns, 144 tiles at M = 4096, 72 at M = 2048) and its lone round is bound by the latency of its K steps; tiles of
// 16*mt rows x 32*wv weight rows with mt chosen so that tiles_m * tiles_n just fits the units put a workgroup on
// (nearly) every unit, each with less to load and to multiply per step.
struct RowsMPlan {
    int mt, wv, tiles_m, tiles_n;
};

static RowsMPlan rowsm_plan(int64_t M, int64_t N, int64_t /*K*/, int cus) {
    RowsMPlan best = {0, 0, 0, 0};
    if (M <= 0 || cus < 8) return best;
    const int64_t blocks = (M + 15) / 16;
    int64_t best_bytes = 0;
    for (int wv = 8; wv >= 5; --wv) {
        const int64_t tn = (N + 32 * wv - 1) / (32 * wv);
        if (tn > cus) continue;
        const int64_t room = cus / tn;                       // m tiles that fit one round
        const int64_t mt = (blocks + room - 1) / room;       // row blocks per tile
        if (mt > 13 || (mt <= 8 && wv == 7)) continue;       // kernels built: 5, 6, 8 waves up to 8 blocks; 5..8 up to 13
        const int64_t tm = (blocks + mt - 1) / mt;
        if (tm < 2 || tm * tn * 20 < (int64_t)cus * 11) continue;
        const int64_t bytes = (16 * mt + 32 * wv) * 128;      // what a unit loads per K step
        if (best.mt == 0 || mt < best.mt || (mt == best.mt && bytes < best_bytes)) {
            best = {(int)mt, wv, (int)tm, (int)tn};
            best_bytes = bytes;
        }
    }
    return best;
}

static bool rowsm_limits_ok(const RowsMPlan &pl, int64_t M, int64_t K, int64_t lda, int64_t as_m, int64_t as_k) {
    if (pl.mt == 0) return false;
    if (M * lda >= (1ll << 32) || M * as_m * 4 >= (1ll << 32) || as_k * 32 >= (1ll << 32)) return false;
    const int64_t steps = K / kBlockK, ns = pl.mt <= 8 ? 3 : 2, bn = 32 * pl.wv, nblk = (bn + 2 * kBlockN - 2) / kBlockN;
    const int64_t ring = ns * (16 * pl.mt * 128 + bn * 128);
    return ((ring + nblk * steps * 4 + 127) & ~127ll) + 2 * 16 * pl.mt * 32 <= 160 * 1024;
}

// Where it pays (forced against the table's previous choice over N = 1024..8192, K = 1536..14336, M = 400..4096,
// 256 units).  With K <= 5120 and at most 8 row blocks per tile (three ring slots) it is ahead on every N <= 5120:
// 1.2 to 2.0 times with up to 4 row blocks (N = 4096, K = 4096, M = 512 / 1024 / 2048: 22.4 / 28.8 / 42.0 us against
// 27.9 / 36.5 / 47.2; N = 2112, K = 2048, M = 1024: 1.95 times), 1.0 to 1.2 with 5..8; from N = 6144 on and with more
// row blocks (two slots) the square tiles are level or ahead.  With K = 6144 .. 7168 the panel split of the 256x256
// tiles shares K between idle units and takes most of the gain: 2..6 row blocks on N <= 3072 are still 1.04 to 1.3
// times ahead (q_a+kv_a, N = 2112, K = 7168, M = 512 / 1024 / 2048: 1.11 / 1.12 / 1.04), a single block or a wider N
// is behind.  From K = 8192 on the kernels that share K win everywhere.
static bool rowsm_pays(int64_t M, int64_t N, int64_t K, int cus) {
    if (M <= 384) return false;
    const int64_t KB = K / kBlockK;
    if (KB < 12 || KB > 56) return false;
    const RowsMPlan pl = rowsm_plan(M, N, K, cus);
    if (pl.mt == 0 || pl.mt > 8) return false;
    if (KB <= 40) return N <= 5120;
    return pl.mt >= 2 && pl.mt <= 6 && N <= 3072;
}

template <int MT>
static int launch_rowsm_mt(GemmArgs &a, const Rows128Plan &pl, hipStream_t st) {
    if constexpr (MT <= 8) {
        switch (pl.wv) {
            case 5: return launch_rows128_as<MT, 5>(a, pl, nullptr, st);
            case 6: return launch_rows128_as<MT, 6>(a, pl, nullptr, st);
            case 8: return launch_rows128_as<MT, 8>(a, pl, nullptr, st);
            default: return MI355_EINVAL;
        }
    } else {
        switch (pl.wv) {
            case 5: return launch_rows128_as<MT, 5, 2>(a, pl, nullptr, st);
            case 6: return launch_rows128_as<MT, 6, 2>(a, pl, nullptr, st);
            case 7: return launch_rows128_as<MT, 7, 2>(a, pl, nullptr, st);
            case 8: return launch_rows128_as<MT, 8, 2>(a, pl, nullptr, st);
            default: return MI355_EINVAL;
        }
    }
}

static int launch_rowsm(GemmArgs &a, const RowsMPlan &mp, hipStream_t st) {
    a.tiles_m = mp.tiles_m;
    a.tiles_n = mp.tiles_n;
    a.total_tiles = mp.tiles_m * mp.tiles_n;
    Rows128Plan pl;
    pl.wv = mp.wv;
    pl.bn = 32 * mp.wv;
    pl.splits = 1;
    pl.tiles = (a.total_tiles + 7) / 8 * 8;  // the kernel numbers its tiles per XCD
    pl.tn = 2;
    switch (mp.mt) {
        case 1: return launch_rowsm_mt<1>(a, pl, st);
        case 2: return launch_rowsm_mt<2>(a, pl, st);
        case 3: return launch_rowsm_mt<3>(a, pl, st);
        case 4: return launch_rowsm_mt<4>(a, pl, st);
        case 5: return launch_rowsm_mt<5>(a, pl, st);
        case 6: return launch_rowsm_mt<6>(a, pl, st);
        case 7: return launch_rowsm_mt<7>(a, pl, st);
        case 8: return launch_rowsm_mt<8>(a, pl, st);
        case 9: return launch_rowsm_mt<9>(a, pl, st);
        case 10: return launch_rowsm_mt<10>(a, pl, st);
        case 11: return launch_rowsm_mt<11>(a, pl, st);
        case 12: return launch_rowsm_mt<12>(a, pl, st);
        case 13: return launch_rowsm_mt<13>(a, pl, st);
        default: return MI355_EINVAL;
    }
}

static bool fast_layout_ok(const void *A, const void *B, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n) {
    return ldb_k == 1 && K % kBlockK == 0 && lda % 16 == 0 && ldb_n % 16 == 0 && ((uintptr_t)A & 15) == 0 &&
           ((uintptr_t)B & 15) == 0;
}

// 256x128 tiles that are too few to occupy the device share the K range the same way.
static int tile256x128_splits(int64_t M, int64_t N, int64_t K, int cus) {
    const int64_t tiles = ((M + 255) / 256) * ((N + 127) / 128);
    const int64_t KB = K / kBlockK;
    if (tiles * 2 > cus || KB < 16) return 1;
    int64_t splits = cus / tiles;
    if (splits > KB / 8) splits = KB / 8;
    return (int)(splits < 1 ? 1 : splits);
}

static size_t tile256x128_workspace(int64_t M, int64_t N, int splits) {
    const int64_t tiles = ((M + 255) / 256) * ((N + 127) / 128);
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)tiles * splits * 256 * 128 * 4;
}

static int64_t n_split_rows(int64_t M, int64_t N, int64_t K, int cus);

// The shape -> kernel table (measured on the DeepSeek-V3 and Llama-3 linears over M = 128..4096):
//   129 <= M <= 384, K >= 2048, at most cus/2 tiles
//     of 128 weight rows (cus if M <= 160; above
//     256 rows only if N*K >= 2e7; 201..256 and
//     337..384 rows on N*K >= 1e8 go to the panel
//     split of stream-K instead)                     the weight stream with the activation block in LDS
//   129 <= M <= 208 (192), 0.55 cus .. cus tiles of
//     160..256 or of 80..112 (64) weight rows         the same, workgroups of that width, K unshared
//   65 <= M <= 128, K >= 2048                        the same with 256 weight rows per workgroup
//   33 <= M <= 64, at most cus tiles, N*K >= 1e8 or
//     (N*K >= 4e7 and the streaming kernel's
//     workgroups neither cus nor 2 cus)              the same, unless the kernel below would run
//   33 <= M <= 128, 0.55 cus .. cus tiles of 160,
//     192 or 256 weight rows with K unshared          the same, workgroups of that width
//   M > 384, N <= 5120 (3072), K <= 5120 (7168), one
//     round of tiles of at most 128 (96) rows         the same kernel tiled over M, K unshared
//   M <= 64                                          weight streaming (M > 32 and N/128 about the unit count: the
//                                                    kernel that shares the activation block in the workgroup)
//   few 256x256 tiles, long K                        stream-K (the plain loop would leave most units idle)
//   128x128 tiles fit one round of two per unit and
//     (few 256x256 tiles or a short K)               128x128 tiles, K shared between workgroups when they are few
//                                                    (M >= 768 and N <= 3072: 256x128 tiles with K shared)
//   otherwise                                        256x256 ping-pong tiles
static int pick_variant(int64_t M, int64_t N, int64_t K, int cus, bool allow_rows128 = true) {
    // up to 16 rows the per-unit stream also beats the stream with the activation block in LDS where both apply
    // (N = 18432, K = 7168, M = 16: 23.6 us against 27.5; N = 7168, K = 18432: 25.4 against 27.2)
    if (streamcu_pays(M, N, K, cus)) return MI355_GEMM_SKINNY_CU;
    if (allow_rows128 && rows128_pays(M, N, K, cus)) return MI355_GEMM_ROWS128;
    if (allow_rows128 && rowsm_pays(M, N, K, cus)) return MI355_GEMM_ROWS_MTILED;
    if (xshare_pays(M, N, K, cus)) return MI355_GEMM_SKINNY_XSHARE;
    if (M <= 64) return MI355_GEMM_SKINNY;
    const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256);
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
    const int64_t KB = K / kBlockK;
    // one or two K steps: the 256x256 tile's first requests and its epilogue are most of its time (N = 7168,
    // K = 256, M = 4096: 21.3 us for the 128x128 tiles against 27.6)
    if (KB <= 2) return MI355_GEMM_TILE128;
    if (M > 128 && stream_k_pays(t256, KB, cus, (M + 255) / 256)) return MI355_GEMM_TILE256_STREAMK;
    // 257..384 rows leave the second 256-row tile at most half full; where the 256x256 tiles need a second round
    // anyway the 128x128 ones are ahead (N = 36864, K = 7168, M = 257 / 384: 144 / 148 us against 161 / 165) -
    // unless the second round is small enough to run as a launch of its own (130 / 139 us then)
    if (M > 256 && M <= 384 && t256 > cus && t128 <= 4 * (int64_t)cus && n_split_rows(M, N, K, cus) == 0)
        return MI355_GEMM_TILE128;
    if (t128 <= 2 * (int64_t)cus && (t256 < (int64_t)cus * 3 / 8 || KB <= 64)) {
        // a narrow N under many rows: 256x128 tiles with K shared load half as much X per product as the 128x128
        // ones and still fill the device (q_a+kv_a, N = 2112, K = 7168, M = 768 / 1024 / 1536: 35.0 / 40.6 / 50.6 us
        // against 38.7 / 60.2 / 60.6; not under 12 n tiles: N = 256 / 512, M = 1024: 17.5 / 17.5 against 20.6 / 21.4)
        // ... and, from two 256-row tiles on, a wider N under a long K (N = 5120, K = 5120, M = 400 / 512: 35.4 /
        // 37.6 us against 44.7 / 45.1; N = 4096, K = 7168, M = 640: 54.6 against 60.3; on N = 1536 the 128x128 tiles
        // keep their lead, 21.8 against 25.2, and with K = 4096 too)
        if (((M >= 768 && (N + 127) / 128 <= 24 && (N + 127) / 128 >= 12) || (M > 384 && KB >= 40 && (N + 127) / 128 >= 20)) &&
            tile256x128_splits(M, N, K, cus) >= 2)
            return MI355_GEMM_TILE256x128;
        return MI355_GEMM_TILE128;
    }
    if (t256 >= (int64_t)cus * 3 / 8) return MI355_GEMM_TILE256;
    return MI355_GEMM_TILE128;
}

// 128x128 tiles that are too few to occupy the device share the K range: about one CTA per CU, at least
// 8 K steps each.
static int tile128_splits(int64_t M, int64_t N, int64_t K, int cus) {
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    const int64_t KB = K / kBlockK;
    if (tiles * 2 > cus || KB < 16) return 1;
    int64_t splits = cus / tiles;
    if (splits > KB / 8) splits = KB / 8;
    return (int)(splits < 1 ? 1 : splits);
}

static size_t tile128_workspace(int64_t M, int64_t N, int splits) {
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return (size_t)MI355_WS_COUNTER_BYTES + (size_t)tiles * splits * 128 * 128 * 4;
}

// A launch of 256x256 tiles that fills the device once and leaves a small rest for a second round runs the rest
// as a launch of its own, with whatever the table gives its shape (mostly 128x128 tiles, which spread it over the
// whole device): N = 36864, K = 7168, M = 512 (288 tiles on 256 units) 137 us against 169; q_b, M = 768, 43.6
// against 50.2.  After two full rounds a rest of up to a quarter round still gains a little (M = 1024, 576 tiles:
// 248 us against 260; q_b, M = 1536: 77.8 against 83.3); with more rounds or a larger rest it gains nothing (3.5
// rounds: 235 against 220).  Returns the number of weight rows of the first launch, 0 for no split.
static int64_t n_split_rows(int64_t M, int64_t N, int64_t K, int cus) {
    (void)K;
    const int64_t tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256, t256 = tiles_m * tiles_n;
    const int64_t rounds = t256 / cus, rest = t256 - rounds * cus;
    if (tiles_m > cus || rounds < 1 || rounds > 2 || rest == 0) return 0;
    if (rest * 2 * rounds > cus) return 0;
    const int64_t n1 = rounds * (int64_t)cus / tiles_m * 256;
    return n1 > 0 && n1 < N ? n1 : 0;
}

// Workspace of a launch plan on a device with `cus` compute units.
static size_t workspace_bytes_for(int64_t M, int64_t N, int64_t K, int32_t variant, int cus) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (K % kBlockK != 0) return 0;
    if (variant == MI355_GEMM_AUTO) {
        variant = pick_variant(M, N, K, cus);
        const int64_t n1 = variant == MI355_GEMM_TILE256 ? n_split_rows(M, N, K, cus) : 0;
        if (n1 > 0) {
            const size_t rest = workspace_bytes_for(M, N - n1, K, MI355_GEMM_AUTO, cus);
            return rest > (size_t)MI355_WS_COUNTER_BYTES ? rest : (size_t)MI355_WS_COUNTER_BYTES;
        }
    }
    if (variant == MI355_GEMM_TILE256_STREAMK) {
        const int groups = stream_k_groups(((M + 255) / 256) * ((N + 255) / 256), K / kBlockK, cus, (M + 255) / 256);
        return groups > 0 ? stream_k_workspace(groups) : (size_t)MI355_WS_COUNTER_BYTES;
    }
    if (variant == MI355_GEMM_TILE128) {
        const int splits = tile128_splits(M, N, K, cus);
        return splits > 1 ? tile128_workspace(M, N, splits) : 0;
    }
    if (variant == MI355_GEMM_TILE256x128) {
        const int splits = tile256x128_splits(M, N, K, cus);
        return splits > 1 ? tile256x128_workspace(M, N, splits) : 0;
    }
    if (variant == MI355_GEMM_TILE256) return MI355_WS_COUNTER_BYTES;  // the tile counters of the persistent launch
    if (variant == MI355_GEMM_SKINNY_XSHARE) {
        const int splits = xshare_splits(N, K, cus);
        return splits > 1 ? xshare_workspace(N, splits) : 0;
    }
    if (variant == MI355_GEMM_ROWS128) {
        if (M > 384) return 0;
        return rows128_workspace(M, N, K, cus);
    }
    if (variant != MI355_GEMM_SKINNY || M > 64) return 0;
    const SkinnyPlan pl = skinny_plan(M, N, K, cus);
    return pl.splits > 1 ? skinny_workspace(M, pl) : 0;
}

// The kernel an AUTO call launches (first) for a problem in the fast layout: the table's choice, or - where a limit
// of that kernel is not met or its workspace is missing - the next kernel with fewer preconditions.  The chain ends
// in tiles that take every fast layout and run unsplit without a workspace, so AUTO never fails for want of one.
// The 256-row stream is checked first because the table's other choice for its shapes can be any of the kernels
// checked after it.
static int resolve_auto(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int64_t as_m, int64_t as_k,
                        bool ws_usable, size_t ws_bytes, int cus) {
    int variant = pick_variant(M, N, K, cus);
    if (variant == MI355_GEMM_ROWS_MTILED && !rowsm_limits_ok(rowsm_plan(M, N, K, cus), M, K, lda, as_m, as_k))
        variant = pick_variant(M, N, K, cus, false);
    if (variant == MI355_GEMM_ROWS128 &&
        (!rows128_limits_ok(M, N, K, lda, as_m, as_k, cus) ||
         (rows128_splits(M, N, K, cus) > 1 && (!ws_usable || ws_bytes < rows128_workspace(M, N, K, cus)))))
        variant = pick_variant(M, N, K, cus, false);
    // stream-K needs its partial-tile slots; without them the plain tile loop gives the same result
    if (variant == MI355_GEMM_TILE256_STREAMK &&
        (!ws_usable || ws_bytes < workspace_bytes_for(M, N, K, variant, cus)))
        variant = MI355_GEMM_TILE256;
    if (variant == MI355_GEMM_SKINNY_XSHARE &&
        (N * ldw >= (1ll << 32) || M * lda >= (1ll << 32) || M * as_m >= (1ll << 32) ||
         (N + XshareCfg::BN - 1) / XshareCfg::BN * 4 > MI355_WS_COUNTER_BYTES))
        variant = MI355_GEMM_TILE128;
    if (variant == MI355_GEMM_SKINNY_CU && streamcu_tnw(M, N, K, lda, ldw, as_m, cus) == 0)
        variant = MI355_GEMM_SKINNY;
    if (variant == MI355_GEMM_SKINNY &&
        skinny_check(M, N, K, lda, ldw, as_m, cus, ws_usable, ws_bytes) != MI355_OK)
        variant = MI355_GEMM_TILE128;
    return variant;
}

}  // namespace mi355

using namespace mi355;

extern "C" size_t mi355_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int32_t variant) {
    // sized from the launch plan of the current device (256 compute units when no device is visible)
    return workspace_bytes_for(M, N, K, variant, device_cus());
}

extern "C" int32_t mi355_block_fp8_gemm_plan(int64_t M, int64_t N, int64_t K, size_t ws_bytes, int32_t cus) {
    if (M <= 0 || N <= 0 || K <= 0 || K % kBlockK != 0) return MI355_GEMM_GENERIC;
    if (cus <= 0) cus = device_cus();
    return resolve_auto(M, N, K, K, K, K / kBlockK, 1, ws_bytes > 0, ws_bytes, cus);
}

/* The kernel the shape table picks for a packed, aligned problem on the current device (256 compute units when no
 * device is visible): one of the MI355_GEMM_* codes.  A launch may still fall back when a limit or the workspace of
 * that kernel is not met. */
extern "C" int32_t mi355_block_fp8_gemm_variant(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % kBlockK != 0) return MI355_GEMM_GENERIC;
    return pick_variant(M, N, K, device_cus());
}

static int block_fp8_gemm_impl(const void *A, const void *B, const float *As, const float *Bs, void *C, int64_t M,
                               int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                               int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n, int32_t block_n,
                               int32_t block_k, void *ws, size_t ws_bytes, int32_t variant, int32_t c_dtype,
                               void *stream) {
    if (M < 0 || N < 0 || K < 0) return MI355_EINVAL;
    if (c_dtype != MI355_DTYPE_BF16 && c_dtype != MI355_DTYPE_F16) return MI355_EUNSUPPORTED;
    const int out_f16 = c_dtype == MI355_DTYPE_F16 ? 1 : 0;
    if (block_n <= 0 || block_k <= 0) return MI355_EINVAL;
    // the tiled kernels are built for 128x128 weight blocks; other block sizes run on the plain kernel
    const bool blocks128 = block_n == kBlockN && block_k == kBlockK;
    if (!blocks128 && variant != MI355_GEMM_AUTO && variant != MI355_GEMM_GENERIC) return MI355_EUNSUPPORTED;
    if (M == 0 || N == 0) return MI355_OK;
    if (K == 0) return MI355_ESHAPE;
    if (!A || !B || !As || !Bs || !C) return MI355_EINVAL;
    if (lda < K || ldc < N) return MI355_ESHAPE;
    if (M >= (1ll << 31) || N >= (1ll << 31) || K >= (1ll << 31)) return MI355_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int cus = device_cus();

    const bool fast = fast_layout_ok(A, B, K, lda, ldb_k, ldb_n) &&
                      // 32-bit byte offsets inside a tile / scale column
                      256 * lda < (1ll << 32) && 256 * ldb_n < (1ll << 32) && 256 * as_m * 4 < (1ll << 32) &&
                      as_m >= 0 && as_k >= 0;
    const bool was_auto = variant == MI355_GEMM_AUTO;
    if (was_auto) {
        const bool ws_usable = ws && ((uintptr_t)ws & 15) == 0;
        variant = fast && blocks128 ? resolve_auto(M, N, K, lda, ldb_n, as_m, as_k, ws_usable, ws_bytes, cus)
                                    : MI355_GEMM_GENERIC;
    }
    if (was_auto && variant == MI355_GEMM_TILE256) {
        const int64_t n1 = n_split_rows(M, N, K, cus);
        if (n1 > 0 && ldb_n * n1 % 16 == 0) {
            const int r = block_fp8_gemm_impl(A, B, As, Bs, C, M, n1, K, lda, ldb_k, ldb_n, ldc, as_m, as_k, bs_k, bs_n,
                                              block_n, block_k, ws, ws_bytes, MI355_GEMM_TILE256, c_dtype, stream);
            if (r != MI355_OK) return r;
            return block_fp8_gemm_impl(A, (const uint8_t *)B + n1 * ldb_n, As, Bs + n1 / kBlockN * bs_n,
                                       (uint16_t *)C + n1, M, N - n1, K, lda, ldb_k, ldb_n, ldc, as_m, as_k, bs_k, bs_n,
                                       block_n, block_k, ws, ws_bytes, MI355_GEMM_AUTO, c_dtype, stream);
        }
    }
    if (variant != MI355_GEMM_GENERIC && !fast) return MI355_EALIGN;

    if (variant == MI355_GEMM_GENERIC) {
        const int64_t blocks = (M * N + 255) / 256;
        if (blocks >= (1ll << 31)) return MI355_EUNSUPPORTED;
        return launch(block_fp8_gemm_generic_kernel, dim3((uint32_t)blocks), dim3(256), 0, st, (const uint8_t *)A,
                      (const uint8_t *)B, As, Bs, (uint16_t *)C, (int)M, (int)N, (int)K, lda, ldb_k, ldb_n, ldc, as_m,
                      as_k, bs_k, bs_n, (int)block_n, (int)block_k, out_f16);
    }

    GemmArgs a = {};
    a.out_f16 = out_f16;
    a.X = (const uint8_t *)A;
    a.W = (const uint8_t *)B;
    a.Xs = As;
    a.Ws = Bs;
    a.C = (uint16_t *)C;
    a.M = (int)M;
    a.N = (int)N;
    a.K = (int)K;
    a.ldx = lda;
    a.ldw = ldb_n;
    a.ldc = ldc;
    a.xs_m = as_m;
    a.xs_k = as_k;
    a.ws_n = bs_n;
    a.ws_k = bs_k;
    a.vec_store = (((uintptr_t)C & 15) == 0 && ldc % 8 == 0 && N % 8 == 0) ? 1 : 0;

    switch (variant) {
        case MI355_GEMM_TILE256_ONCE:  // kept for comparison
            ws = nullptr;
            [[fallthrough]];
        case MI355_GEMM_TILE256:
        case MI355_GEMM_TILE256_STREAMK: {
            a.tiles_m = (a.M + 255) / 256;
            a.tiles_n = (a.N + 255) / 256;
            a.total_tiles = a.tiles_m * a.tiles_n;
            // stream-K when asked for and worth it on this device; the plain tile loop otherwise
            const int groups =
                variant == MI355_GEMM_TILE256_STREAMK ? stream_k_groups(a.total_tiles, a.K / kBlockK, cus, a.tiles_m) : 0;
            const int r = launch_pp<false>(a, ws, ws_bytes, cus, groups, st);
            if (r != MI355_EUNSUPPORTED) return r;
            return launch_dense<256, 256, 2, 4, 2>(a, st);  // K ranges past the ping-pong kernel's LDS layout
        }
        case MI355_GEMM_TILE256_RING:  // kept for comparison
            return launch_dense<256, 256, 2, 4, 2>(a, st);
        case MI355_GEMM_TILE256x128: {
            const int splits = tile256x128_splits(M, N, K, cus);
            if (splits <= 1 || !ws || ws_bytes < tile256x128_workspace(M, N, splits) || ((uintptr_t)ws & 15))
                return launch_dense<256, 128, 2, 4, 3>(a, st);
            a.tiles_m = (a.M + 255) / 256;
            a.tiles_n = (a.N + 127) / 128;
            a.total_tiles = a.tiles_m * a.tiles_n;
            a.splits = splits;
            a.counters = (uint32_t *)ws;
            a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);  // the counter words stay untouched
            const int r = launch_tile<256, 128, 2, 4, 3, kSplitK>(a, a.total_tiles * splits, st);
            if (r != MI355_OK) return r;
            return launch(tile_splitk_reduce_kernel<256, 128, 2, 4>, dim3(a.total_tiles * 16), dim3(512), 0, st, a);
        }
        case MI355_GEMM_TILE128: {
            const int splits = tile128_splits(M, N, K, cus);
            if (splits <= 1 || !ws || ws_bytes < tile128_workspace(M, N, splits) || ((uintptr_t)ws & 15))
                return launch_dense<128, 128, 2, 2, 2>(a, st);  // without a workspace the split is simply not used
            a.tiles_m = (a.M + 127) / 128;
            a.tiles_n = (a.N + 127) / 128;
            a.total_tiles = a.tiles_m * a.tiles_n;
            a.splits = splits;
            a.counters = (uint32_t *)ws;
            a.partials = (float *)((uint8_t *)ws + MI355_WS_COUNTER_BYTES);
            const int r = launch_tile<128, 128, 2, 2, 2, kSplitK>(a, a.total_tiles * splits, st);
            if (r != MI355_OK) return r;
            return launch(tile_splitk_reduce_kernel<128, 128, 2, 2>, dim3(a.total_tiles * 16), dim3(256), 0, st, a);
        }
        case MI355_GEMM_SKINNY_XSHARE: {
            if (M <= 32 || M > 64) return MI355_EUNSUPPORTED;
            if (N * ldb_n >= (1ll << 32) || M * lda >= (1ll << 32) || M * as_m >= (1ll << 32)) return MI355_EUNSUPPORTED;
            if ((N + XshareCfg::BN - 1) / XshareCfg::BN * 4 > MI355_WS_COUNTER_BYTES) return MI355_EUNSUPPORTED;
            int splits = xshare_splits(N, K, cus);
            if (splits > 1 && (!ws || ws_bytes < xshare_workspace(N, splits) || ((uintptr_t)ws & 15))) {
                if (was_auto) splits = 1;  // the table's choice runs unsplit without a workspace
                else return MI355_EWORKSPACE;
            }
            return launch_xshare(a, splits, ws, st);
        }
        case MI355_GEMM_ROWS128: {
            if (!rows128_limits_ok(M, N, K, lda, as_m, as_k, cus)) return MI355_EUNSUPPORTED;
            const Rows128Plan pl = rows128_plan(M, N, K, cus);
            if (pl.splits > 1 && (!ws || ws_bytes < rows128_workspace(M, N, K, cus) || ((uintptr_t)ws & 15)))
                return MI355_EWORKSPACE;
            switch (rows128_mt(M)) {
                case 1: return launch_rows128<1>(a, pl, ws, st);
                case 2: return launch_rows128<2>(a, pl, ws, st);
                case 3: return launch_rows128<3>(a, pl, ws, st);
                case 4: return launch_rows128<4>(a, pl, ws, st);
                case 5: return launch_rows128<5>(a, pl, ws, st);
                case 6: return launch_rows128<6>(a, pl, ws, st);
                case 7: return launch_rows128<7>(a, pl, ws, st);
                case 8: return launch_rows128<8>(a, pl, ws, st);
                case 9: return launch_rows128<9>(a, pl, ws, st);
                case 10: return launch_rows128<10>(a, pl, ws, st);
                case 11: return launch_rows128<11>(a, pl, ws, st);
                case 12: return launch_rows128<12>(a, pl, ws, st);
                case 13: return launch_rows128<13>(a, pl, ws, st);
                case 14: return launch_rows128<14>(a, pl, ws, st);
                case 15: return launch_rows128<15>(a, pl, ws, st);
                case 16: return launch_rows128<16>(a, pl, ws, st);
                case 17: return launch_rows128<17>(a, pl, ws, st);
                case 18: return launch_rows128<18>(a, pl, ws, st);
                case 19: return launch_rows128<19>(a, pl, ws, st);
                case 20: return launch_rows128<20>(a, pl, ws, st);
                case 21: return launch_rows128<21>(a, pl, ws, st);
                case 22: return launch_rows128<22>(a, pl, ws, st);
                case 23: return launch_rows128<23>(a, pl, ws, st);
                default: return launch_rows128<24>(a, pl, ws, st);
            }
        }
        case MI355_GEMM_ROWS_MTILED: {
            const RowsMPlan mp = rowsm_plan(M, N, K, cus);
            if (!rowsm_limits_ok(mp, M, K, lda, as_m, as_k)) return MI355_EUNSUPPORTED;
            return launch_rowsm(a, mp, st);
        }
        case MI355_GEMM_SKINNY_CU: {
            const int tnw = streamcu_tnw(M, N, K, lda, ldb_n, as_m, cus);
            if (tnw == 0) return MI355_EUNSUPPORTED;
            return launch_streamcu(a, tnw, st);
        }
        case MI355_GEMM_SKINNY: {
            const int ok = skinny_check(M, N, K, lda, ldb_n, as_m, cus, ws && ((uintptr_t)ws & 15) == 0, ws_bytes);
            if (ok != MI355_OK) return ok;
            const SkinnyPlan pl = skinny_plan(M, N, K, cus);
            switch (skinny_mt(M)) {
                case 1: return launch_stream_mt<1>(a, pl, ws, st);
                case 2: return launch_stream_mt<2>(a, pl, ws, st);
                default: return launch_stream_mt<4>(a, pl, ws, st);
            }
        }
        default:
            return MI355_EINVAL;
    }
}

extern "C" int mi355_block_fp8_gemm(const void *A, const void *B, const float *As, const float *Bs, void *C,
                                    int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n,
                                    int64_t ldc, int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n,
                                    int32_t block_n, int32_t block_k, void *ws, size_t ws_bytes, int32_t variant,
                                    void *stream) {
    return block_fp8_gemm_impl(A, B, As, Bs, C, M, N, K, lda, ldb_k, ldb_n, ldc, as_m, as_k, bs_k, bs_n, block_n,
                               block_k, ws, ws_bytes, variant, MI355_DTYPE_BF16, stream);
}

extern "C" int mi355_block_fp8_gemm_dtype(const void *A, const void *B, const float *As, const float *Bs, void *C,
                                          int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                                          int64_t ldb_n, int64_t ldc, int64_t as_m, int64_t as_k, int64_t bs_k,
                                          int64_t bs_n, int32_t block_n, int32_t block_k, void *ws, size_t ws_bytes,
                                          int32_t variant, int32_t c_dtype, void *stream) {
    return block_fp8_gemm_impl(A, B, As, Bs, C, M, N, K, lda, ldb_k, ldb_n, ldc, as_m, as_k, bs_k, bs_n, block_n,
                               block_k, ws, ws_bytes, variant, c_dtype, stream);
}

namespace mi355 {

__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t *p, uint32_t n) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace mi355

// ---- the entry point that allocates nothing -------------------------------------------------------------
// Split-K partials, arrival counters and the tile counters of the persistent launch live in a fixed array in
// the library's own device image instead of a caller-owned workspace.  Every GPU holds its own copy of the
// array at its own address; in host code the array's name is only a handle for hipGetSymbolAddress.
namespace mi355 {

constexpr size_t kScratchBytes = (size_t)MI355_WS_COUNTER_BYTES + ((size_t)MI355_NOALLOC_PARTIAL_MIB << 20);
static __device__ __align__(256) uint8_t scratch[kScratchBytes];

// Device address of `scratch` on the current device, looked up on the first call per device.
static void *scratch_ptr() {
    static std::atomic<void *> ptrs[kMaxDevices];
    const int dev = current_device();
    if (dev < 0 || dev >= kMaxDevices) return nullptr;
    void *p = ptrs[dev].load(std::memory_order_acquire);
    if (p) return p;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
    ptrs[dev].store(p, std::memory_order_release);
    return p;
}

}  // namespace mi355

extern "C" int mi355_block_fp8_gemm_noalloc(const void *A, const void *B, const float *As, const float *Bs, void *C,
                                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb_k,
                                            int64_t ldb_n, int64_t ldc, int64_t as_m, int64_t as_k, int64_t bs_k,
                                            int64_t bs_n, int32_t block_n, int32_t block_k, int32_t variant,
                                            void *stream) {
    const size_t need = mi355_block_fp8_gemm_workspace_bytes(M, N, K, variant);
    // a forced kernel that needs more than the array holds is an error; the shape table (MI355_GEMM_AUTO) gets
    // the whole array and takes the next best plan that fits into it
    if (need > kScratchBytes && variant != MI355_GEMM_AUTO) return MI355_ESCRATCH;
    void *ws = nullptr;
    if (need > 0) {
        ws = scratch_ptr();
        if (!ws) return MI355_ELAUNCH;
        // The array keeps what the last call left.  The kernels need their counter words zero and leave them
        // zero, but a launch that was aborted would not have: clear them here (a fill kernel, not a memset node,
        // so that the call can be captured into a HIP graph).
        const uint32_t words = MI355_WS_COUNTER_BYTES / 4;
        const int rc = launch(zero_words_kernel, dim3(words / 256), dim3(256), 0, (hipStream_t)stream, (uint32_t *)ws, words);
        if (rc != MI355_OK) return rc;
    }
    return mi355_block_fp8_gemm(A, B, As, Bs, C, M, N, K, lda, ldb_k, ldb_n, ldc, as_m, as_k, bs_k, bs_n, block_n,
                                block_k, ws, ws ? kScratchBytes : 0, variant, stream);
}

/* Re-zeroes the counter words of a caller-owned workspace (recovery after an aborted launch). */
extern "C" int mi355_reset_workspace(void *ws, size_t ws_bytes, void *stream) {
    if (!ws || ws_bytes < (size_t)MI355_WS_COUNTER_BYTES || ((uintptr_t)ws & 3)) return MI355_EWORKSPACE;
    const uint32_t words = MI355_WS_COUNTER_BYTES / 4;
    return launch(zero_words_kernel, dim3(words / 256), dim3(256), 0, (hipStream_t)stream, (uint32_t *)ws, words);
}

extern "C" int32_t mi355_grouped_block_m(int64_t num_pairs, int32_t num_experts, int64_t N, int64_t K) {
    (void)K;
    if (num_experts <= 0) return 64;
    const int64_t avg = num_pairs / num_experts;
    // 256-row schedule blocks run as the persistent launch with two queues: blocks of more than 64 rows on the
    // 256x256 ping-pong tile (it skips the empty 64-row halves of ragged blocks), the others on the 64x512
    // weight-streaming tile.  That launch needs more tiles than compute units; where it has them it is the faster
    // one from about 12 rows per expert on (256 experts, top-8, N=4096 K=7168: 512 tokens 1275 us against 1291 for
    // 32-row blocks, 1024 tokens 1314 against 1500, 2048 tokens 1421 against 1885; the same within 1 % at 384
    // tokens).  With fewer rows the 16-row tiles stream the weights at 6.0 TB/s and nothing beats them.
    const int cus = device_cus();
    const int64_t tiles256 = (int64_t)num_experts * ((N + 255) / 256);
    const bool two_queues = tiles256 > cus;
    // Measured over Qwen3-MoE (128 experts), DeepSeek-V2-Lite (64), Mixtral (8), a DeepSeek-V3 expert-parallel slice
    // (32 experts, N = 512) and a 16-expert shape, 8 to 8192 tokens, uniform routing:
    //  * 128-row blocks are ahead of the 256-row launch up to a few hundred rows per expert where the whole launch
    //    is small - few tiles (32 experts x N = 512, 128 rows each: 63.9 us against 85.5; Mixtral down, 64 / 128
    //    rows: 128 / 150 against 154 / 163) or under 0.5 GB of weights with a short K (Qwen3-30B down, K = 768,
    //    64 / 128 rows: 60.5 / 89.9 against 81.1 / 105.6; DeepSeek-V2-Lite down, 96 rows: 52.3 against 87.1) -
    //    and behind it on the large ones (DeepSeek-V3, 128 rows: 2189 against 1747)
    if (avg > 32) {
        // (few tiles: from 33 rows per expert where an expert is large and a second block of it costs a second
        // read of its weights, from 65 where it is small - 32 experts x N = 512, 64 rows: 43.6 us for 64-row blocks
        // against 63.0 - and there up to 256 rows: 74.0 against 88.5)
        const bool large_expert = N * K >= 30000000ll;
        if (tiles256 * 2 <= cus && avg > (large_expert ? 32 : 64) && avg <= (large_expert ? 160 : 256)) return 128;
        if ((int64_t)num_experts * N * K <= 500000000ll && K <= 2048 && avg <= (K <= 1536 ? 224 : 112)) return 128;
    }
    //  * with 8 experts every block re-reads a large expert, and 64-row blocks beat blocks of the average size
    //    (Mixtral down, 16 / 32 rows per expert: 84.2 / 86.6 us against 102.5 / 108.9)
    if (num_experts <= 8 && avg > 8 && avg <= 40) return 64;
    //  * the two-queue launch takes over from 12 rows per expert where an expert's N is wide, from 25 where it is
    //    not: the row-sized ring tiles stream small experts better (Qwen3-235B gate_up, N = 3072, 16 rows: 308 us
    //    against 373; DeepSeek-V2-Lite, 12 / 24 rows: 68.3 / 81.7 against 86.1 / 89.0)
    if (avg > 64 || (two_queues && avg >= (N >= 4096 ? 12 : 25))) return 256;
    if (avg <= 16) return 16;
    if (avg <= 32) return 32;
    return 64;
}

extern "C" size_t mi355_grouped_workspace_bytes(int64_t table_rows) {
    return grouped_workspace(table_rows < 0 ? 0 : table_rows);
}

static int grouped_block_fp8_gemm_impl(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                       const int32_t *expert_to_token_index, const float *expert_to_weight,
                                       const int32_t *expert_token_num, const int32_t *table, int64_t table_rows,
                                       int32_t block_m, int64_t num_pairs, int64_t num_tokens, int32_t num_experts,
                                       int32_t topk_num, int64_t N, int64_t K, int32_t mul_routed_weight, void *out,
                                       void *ws, size_t ws_bytes, int32_t out_dtype, const void *bias,
                                       int32_t bias_dtype, int64_t bias_stride_e, void *stream) {
    if (out_dtype != MI355_DTYPE_BF16 && out_dtype != MI355_DTYPE_F16) return MI355_EUNSUPPORTED;
    if (bias && bias_dtype != MI355_DTYPE_BF16 && bias_dtype != MI355_DTYPE_F16 && bias_dtype != MI355_DTYPE_F32)
        return MI355_EUNSUPPORTED;
    if (bias && bias_stride_e < 0) return MI355_EINVAL;
    if (num_pairs < 0 || num_tokens < 0 || num_experts <= 0 || topk_num <= 0 || N < 0 || K < 0 || table_rows < 0)
        return MI355_EINVAL;
    if (num_pairs == 0 || N == 0 || table_rows == 0) return MI355_OK;
    if (!Xq || !Xs || !W || !Ws || !expert_to_token_index || !expert_to_weight || !expert_token_num || !table || !out)
        return MI355_EINVAL;
    if (K == 0 || K % kBlockK != 0) return MI355_ESHAPE;
    if (((uintptr_t)Xq & 15) || ((uintptr_t)W & 15)) return MI355_EALIGN;
    if (num_tokens * K >= (1ll << 32) || 256 * K >= (1ll << 32) || num_tokens * (K / kBlockK) * 4 >= (1ll << 32) ||
        N >= (1ll << 31) || num_pairs >= (1ll << 31))
        return MI355_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const int64_t KB = K / kBlockK, NB = (N + kBlockN - 1) / kBlockN;

    GemmArgs a = {};
    a.out_f16 = out_dtype == MI355_DTYPE_F16 ? 1 : 0;
    a.X = (const uint8_t *)Xq;
    a.W = (const uint8_t *)W;
    a.Xs = Xs;
    a.Ws = Ws;
    a.C = (uint16_t *)out;
    a.M = (int)num_pairs;
    a.N = (int)N;
    a.K = (int)K;
    a.ldx = K;
    a.ldw = K;
    a.ldc = N;
    a.xs_m = KB;
    a.xs_k = 1;
    a.ws_n = KB;
    a.ws_k = 1;
    a.vec_store = (((uintptr_t)out & 15) == 0 && N % 8 == 0) ? 1 : 0;
    a.table = table;
    a.e2t_index = expert_to_token_index;
    a.e2t_weight = expert_to_weight;
    a.e_num = expert_token_num;
    a.w_e = N * K;
    a.ws_e = NB * KB;
    a.num_pairs = (int)num_pairs;
    a.topk = topk_num;
    a.mul_weight = mul_routed_weight ? 1 : 0;
    a.bias = bias;
    a.bias_e = bias_stride_e;
    a.bias_dtype = bias_dtype;
    a.tiles_m = (int)table_rows;

    auto finish = [&](int BN) {
        a.tiles_n = (int)((N + BN - 1) / BN);
        a.total_tiles = a.tiles_m * a.tiles_n;
        a.blocks_per_xcd = (a.total_tiles + 7) / 8;
        return a.blocks_per_xcd * 8;
    };
    if ((int64_t)table_rows * ((N + 127) / 128) >= (1ll << 31)) return MI355_EUNSUPPORTED;
    switch (block_m) {
        case 16: return launch_grouped_tile<16, 128, 1, 4, 4>(a, finish(128), st);
        case 32: return launch_grouped_tile<32, 128, 1, 4, 4>(a, finish(128), st);
        case 64: return launch_grouped_tile<64, 128, 1, 4, 4>(a, finish(128), st);
        case 128: return launch_grouped_tile<128, 128, 2, 2, 2>(a, finish(128), st);
        case 256:
            finish(256);
            return launch_grouped_pp(a, ws, ws_bytes, device_cus(), st);
        default: return MI355_EINVAL;
    }
}

extern "C" int mi355_grouped_block_fp8_gemm(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                            const int32_t *expert_to_token_index, const float *expert_to_weight,
                                            const int32_t *expert_token_num, const int32_t *table,
                                            int64_t table_rows, int32_t block_m, int64_t num_pairs,
                                            int64_t num_tokens, int32_t num_experts, int32_t topk_num, int64_t N,
                                            int64_t K, int32_t mul_routed_weight, void *out, void *ws,
                                            size_t ws_bytes, void *stream) {
    return grouped_block_fp8_gemm_impl(Xq, Xs, W, Ws, expert_to_token_index, expert_to_weight, expert_token_num, table,
                                       table_rows, block_m, num_pairs, num_tokens, num_experts, topk_num, N, K,
                                       mul_routed_weight, out, ws, ws_bytes, MI355_DTYPE_BF16, nullptr, 0, 0, stream);
}

extern "C" int mi355_grouped_block_fp8_gemm_dtype(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                                  const int32_t *expert_to_token_index,
                                                  const float *expert_to_weight, const int32_t *expert_token_num,
                                                  const int32_t *table, int64_t table_rows, int32_t block_m,
                                                  int64_t num_pairs, int64_t num_tokens, int32_t num_experts,
                                                  int32_t topk_num, int64_t N, int64_t K, int32_t mul_routed_weight,
                                                  void *out, void *ws, size_t ws_bytes, int32_t out_dtype,
                                                  void *stream) {
    return grouped_block_fp8_gemm_impl(Xq, Xs, W, Ws, expert_to_token_index, expert_to_weight, expert_token_num, table,
                                       table_rows, block_m, num_pairs, num_tokens, num_experts, topk_num, N, K,
                                       mul_routed_weight, out, ws, ws_bytes, out_dtype, nullptr, 0, 0, stream);
}

extern "C" int mi355_grouped_block_fp8_gemm_bias(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                                 const int32_t *expert_to_token_index, const float *expert_to_weight,
                                                 const int32_t *expert_token_num, const int32_t *table,
                                                 int64_t table_rows, int32_t block_m, int64_t num_pairs,
                                                 int64_t num_tokens, int32_t num_experts, int32_t topk_num, int64_t N,
                                                 int64_t K, int32_t mul_routed_weight, void *out, void *ws,
                                                 size_t ws_bytes, int32_t out_dtype, const void *bias,
                                                 int32_t bias_dtype, int64_t bias_stride_e, void *stream) {
    return grouped_block_fp8_gemm_impl(Xq, Xs, W, Ws, expert_to_token_index, expert_to_weight, expert_token_num, table,
                                       table_rows, block_m, num_pairs, num_tokens, num_experts, topk_num, N, K,
                                       mul_routed_weight, out, ws, ws_bytes, out_dtype, bias, bias_dtype,
                                       bias_stride_e, stream);
}

// Routing tables for the grouped GEMM: bucket (token, slot) pairs by expert, then expand the per-expert
// counts into the schedule of m-blocks.  Integer work, one workgroup per expert.
#include "common.hpp"

namespace mi355 {

// moe_align: out[e, j] = 1 where pair j is routed to expert e, else 0 (every element of the [E, pairs] table is
// written, so the caller's zero fill is part of the kernel).
__global__ __launch_bounds__(256) void moe_align_mask_kernel(const int32_t *__restrict__ topk_ids, int32_t num_pairs,
                                                             int32_t *__restrict__ out, int64_t out_stride_m) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= num_pairs) return;
    out[(int64_t)blockIdx.y * out_stride_m + j] = topk_ids[j] == (int32_t)blockIdx.y ? 1 : 0;
}

// One workgroup (1024 threads) per expert scans all pairs in order, 4 pairs per thread per step, and
// compacts the indices of the pairs routed to its expert: ascending pair index for every input size.
// FROM_MASK = false (moe_align_fused): pair j belongs to the expert when topk_ids[j] == expert.
// FROM_MASK = true  (moe_align1): when the expert's row of the 0/1 table holds 1 at j; the row is compacted in
// place (a pair's index lands at or before its own position, and a step reads its 4096 entries before it
// writes), entries past the count keep what they held.
template <bool FROM_MASK>
__global__ __launch_bounds__(1024) void moe_align_fused_kernel(const int32_t *__restrict__ topk_ids,
                                                               const float *__restrict__ topk_weights,
                                                               int32_t num_pairs, int32_t *e2t_index,
                                                               int64_t index_stride_m, float *__restrict__ e2t_weight,
                                                               int64_t weight_stride_m, int32_t *__restrict__ e_num) {
    __shared__ int wave_cnt[16];
    const int expert = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int32_t *out_i = e2t_index + (int64_t)expert * index_stride_m;
    float *out_w = e2t_weight + (int64_t)expert * weight_stride_m;
    const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    int base = 0;
    for (int start = 0; start < num_pairs; start += 4096) {
        const int p0 = start + tid * 4;
        bool hit[4];
        uint64_t bal[4];
        int before = 0, total = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (FROM_MASK) hit[j] = p0 + j < num_pairs && out_i[p0 + j] == 1;
            else hit[j] = p0 + j < num_pairs && topk_ids[p0 + j] == expert;
            bal[j] = __ballot(hit[j]);
            before += __popcll(bal[j] & lt);
            total += __popcll(bal[j]);
        }
        if (lane == 0) wave_cnt[wave] = total;
        __syncthreads();
        int pos = base + before;
        int all = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int c = wave_cnt[w];
            if (w < wave) pos += c;
            all += c;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (hit[j]) {
                out_i[pos] = p0 + j;
                out_w[pos] = topk_weights[p0 + j];
                ++pos;
            }
        base += all;
        __syncthreads();
    }
    if (tid == 0) e_num[expert] = base;
}

// One workgroup per expert: exclusive prefix sums of token counts and of block counts over the experts
// before it, then one table row per block.  The last expert also marks the padding rows.
__global__ __launch_bounds__(256) void moe_align2_kernel(const int32_t *__restrict__ e_num, int32_t num_experts,
                                                         int32_t block_m, int64_t rows, int32_t *__restrict__ table) {
    __shared__ int red_t[4], red_b[4];
    const int expert = blockIdx.x, tid = threadIdx.x;
    int tok = 0, blk = 0;
    for (int e = tid; e < expert; e += 256) {
        const int c = e_num[e];
        tok += c;
        blk += (c + block_m - 1) / block_m;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        tok += __shfl_xor(tok, off);
        blk += __shfl_xor(blk, off);
    }
    if ((tid & 63) == 0) {
        red_t[tid >> 6] = tok;
        red_b[tid >> 6] = blk;
    }
    __syncthreads();
    const int token_start = red_t[0] + red_t[1] + red_t[2] + red_t[3];
    const int block_start = red_b[0] + red_b[1] + red_b[2] + red_b[3];
    const int cnt = e_num[expert];
    const int nblk = (cnt + block_m - 1) / block_m;
    for (int b = tid; b < nblk; b += 256) {
        const int64_t r = (int64_t)block_start + b;
        if (r < rows) {
            table[r * 4 + 0] = expert;
            table[r * 4 + 1] = b;
            table[r * 4 + 2] = token_start + b * block_m;
            table[r * 4 + 3] = min(cnt - b * block_m, block_m);
        }
    }
    if (expert == num_experts - 1)
        for (int64_t r = (int64_t)block_start + nblk + tid; r < rows; r += 256) table[r * 4 + 0] = -1;
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_moe_align_fused(const int32_t *topk_ids, const float *topk_weights, int64_t num_pairs,
                                     int32_t num_experts, int32_t *expert_to_token_index, float *expert_to_weight,
                                     int32_t *expert_token_num, void *stream) {
    if (num_pairs < 0 || num_experts <= 0) return MI355_EINVAL;
    if (num_pairs >= (1ll << 31) - 8192) return MI355_EUNSUPPORTED;
    if (!expert_token_num || (num_pairs > 0 && (!topk_ids || !topk_weights || !expert_to_token_index || !expert_to_weight)))
        return MI355_EINVAL;
    return launch(moe_align_fused_kernel<false>, dim3((uint32_t)num_experts), dim3(1024), 0, (hipStream_t)stream,
                  topk_ids, topk_weights, (int32_t)num_pairs, expert_to_token_index, num_pairs, expert_to_weight,
                  num_pairs, expert_token_num);
}

extern "C" int mi355_moe_align(const int32_t *topk_ids, int64_t num_pairs, int32_t num_experts, int32_t *out,
                               int64_t out_stride_m, void *stream) {
    if (num_pairs < 0 || num_experts <= 0 || num_experts > 65535) return MI355_EINVAL;
    if (num_pairs >= (1ll << 31) - 8192) return MI355_EUNSUPPORTED;
    if (num_pairs == 0) return MI355_OK;
    if (!topk_ids || !out) return MI355_EINVAL;
    if (out_stride_m < num_pairs) return MI355_ESHAPE;
    return launch(moe_align_mask_kernel, dim3((uint32_t)((num_pairs + 255) / 256), (uint32_t)num_experts), dim3(256), 0,
                  (hipStream_t)stream, topk_ids, (int32_t)num_pairs, out, out_stride_m);
}

extern "C" int mi355_moe_align1(int32_t *experts_info, int64_t info_stride_m, const float *topk_weights,
                                int64_t num_pairs, int32_t num_experts, float *experts_weight_info,
                                int64_t weight_stride_m, int32_t *expert_token_num, void *stream) {
    if (num_pairs < 0 || num_experts <= 0) return MI355_EINVAL;
    if (num_pairs >= (1ll << 31) - 8192) return MI355_EUNSUPPORTED;
    if (!expert_token_num || (num_pairs > 0 && (!experts_info || !topk_weights || !experts_weight_info)))
        return MI355_EINVAL;
    if (info_stride_m < num_pairs || weight_stride_m < num_pairs) return MI355_ESHAPE;
    return launch(moe_align_fused_kernel<true>, dim3((uint32_t)num_experts), dim3(1024), 0, (hipStream_t)stream,
                  (const int32_t *)nullptr, topk_weights, (int32_t)num_pairs, experts_info, info_stride_m,
                  experts_weight_info, weight_stride_m, expert_token_num);
}

extern "C" int64_t mi355_moe_align2_rows(int64_t num_pairs, int32_t num_experts, int32_t block_m) {
    if (num_pairs <= 0 || num_experts <= 0 || block_m <= 0) return 0;
    const int64_t padded = num_pairs + (int64_t)num_experts * (block_m - 1);
    const int64_t blocks = (padded + block_m - 1) / block_m;
    return blocks < num_pairs ? blocks : num_pairs;
}

extern "C" int mi355_moe_align2(const int32_t *expert_token_num, int32_t num_experts, int32_t block_m, int64_t rows,
                                int32_t *table, void *stream) {
    if (num_experts <= 0 || block_m <= 0 || rows < 0) return MI355_EINVAL;
    if (rows == 0) return MI355_OK;
    if (!expert_token_num || !table) return MI355_EINVAL;
    return launch(moe_align2_kernel, dim3((uint32_t)num_experts), dim3(256), 0, (hipStream_t)stream,
                       expert_token_num, num_experts, block_m, rows, table);
}

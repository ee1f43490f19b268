// Routing tables for the grouped GEMM: bucket (token, slot) pairs by expert, then expand the per-expert
// counts into the schedule of m-blocks.  Integer work, one workgroup per expert.
#include "common.hpp"

namespace mi355 {

// One workgroup (1024 threads) per expert scans all pairs in order, 4 pairs per thread per step, and
// compacts the indices of the pairs routed to its expert: ascending pair index for every input size.
__global__ __launch_bounds__(1024) void moe_align_fused_kernel(const int32_t *__restrict__ topk_ids,
                                                               const float *__restrict__ topk_weights,
                                                               int32_t num_pairs, int32_t *__restrict__ e2t_index,
                                                               float *__restrict__ e2t_weight,
                                                               int32_t *__restrict__ e_num) {
    __shared__ int wave_cnt[16];
    const int expert = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int32_t *out_i = e2t_index + (int64_t)expert * num_pairs;
    float *out_w = e2t_weight + (int64_t)expert * num_pairs;
    const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    int base = 0;
    for (int start = 0; start < num_pairs; start += 4096) {
        const int p0 = start + tid * 4;
        bool hit[4];
        uint64_t bal[4];
        int before = 0, total = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            hit[j] = p0 + j < num_pairs && topk_ids[p0 + j] == expert;
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
    hipLaunchKernelGGL(moe_align_fused_kernel, dim3((uint32_t)num_experts), dim3(1024), 0, (hipStream_t)stream, topk_ids,
                       topk_weights, (int32_t)num_pairs, expert_to_token_index, expert_to_weight, expert_token_num);
    return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ELAUNCH;
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
    hipLaunchKernelGGL(moe_align2_kernel, dim3((uint32_t)num_experts), dim3(256), 0, (hipStream_t)stream,
                       expert_token_num, num_experts, block_m, rows, table);
    return hipGetLastError() == hipSuccess ? MI355_OK : MI355_ELAUNCH;
}

/*
 * mi355_fp8.h - C ABI of libmi355fp8.so: hand-written gfx950 (MI355X) kernels for
 * LightLLM's block-FP8 W8A8 linear path.
 *
 * Plain C: pointers are device pointers unless a comment says "host"; sizes and
 * strides are in ELEMENTS of the tensor they describe; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  No entry point allocates or
 * frees device memory, synchronises the host with the device, or keeps mutable
 * global state, so all of them may be called under HIP graph capture and from
 * several host threads at once.  Workspaces are caller-owned.
 *
 * Every function returns 0 on success or a negative MI355_E* code; nothing is
 * launched when a precondition fails.  mi355_error_string() names the code.
 *
 * Paths in the citations are relative to the reference tree (LightLLM v1.2.0).
 */
#ifndef MI355_FP8_H
#define MI355_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_OK 0
#define MI355_EINVAL -1        /* a size or enum argument is out of range */
#define MI355_ESHAPE -2        /* shapes/strides break a precondition the reference asserts */
#define MI355_EALIGN -3        /* a pointer or leading dimension is not aligned as the kernel needs */
#define MI355_EWORKSPACE -4    /* workspace missing or smaller than *_workspace_bytes() */
#define MI355_ELAUNCH -5       /* the HIP runtime refused the launch (hipLaunchKernel / hipFuncSetAttribute failed) */
#define MI355_EUNSUPPORTED -6  /* valid request that no kernel variant covers */
#define MI355_ESCRATCH -7      /* mi355_block_fp8_gemm_noalloc: the launch needs more scratch than the library holds */

const char *mi355_error_string(int code);

/* Device facts the host side sizes launches and rooflines with.
 * out[0]=compute units, out[1]=max engine clock kHz, out[2]=LDS bytes per workgroup (opt-in max),
 * out[3]=L2 bytes, out[4]=memory clock kHz, out[5]=memory bus width bits, out[6]=1 if the device is gfx950.
 * `device` < 0 means the current device. */
int mi355_device_info(int device, int64_t out[8]);

/* ---------------------------------------------------------------------------
 * per_token_group_quant_fp8
 * replaces: lightllm_per_token_group_quant_fp8 + _per_token_group_quant_fp8
 *           (lightllm/common/basemodel/triton_kernel/quantization/fp8act_quant_kernel.py:18-113)
 *
 * x  [M,K] contiguous (asserted there at :81); `x_dtype` MI355_DTYPE_BF16 (the hot path), _F32 or _F16:
 *    the reference widens whatever it gets to fp32 first (:52)
 * q  e4m3fn bytes [M,K] contiguous
 * s  fp32, element (m,g) at s[m*s_stride_m + g*s_stride_g], g < K/group
 *    row-major (K/group, 1) and column-major (1, ld) are both what the reference
 *    writes (:37-42); any pair of strides is accepted.
 * group must divide K (:80): 128 is the hot path (16-byte aligned x, 8-byte aligned q), any other size - the whole
 * row for a per-token scale, as the reference's other callers use it - takes a general kernel; eps is the floor on
 * the group amax (:55).
 * Arithmetic: s = max(amax,eps)/448 and q = e4m3fn_rtne(clamp(x/s,+-448)) with
 * IEEE fp32 division results, bit for bit.
 * A group that holds a NaN or an infinity (undefined in the reference) gets s = NaN and every byte 0x7F with
 * the sign bit of its element.
 */
#define MI355_DTYPE_BF16 0
#define MI355_DTYPE_F32 1
#define MI355_DTYPE_F16 2
int mi355_group_quant_fp8(const void *x, int32_t x_dtype, void *q, float *s, int64_t M, int64_t K, int32_t group,
                          float eps, int64_t s_stride_m, int64_t s_stride_g, void *stream);

/* ---------------------------------------------------------------------------
 * weight_quant (load-time 128x128 block quantizer)
 * replaces: mm_weight_quant / weight_quant_kernel
 *           (.../quantization/fp8w8a8_block_quant_kernel.py:7-42)
 *
 * w bf16 [N,K] contiguous; q e4m3fn [N,K]; s fp32 [ceil(N/128), ceil(K/128)] contiguous.
 * Keeps the reference's quirk: the stored scale is amax/448 while values are
 * divided by (scale + 1e-6), without clamp (:22-24).  `w_dtype`: MI355_DTYPE_BF16 / _F32 / _F16.
 */
int mi355_block_weight_quant_fp8(const void *w, int32_t w_dtype, void *q, float *s, int64_t N, int64_t K,
                                 int32_t block, void *stream);

/* ---------------------------------------------------------------------------
 * w8a8_block_fp8_matmul
 * replaces: w8a8_block_fp8_matmul + _block_scaled_block_gemm
 *           (.../quantization/fp8w8a8_block_gemm_kernel.py:24-84, 127-192)
 *
 * C[m,n] = bf16( sum_kb ( sum_{k in kb} A[m,k]*B[k,n] ) * As[m,kb] * Bs[kb, n/block_n] ), fp32 accumulation.
 *
 * A   e4m3fn [M,K], row stride lda, unit column stride (the reference asserts A contiguous, :152)
 * B   e4m3fn logical [K,N]: element (k,n) at B[k*ldb_k + n*ldb_n].  The reference passes the
 *     transposed view of an [N,K] weight, i.e. ldb_k = 1, ldb_n = K (common/quantization/w8a8.py:442);
 *     that layout takes the MFMA kernels, any other pair of strides takes a slow generic kernel.
 * As  fp32 [M, K/block_k]   element (m,kb) at As[m*as_m + kb*as_k]
 * Bs  fp32 [K/block_k, ceil(N/block_n)] element (kb,nb) at Bs[kb*bs_k + nb*bs_n]   (w8a8.py:443: strides (1, K/128))
 * C   bf16 [M,N], row stride ldc, unit column stride (:152)
 * block_n = block_k = 128 for the tiled kernels; any other positive block sizes run on the plain kernel
 * (MI355_GEMM_AUTO or MI355_GEMM_GENERIC), the last K block may be partial.
 *
 * `variant` picks the kernel: MI355_GEMM_AUTO applies the built-in shape table (and falls back, kernel by kernel,
 * to one that runs when a limit of the chosen kernel - 32-bit row offsets, LDS, workspace - is not met: it never
 * fails for want of a workspace, see mi355_block_fp8_gemm_plan); the
 * others force one (for tests and tuning) and report such a limit as an error.  Split-K variants need `ws` of at least
 * mi355_block_fp8_gemm_workspace_bytes() bytes, whose first MI355_WS_COUNTER_BYTES must be zero
 * on the first call; the kernels leave them zero again, so one zero-initialised buffer serves every call
 * issued in order on one stream.  MI355_GEMM_TILE256 uses only those counter bytes and only if it gets them:
 * with them the launch is persistent (one workgroup per compute unit takes tiles from per-XCD counters and
 * overlaps the first requests of a tile with the stores of the previous one), without them (ws = NULL) every
 * tile gets its own workgroup; same results.
 */
#define MI355_GEMM_AUTO 0
#define MI355_GEMM_TILE256 1     /* 256x256x128 CTA tile, 8 waves, LDS double buffer: compute-bound M */
#define MI355_GEMM_TILE128 2     /* 128x128x128 CTA tile, 4 waves: mid M or few tiles */
#define MI355_GEMM_SKINNY 3      /* weight-streaming split-K, M <= 64 */
#define MI355_GEMM_GENERIC 4     /* any strides, no MFMA; correctness fallback */
#define MI355_GEMM_TILE256x128 5 /* 256x128x128 CTA tile, 8 waves */
#define MI355_GEMM_TILE256_RING 6 /* the 256x256 tile on the plain ring pipeline (comparison / any scale layout) */
#define MI355_GEMM_TILE256_ONCE 7 /* MI355_GEMM_TILE256 with one workgroup per tile even when a workspace is given */
#define MI355_GEMM_TILE256_STREAMK 8 /* the 256x256 tile with the K steps of all tiles shared evenly between the
                                        compute units (partial tiles added up through the workspace, in K order:
                                        deterministic); falls back to MI355_GEMM_TILE256 where sharing gains nothing */

#define MI355_GEMM_SKINNY_XSHARE 9 /* weight streaming, M <= 64, the activation block of a K step shared by the workgroup */
#define MI355_GEMM_ROWS128 10 /* weight streaming, M <= 384, the activation block of a K step in LDS: 256 weight rows per
                                 workgroup up to 128 rows, 128 beyond; a second launch adds the partial sums when K is shared */

#define MI355_GEMM_SKINNY_CU 11 /* weight streaming, M <= 16: the weight rows cut into one equal share per compute unit,
                                  one workgroup of 8 waves per share and the whole K (no partial sums between
                                  workgroups); where N / 16 gives the units 1..8 row blocks each */

#define MI355_GEMM_ROWS_MTILED 12 /* the kernel of MI355_GEMM_ROWS128 tiled over M as well: one round of tiles of
                                     16..128 rows x 160..256 weight rows, K unshared, no workspace; for more than 384
                                     rows on a narrow N (at most 5120 weight rows, K <= 7168) */

#define MI355_WS_COUNTER_BYTES 65536

/* The kernel MI355_GEMM_AUTO picks for a packed, 16-byte aligned problem of this shape on the CURRENT device (one of
 * the codes above; MI355_GEMM_GENERIC when K is not a multiple of 128).  No counterpart in the reference, whose
 * autotuner picks tile sizes at run time (fp8w8a8_block_gemm_kernel.py:120-146); for logs and tests. */
int32_t mi355_block_fp8_gemm_variant(int64_t M, int64_t N, int64_t K);

/* The kernel an MI355_GEMM_AUTO call launches (first) for a packed, 16-byte aligned problem when it is handed a
 * workspace of `ws_bytes` bytes (0 = none), on a device with `cus` compute units (<= 0: the current device): the
 * table's choice, or the kernel it falls back to where that choice's workspace is missing - the chain always ends in
 * a kernel that runs without one, so AUTO never returns MI355_EWORKSPACE.  Launches nothing.  No counterpart in the
 * reference; for tests of the table off the device it was measured on, and for callers that size workspaces. */
int32_t mi355_block_fp8_gemm_plan(int64_t M, int64_t N, int64_t K, size_t ws_bytes, int32_t cus);

/* Bytes of workspace the launch plan of the CURRENT device needs for this shape and variant (0 = none). */
size_t mi355_block_fp8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int32_t variant);

/* mi355_block_fp8_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and results as
 * mi355_block_fp8_gemm without the workspace pair: split-K partials and counters go to a fixed array inside the
 * library's device image, MI355_WS_COUNTER_BYTES + MI355_NOALLOC_PARTIAL_MIB MiB per GPU, held from the first call
 * on that GPU until the process ends.  A forced variant whose launch plan needs more returns MI355_ESCRATCH and
 * launches nothing (mi355_block_fp8_gemm_workspace_bytes() tells the need); under MI355_GEMM_AUTO the shape table
 * falls back to the best plan that fits (fewer or no K splits).  The call allocates and frees nothing; it clears the
 * counter words with a small fill kernel first.  All calls on one GPU share the array: calls that may overlap on
 * one GPU (different streams, concurrently replayed graphs) race - use mi355_block_fp8_gemm with one workspace per
 * stream there. */
#define MI355_NOALLOC_PARTIAL_MIB 8
int mi355_block_fp8_gemm_noalloc(const void *A, const void *B, const float *As, const float *Bs, void *C, int64_t M,
                                 int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                                 int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n, int32_t block_n,
                                 int32_t block_k, int32_t variant, void *stream);

/* Re-zeroes the MI355_WS_COUNTER_BYTES counter bytes of a workspace (a small fill kernel on `stream`).  The
 * kernels leave the counters zero themselves; this is the recovery path after a launch that was aborted, or
 * after two launches were wrongly run at the same time on one workspace.  No counterpart in the reference. */
int mi355_reset_workspace(void *ws, size_t ws_bytes, void *stream);

int mi355_block_fp8_gemm(const void *A, const void *B, const float *As, const float *Bs, void *C, int64_t M,
                         int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                         int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n, int32_t block_n,
                         int32_t block_k, void *ws, size_t ws_bytes, int32_t variant, void *stream);
/* The same with the dtype of C stated: MI355_DTYPE_BF16 or MI355_DTYPE_F16 (the reference casts the accumulator to
 * whatever C holds, fp8w8a8_block_gemm_kernel.py:78; LightLLM allocates C in the activations' dtype, w8a8.py:515). */
int mi355_block_fp8_gemm_dtype(const void *A, const void *B, const float *As, const float *Bs, void *C, int64_t M,
                               int64_t N, int64_t K, int64_t lda, int64_t ldb_k, int64_t ldb_n, int64_t ldc,
                               int64_t as_m, int64_t as_k, int64_t bs_k, int64_t bs_n, int32_t block_n,
                               int32_t block_k, void *workspace, size_t workspace_bytes, int32_t variant,
                               int32_t c_dtype, void *stream);

/* ---------------------------------------------------------------------------
 * moe_align_fused / moe_align2 : routing tables for the grouped GEMM
 * replaces: moe_align_fused (lightllm/common/basemodel/triton_kernel/fused_moe/grouped_fused_moe.py:388-396)
 *           moe_align2      (same file :399-477)
 *
 * topk_ids int32 [num_pairs] (flattened [tokens, topk]); topk_weights fp32 [num_pairs];
 * expert_to_token_index int32 [E, num_pairs]; expert_to_weight fp32 [E, num_pairs]; expert_token_num int32 [E].
 * Within an expert, pair indices come out in ascending order for every size (the reference only
 * guarantees that below 129 tokens, :391-395).
 */
int mi355_moe_align_fused(const int32_t *topk_ids, const float *topk_weights, int64_t num_pairs,
                          int32_t num_experts, int32_t *expert_to_token_index, float *expert_to_weight,
                          int32_t *expert_token_num, void *stream);

/* The two-step form of the same tables.
 * moe_align  (grouped_fused_moe.py:39-98):   out int32 [E, num_pairs] (row stride out_stride_m), out[e, j] = 1 if
 *            topk_ids[j] == e else 0; every element is written (the reference zero-fills first, :86).
 * moe_align1 (grouped_fused_moe.py:101-214): compacts each row of that 0/1 table IN PLACE into the ascending pair
 *            indices of its ones and writes the matching weights and the per-expert counts; entries past an
 *            expert's count keep what they held. */
int mi355_moe_align(const int32_t *topk_ids, int64_t num_pairs, int32_t num_experts, int32_t *out,
                    int64_t out_stride_m, void *stream);
int mi355_moe_align1(int32_t *experts_info, int64_t info_stride_m, const float *topk_weights, int64_t num_pairs,
                     int32_t num_experts, float *experts_weight_info, int64_t weight_stride_m,
                     int32_t *expert_token_num, void *stream);

/* rows of the schedule table: min(num_pairs, ceil((num_pairs + E*(block_m-1)) / block_m))  (:457-458) */
int64_t mi355_moe_align2_rows(int64_t num_pairs, int32_t num_experts, int32_t block_m);

/* table int32 [rows,4] = (expert, m_index, token_start, tokens in the block); padding rows get expert = -1
 * (:439-446; the fourth column is derived, min(block_m, count - m_index*block_m), so that a GEMM tile needs one
 * 16-byte load to know its work). */
int mi355_moe_align2(const int32_t *expert_token_num, int32_t num_experts, int32_t block_m, int64_t rows,
                     int32_t *table, void *stream);

/* ---------------------------------------------------------------------------
 * grouped_matmul, fp8 128x128-block branch
 * replaces: grouped_matmul_kernel + the launch in grouped_matmul
 *           (.../fused_moe/grouped_fused_moe.py:480-728, 925-988), gather/scatter form
 *
 * For each schedule row (e, mi, start) and j in [mi*block_m, min((mi+1)*block_m, expert_token_num[e])):
 *     idx = expert_to_token_index[e*num_pairs + j];  row = idx / topk_num
 *     out[idx, :] = bf16( blockscaled(Xq[row,:] . W[e]^T) * (mul_routed_weight ? expert_to_weight[e*num_pairs+j] : 1) )
 * Xq e4m3fn [T,K] contiguous, Xs fp32 [T,K/128] contiguous (the activation quantizer's output);
 * W e4m3fn [E,N,K] contiguous; Ws fp32 [E, ceil(N/128), K/128] contiguous; out bf16 [num_pairs, N] contiguous.
 * num_pairs is only used as the row stride of expert_to_token_index / expert_to_weight (the number of (token, slot)
 * pairs in LightLLM's use); the masked expert-parallel layout passes a [E, T_pad] table with num_pairs = T_pad.
 * block_m must be one the library was built for: 16, 32, 64, 128 or 256; mi355_grouped_block_m() suggests one
 * from the rows per expert, the number of experts and an expert's N and K (256 also for batches of 12 to 64 rows
 * per expert when the launch has more tiles than compute units: that suggestion counts on the workspace of
 * mi355_grouped_workspace_bytes(), see below; 128 for small launches; 64 for models of 8 experts).
 * workspace: optional, used by block_m = 256 only: MI355_WS_COUNTER_BYTES bytes that are zero before the launch
 * (the kernel leaves them zero).  With it the launch is persistent - one workgroup per compute unit takes tiles
 * from per-XCD counters and overlaps the first requests of a tile with the stores of the previous one;
 * without it (NULL) every tile gets its own workgroup, same results.  With mi355_grouped_workspace_bytes(table_rows)
 * bytes the persistent launch also sorts the schedule rows by size and runs the blocks of at most 64 rows on a
 * 64x512 weight-streaming tile (same results; the bytes behind the counters are scratch and need no clearing).
 * Launches that may run concurrently need separate workspaces.
 */
int32_t mi355_grouped_block_m(int64_t num_pairs, int32_t num_experts, int64_t N, int64_t K);
size_t mi355_grouped_workspace_bytes(int64_t table_rows);

int mi355_grouped_block_fp8_gemm(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                 const int32_t *expert_to_token_index, const float *expert_to_weight,
                                 const int32_t *expert_token_num, const int32_t *table, int64_t table_rows,
                                 int32_t block_m, int64_t num_pairs, int64_t num_tokens, int32_t num_experts,
                                 int32_t topk_num, int64_t N, int64_t K, int32_t mul_routed_weight, void *out,
                                 void *workspace, size_t workspace_bytes, void *stream);
/* The same with the dtype of `out` stated (MI355_DTYPE_BF16 or MI355_DTYPE_F16; `accumulator.to(compute_type)`,
 * grouped_fused_moe.py:717). */
int mi355_grouped_block_fp8_gemm_dtype(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                       const int32_t *expert_to_token_index, const float *expert_to_weight,
                                       const int32_t *expert_token_num, const int32_t *table, int64_t table_rows,
                                       int32_t block_m, int64_t num_pairs, int64_t num_tokens, int32_t num_experts,
                                       int32_t topk_num, int64_t N, int64_t K, int32_t mul_routed_weight, void *out,
                                       void *ws, size_t ws_bytes, int32_t out_dtype, void *stream);

/* The same with a per-expert bias (ADD_BIAS, grouped_fused_moe.py:501-503, 702-707): bias [E, N] of `bias_dtype`
 * (MI355_DTYPE_BF16 / _F16 / _F32), expert stride bias_stride_e elements, widened to fp32 and added to the
 * accumulator before the routed weight is applied (:709-715):
 *     out[idx, :] = cast( (blockscaled(Xq[row,:] . W[e]^T) + bias[e, :]) * (mul_routed_weight ? weight : 1) ).
 * bias == NULL is mi355_grouped_block_fp8_gemm_dtype. */
int mi355_grouped_block_fp8_gemm_bias(const void *Xq, const float *Xs, const void *W, const float *Ws,
                                      const int32_t *expert_to_token_index, const float *expert_to_weight,
                                      const int32_t *expert_token_num, const int32_t *table, int64_t table_rows,
                                      int32_t block_m, int64_t num_pairs, int64_t num_tokens, int32_t num_experts,
                                      int32_t topk_num, int64_t N, int64_t K, int32_t mul_routed_weight, void *out,
                                      void *ws, size_t ws_bytes, int32_t out_dtype, const void *bias,
                                      int32_t bias_dtype, int64_t bias_stride_e, void *stream);

/* ---- element-wise steps between / after the two expert GEMMs ------------------------------------------------ */

/*
 * out[m, h] = bf16( bf16(silu(in[m, h])) * in[m, H + h] ),  silu(g) = g / (1 + exp(-g)) in fp32.
 * in bf16 [M, 2H] = [gate | up] with row stride in_stride_m (elements), out bf16 [M, H] with row stride out_stride_m.
 * Replaces: silu_and_mul_fwd(input, output, layout="blocked")
 *           (lightllm/common/basemodel/triton_kernel/fused_moe/moe_silu_and_mul.py:9-93, 117-176).
 */
int mi355_silu_and_mul(const void *in, void *out, int64_t M, int64_t H, int64_t in_stride_m, int64_t out_stride_m,
                       void *stream);

/*
 * The other forms of the same reference kernel (moe_silu_and_mul.py:46-71): `interleaved` input
 * [gate0, up0, gate1, up1, ...] instead of [gate | up], and with `use_limit`
 *     g = min(gate, limit); u = clamp(up, -limit, limit)  (u stays bf16: the bound is limit rounded to bf16)
 *     out = bf16( bf16(u + 1) * bf16( g / (1 + exp(-g * alpha)) ) ).
 * Without either flag this is mi355_silu_and_mul.  The reference holds no test of these forms.
 */
int mi355_silu_and_mul_ex(const void *in, void *out, int64_t M, int64_t H, int64_t in_stride_m, int64_t out_stride_m,
                          int32_t interleaved, int32_t use_limit, float limit, float alpha, void *stream);

/*
 * The same product, quantized on the fly: q e4m3fn [M, H] contiguous and one fp32 scale per 1x128 group at
 * s[m * s_stride_m + g * s_stride_g]; arithmetic of mi355_group_quant_fp8 with eps = 1e-10 applied to the bf16
 * products, so the result equals mi355_silu_and_mul followed by mi355_group_quant_fp8 byte for byte.
 * masked_m == NULL: every row.  masked_m != NULL: the M rows are M / rows_per_expert experts of rows_per_expert
 * rows each and only the first masked_m[e] rows of expert e are computed; other rows of q and s are not written.
 * Replaces: silu_and_mul_masked_post_quant_fwd(input, output, output_scale, quant_group_size, masked_m)
 *           (lightllm/common/basemodel/triton_kernel/fused_moe/moe_silu_and_mul_mix_quant_ep.py:9-141), and the
 *           pair silu_and_mul_fwd + per_token_group_quant_fp8 inside fused_experts_impl
 *           (fused_moe/grouped_fused_moe.py:1084-1090 and :862-875).
 */
int mi355_silu_and_mul_group_quant_fp8(const void *in, void *q, float *s, int64_t M, int64_t H, int64_t in_stride_m,
                                       int32_t group, int64_t s_stride_m, int64_t s_stride_g,
                                       const int32_t *masked_m, int64_t rows_per_expert, void *stream);

/*
 * out[t, h] = bf16( sum_k in[t, k, h] ), fp32 accumulation in ascending k.  in bf16 [T, topk, H], out bf16 [T, H],
 * both contiguous.
 * Replaces: moe_sum_reduce(input, output) (lightllm/common/basemodel/triton_kernel/fused_moe/moe_sum_reduce.py:8-108).
 */
int mi355_moe_sum_reduce(const void *in, void *out, int64_t T, int32_t topk, int64_t H, void *stream);

/*
 * out[n, k] = bf16( float(q[n, k]) * s[n / 128, k / 128] ).  q e4m3fn [N, K] contiguous, s fp32
 * [ceil(N/128), ceil(K/128)] contiguous, out bf16 [N, K] contiguous.  The inverse of the block weight quantizer.
 * Replaces: weight_dequant(x, s, block_size=128) (lightllm/models/deepseek2/triton_kernel/weight_dequant.py:9-59).
 */
int mi355_block_weight_dequant(const void *q, const float *s, void *out, int64_t N, int64_t K, int32_t block,
                               void *stream);

/* ---- measurement aid ------------------------------------------------------------------------------------------
 * The inner arithmetic of the block-scaled GEMM with everything else taken away: one workgroup of `waves` (4 or 8)
 * waves per compute unit, each wave running `iters` times the 32 products v_mfma_f32_16x16x128_f8f6f4 of a
 * 128 x 64 sub-tile and one K step on operand fragments held in registers - accumulating in the matrix core
 * (fold = 0), or product by product with the fp32 scale fold of the kernels (fold = 1).  No LDS or memory traffic in
 * the loop.  `operands`: 128 KiB of e4m3 bytes (32-byte aligned; zeros or random bytes - the clock the part holds
 * depends on them); `sink`: 4 bytes per thread of the launch (compute units x 64 x waves).  Flops of a launch:
 * compute units x waves x iters x 32 x 65536.  No counterpart in the reference; bench.py --only ceiling times it to
 * state what the hardware gives this arithmetic at most. */
int mi355_probe_mfma(const void *operands, void *sink, int32_t fold, int32_t waves, int32_t iters, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_FP8_H */

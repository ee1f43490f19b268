/*
 * CPU oracle for the block-FP8 W8A8 linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests, the smoke check and
 * the benchmark's cpu_baseline leg may build, link or call it.  Nothing under
 * the shipped package may include or load it.
 *
 * Every function restates, in plain scalar C with IEEE-754 binary32 arithmetic
 * (compile with -O2 -ffp-contract=off, never -ffast-math), the arithmetic of
 * one function of the reference.  The citations name the reference file and
 * lines each function follows (paths relative to the reference tree).
 *
 * Pinning status (which independent facts each function is checked against
 * lives in tests/test_oracle_*.py):
 *   oracle_f32_to_e4m3fn        pinned: known-answer table + torch CPU cast over
 *                               every bf16 pattern and a dense fp32 sweep
 *   oracle_group_quant_fp8(_f32) pinned: torch closed form (bf16, fp16 and fp32 inputs), special cases,
 *                               invariants; groups holding NaN/Inf: own definition, outside the reference's contract
 *   oracle_block_weight_quant   pinned: torch closed form
 *   oracle_block_gemm*          pinned: unit-scale / one-hot special cases, numpy f64
 *   oracle_moe_align, _align1, _align_fused, _align2   pinned: the reference's own golden vectors
 *   oracle_grouped_block_gemm   pinned: per-expert loop of the dense oracle; the bias term by zero bias (= no bias),
 *                               zero activations (= bf16(bias * routed weight) exactly) and the torch closed form
 *   oracle_silu_and_mul         pinned: torch closed form (bit-equal but for rare 1-ulp exp differences), special values
 *   oracle_moe_sum_reduce       pinned: exactly summable inputs, torch closed form
 *   oracle_block_weight_dequant pinned: torch closed form, round trip through oracle_block_weight_quant
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bf16 -> fp32 is exact: the 16 bits are the top half of the fp32 pattern. */
float oracle_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even (the cast `acc.to(C.dtype.element_ty)`,
 * quantization/fp8w8a8_block_gemm_kernel.py:78). NaN stays NaN. */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* e4m3fn (OCP FP8 E4M3, finite-only: bias 7, max 448, 0x7F/0xFF = NaN) -> fp32. */
float oracle_e4m3fn_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    float v;
    if (e == 0xf && m == 7) return bits_to_f32(sign | 0x7fc00000u);
    if (e == 0) v = ldexpf((float)m, -9);            /* subnormal: m * 2^-9 */
    else v = ldexpf((float)(8u + m), (int)e - 10);    /* (1 + m/8) * 2^(e-7) */
    return sign ? -v : v;
}

/* fp32 -> e4m3fn, round to nearest even on the 3-bit mantissa, subnormals kept,
 * NOT saturating: anything that rounds above 448 becomes NaN (0x7F | sign).
 * This is the cast the reference applies after its clamp
 * (`.to(y_q_ptr.dtype.element_ty)`, quantization/fp8act_quant_kernel.py:57,
 *  and `.to(dtype)` in torch_quant, same file :250). */
uint8_t oracle_f32_to_e4m3fn(float f) {
    uint32_t u = f32_to_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7f);          /* NaN */
    if (a >= 0x43f00000u) return (uint8_t)(sign | 0x7f);         /* |x| >= 480: past the last finite code;
                                                                    (464, 480) rounds up into 0x7F below,
                                                                    464 itself ties to even = 448 */
    if (a < 0x3a800000u) {                                       /* |x| < 2^-10 */
        return sign;                                             /* rounds to zero */
    }
    int32_t exp = (int32_t)(a >> 23) - 127;                      /* unbiased */
    uint32_t man = (a & 0x7fffffu) | 0x800000u;                  /* 24-bit significand */
    uint32_t q;                                                  /* value in units of the target ulp */
    int shift;
    if (exp < -6) {
        /* subnormal target: ulp = 2^-9; value = man * 2^(exp-23) = q * 2^-9 */
        shift = 23 - (exp + 9);                                  /* >= 21 */
    } else {
        shift = 20;                                              /* keep 1+3 bits */
    }
    if (shift > 31) return sign;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    q = man >> shift;
    if (rem > half || (rem == half && (q & 1u))) q += 1u;
    uint8_t out;
    if (exp < -6) {
        /* q in [0, 8]; q == 8 is the smallest normal (0x08) and encodes itself */
        out = (uint8_t)q;
    } else {
        /* q in [8, 16]; 16 means carry into the next binade */
        uint32_t e = (uint32_t)(exp + 7);
        if (q == 16u) { q = 8u; e += 1u; }
        out = (uint8_t)((e << 3) | (q & 7u));
    }
    return (uint8_t)(sign | out);
}

/*
 * per_token_group_quant_fp8: one scale per `group` contiguous elements of a row.
 * Follows quantization/fp8act_quant_kernel.py:52-57 (kernel body: any input dtype is
 * widened to fp32 first, :52) and :239-251 (the reference's own torch restatement):
 *     y      = x.to(f32)
 *     absmax = max(max(|y|), eps)
 *     s      = absmax / 448           (IEEE division)
 *     q      = clamp(y / s, -448, 448).to(e4m3fn)
 * x: fp32 values [M,K] contiguous (bf16 and fp16 inputs widen exactly); q: bytes
 * [M,K]; s: fp32 with element strides (s_stride_m, s_stride_g) so both the
 * row-major and the column-major scale layouts (:37-42) are covered.
 *
 * Non-finite inputs are outside the reference's contract (its max and clamp on NaN
 * are unspecified).  This build defines them: a group that holds a NaN or an
 * infinity gets the scale NaN (0x7FC00000) and every byte 0x7F with the sign bit of
 * its element, so bad activations stay visible downstream instead of turning into
 * plausible numbers.
 */
static void group_quant_row(const float *xp, int32_t group, float eps, uint8_t *qp, float *sp) {
    const float fp8_max = 448.0f;
    float amax = 0.0f;
    int finite = 1;
    for (int32_t j = 0; j < group; ++j) {
        float a = fabsf(xp[j]);
        if (!(a <= 3.4028234663852886e38f)) finite = 0;   /* NaN or infinity */
        if (a > amax) amax = a;
    }
    if (!finite) {
        for (int32_t j = 0; j < group; ++j) qp[j] = (uint8_t)(((f32_to_bits(xp[j]) >> 24) & 0x80u) | 0x7fu);
        *sp = bits_to_f32(0x7fc00000u);
        return;
    }
    if (!(amax > eps)) amax = eps;
    volatile float sc = amax / fp8_max;
    for (int32_t j = 0; j < group; ++j) {
        volatile float y = xp[j] / sc;
        float c = y;
        if (c > fp8_max) c = fp8_max;
        if (c < -fp8_max) c = -fp8_max;
        qp[j] = oracle_f32_to_e4m3fn(c);
    }
    *sp = sc;
}

void oracle_group_quant_fp8_f32(const float *x, int64_t M, int64_t K, int32_t group, float eps,
                                uint8_t *q, float *s, int64_t s_stride_m, int64_t s_stride_g) {
    int64_t G = K / group;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t g = 0; g < G; ++g)
            group_quant_row(x + m * K + g * group, group, eps, q + m * K + g * group,
                            s + m * s_stride_m + g * s_stride_g);
}

/* The same for bf16 bit patterns (the layout the hot path sees). */
void oracle_group_quant_fp8(const uint16_t *x, int64_t M, int64_t K, int32_t group, float eps,
                            uint8_t *q, float *s, int64_t s_stride_m, int64_t s_stride_g) {
    int64_t G = K / group;
    float *row = (float *)malloc((size_t)group * sizeof(float));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t g = 0; g < G; ++g) {
            const uint16_t *xp = x + m * K + g * group;
            for (int32_t j = 0; j < group; ++j) row[j] = oracle_bf16_to_f32(xp[j]);
            group_quant_row(row, group, eps, q + m * K + g * group, s + m * s_stride_m + g * s_stride_g);
        }
    free(row);
}

/*
 * Load-time 128x128 block weight quantizer, quirk included
 * (quantization/fp8w8a8_block_quant_kernel.py:18-27):
 *     amax  = max |w| over the block (out-of-range elements read as 0)
 *     scale = amax / 448                       <- this is what is stored
 *     q     = (w / (scale + 1e-6)).to(e4m3fn)  <- no clamp, divisor differs from the stored scale
 * w: fp32 [N,K] contiguous; q: [N,K]; s: [ceil(N/block), ceil(K/block)].
 */
void oracle_block_weight_quant(const float *w, int64_t N, int64_t K, int32_t block, uint8_t *q, float *s) {
    int64_t nb = (N + block - 1) / block, kb = (K + block - 1) / block;
    for (int64_t bi = 0; bi < nb; ++bi) {
        for (int64_t bj = 0; bj < kb; ++bj) {
            int64_t n1 = (bi + 1) * block < N ? (bi + 1) * block : N;
            int64_t k1 = (bj + 1) * block < K ? (bj + 1) * block : K;
            float amax = 0.0f;
            for (int64_t n = bi * block; n < n1; ++n)
                for (int64_t k = bj * block; k < k1; ++k) {
                    float a = fabsf(w[n * K + k]);
                    if (a > amax) amax = a;
                }
            volatile float scale = amax / 448.0f;
            volatile float div = scale + 1e-6f;
            for (int64_t n = bi * block; n < n1; ++n)
                for (int64_t k = bj * block; k < k1; ++k) {
                    volatile float y = w[n * K + k] / div;
                    q[n * K + k] = oracle_f32_to_e4m3fn(y);
                }
            s[bi * kb + bj] = scale;
        }
    }
}

static float e4m3_lut[256];
static int e4m3_lut_ready = 0;
static void init_lut(void) {
    if (e4m3_lut_ready) return;
    for (int i = 0; i < 256; ++i) e4m3_lut[i] = oracle_e4m3fn_to_f32((uint8_t)i);
    e4m3_lut_ready = 1;
}

/* One output element in the reference kernel's own order
 * (quantization/fp8w8a8_block_gemm_kernel.py:67-76):
 *     acc += dot(a_blk, b_blk) * a_s * b_s      per K block, fp32
 * The per-block dot of fp8 values is exact in double (products of two 4-bit
 * significands, 128 terms), so it is rounded to fp32 once, as an ideal
 * fp32-accumulating matrix unit would. */
static float gemm_element_f32(const uint8_t *a, const float *as, int64_t as_stride,
                              const uint8_t *b, const float *bs, int64_t bs_stride,
                              int64_t K, int32_t bk) {
    float acc = 0.0f;
    int64_t kb = 0;
    for (int64_t k0 = 0; k0 < K; k0 += bk, ++kb) {
        int64_t k1 = k0 + bk < K ? k0 + bk : K;
        double d = 0.0;
        for (int64_t k = k0; k < k1; ++k) d += (double)e4m3_lut[a[k]] * (double)e4m3_lut[b[k]];
        volatile float t = (float)d;
        t = t * as[kb * as_stride];
        t = t * bs[kb * bs_stride];
        acc = acc + t;
    }
    return acc;
}

/*
 * w8a8_block_fp8_matmul (quantization/fp8w8a8_block_gemm_kernel.py:24-84, 127-192).
 * Aq [M,K] bytes; As fp32 [M, ceil(K/bk)] row-major; Bq given as the weight's
 * storage [N,K] (the reference receives its transposed view, common/quantization/w8a8.py:442);
 * Bs fp32 [ceil(N/bn), ceil(K/bk)] (weight-scale storage, w8a8.py:443 passes its .t()).
 * Writes fp32 results to C32 (may be NULL) and bf16 bit patterns to Cbf (may be NULL).
 */
void oracle_block_gemm(const uint8_t *Aq, const float *As, const uint8_t *Bq, const float *Bs,
                       int64_t M, int64_t N, int64_t K, int32_t bn, int32_t bk,
                       float *C32, uint16_t *Cbf) {
    init_lut();
    int64_t KB = (K + bk - 1) / bk;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float v = gemm_element_f32(Aq + m * K, As + m * KB, 1, Bq + n * K, Bs + (n / bn) * KB, 1, K, bk);
            if (C32) C32[m * N + n] = v;
            if (Cbf) Cbf[m * N + n] = oracle_f32_to_bf16(v);
        }
}

/* Ground truth at chosen entries: dequantise, then multiply, all in double.
 * This is the "fp32 dequant-then-matmul" the tolerance is stated against
 * (fp8w8a8_block_gemm_kernel.py:213-217), computed at a precision where its own
 * rounding is invisible.  out[i*ncols+j] = C[rows[i], cols[j]]. */
void oracle_dequant_matmul_sampled(const uint8_t *Aq, const float *As, const uint8_t *Bq, const float *Bs,
                                   int64_t M, int64_t N, int64_t K, int32_t bn, int32_t bk,
                                   const int64_t *rows, int64_t nrows, const int64_t *cols, int64_t ncols,
                                   double *out) {
    init_lut();
    (void)M; (void)N;
    int64_t KB = (K + bk - 1) / bk;
    for (int64_t i = 0; i < nrows; ++i)
        for (int64_t j = 0; j < ncols; ++j) {
            int64_t m = rows[i], n = cols[j];
            const uint8_t *a = Aq + m * K, *b = Bq + n * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                double da = (double)(e4m3_lut[a[k]] * As[m * KB + k / bk]);   /* fp32 dequant */
                double db = (double)(e4m3_lut[b[k]] * Bs[(n / bn) * KB + k / bk]);
                acc += da * db;
            }
            out[i * ncols + j] = acc;
        }
}

/*
 * moe_align_fused, ordered form (fused_moe/grouped_fused_moe.py:216-253, 388-396):
 * bucket the flattened (token, slot) pairs by expert, keeping ascending pair
 * index inside every expert; copy the routing weight alongside; count per expert.
 * Entries past an expert's count are left untouched (the reference leaves
 * torch.empty garbage there).
 */
void oracle_moe_align_fused(const int32_t *topk_ids, const float *topk_weights, int64_t num_pairs,
                            int32_t num_experts, int32_t *expert_to_token_index, float *expert_to_weight,
                            int32_t *expert_token_num) {
    for (int32_t e = 0; e < num_experts; ++e) expert_token_num[e] = 0;
    for (int64_t i = 0; i < num_pairs; ++i) {
        int32_t e = topk_ids[i];
        if (e < 0 || e >= num_experts) continue;
        int32_t pos = expert_token_num[e]++;
        expert_to_token_index[(int64_t)e * num_pairs + pos] = (int32_t)i;
        expert_to_weight[(int64_t)e * num_pairs + pos] = topk_weights[i];
    }
}

/*
 * moe_align (grouped_fused_moe.py:39-98): 0/1 table [E, num_pairs], zero-filled first (:86), then 1 at
 * (topk_ids[j], j) (:49-55).
 */
void oracle_moe_align(const int32_t *topk_ids, int64_t num_pairs, int32_t num_experts, int32_t *out) {
    for (int64_t i = 0; i < (int64_t)num_experts * num_pairs; ++i) out[i] = 0;
    for (int64_t j = 0; j < num_pairs; ++j) {
        int32_t e = topk_ids[j];
        if (e >= 0 && e < num_experts) out[(int64_t)e * num_pairs + j] = 1;
    }
}

/*
 * moe_align1 (grouped_fused_moe.py:101-214): for every expert, walk its row of the 0/1 table in order and
 * write, IN PLACE, the position of each 1 at the next free slot (running count, :127-133), the weight of that
 * pair at the same slot of experts_weight_info (:134-138), and the count (:140).  Slots past the count keep
 * their old contents, which is what the reference's golden vector shows.
 */
void oracle_moe_align1(int32_t *experts_info, const float *topk_weights, int64_t num_pairs, int32_t num_experts,
                       float *experts_weight_info, int32_t *expert_token_num) {
    for (int32_t e = 0; e < num_experts; ++e) {
        int32_t *row = experts_info + (int64_t)e * num_pairs;
        float *wrow = experts_weight_info + (int64_t)e * num_pairs;
        int32_t cnt = 0;
        for (int64_t j = 0; j < num_pairs; ++j) {
            if (row[j] == 1) {
                row[cnt] = (int32_t)j;      /* cnt <= j: never overwrites an entry not yet visited */
                wrow[cnt] = topk_weights[j];
                ++cnt;
            }
        }
        expert_token_num[e] = cnt;
    }
}

/* Number of rows of the m-block schedule table (grouped_fused_moe.py:457-458). */
int64_t oracle_moe_align2_rows(int64_t num_pairs, int32_t num_experts, int32_t block_m) {
    int64_t padded = num_pairs + (int64_t)num_experts * (block_m - 1);
    int64_t blocks = (padded + block_m - 1) / block_m;
    return blocks < num_pairs ? blocks : num_pairs;
}

/*
 * moe_align2 (grouped_fused_moe.py:399-477): expand per-expert counts into the
 * schedule table of (expert, m_index, token_start, rows) rows, one per block
 * of block_m tokens, experts in ascending order (`rows` = tokens in the block,
 * derived: min(block_m, count - m_index*block_m)); rows past the last real
 * block get expert = -1 (only column 0 is written for them).
 */
void oracle_moe_align2(const int32_t *expert_token_num, int32_t num_experts, int32_t block_m,
                       int64_t max_blocks, int32_t *table /* [max_blocks,4] */) {
    int64_t row = 0;
    int32_t token_start = 0;
    for (int32_t e = 0; e < num_experts; ++e) {
        int32_t cnt = expert_token_num[e];
        int32_t nblk = (cnt + block_m - 1) / block_m;
        for (int32_t b = 0; b < nblk && row < max_blocks; ++b, ++row) {
            table[row * 4 + 0] = e;
            table[row * 4 + 1] = b;
            table[row * 4 + 2] = token_start + b * block_m;
            table[row * 4 + 3] = cnt - b * block_m < block_m ? cnt - b * block_m : block_m;
        }
        token_start += cnt;
    }
    for (; row < max_blocks; ++row) table[row * 4 + 0] = -1;
}

/*
 * grouped_matmul, fp8 block branch, gather/scatter form
 * (grouped_fused_moe.py:480-728 with OUT_SORTED = TOKEN_INPUT_USE_TMA = False):
 * for expert e and slot j < expert_token_num[e]:
 *     idx = expert_to_token_index[e, j]
 *     row = idx / topk_num                      (:587, :619)
 *     out[idx, :] = bf16( (blockscaled(Xq[row] . W[e]^T) [+ bias[e, :]]) [* expert_to_weights[e, j]] )   (:702-725)
 * Xq [T,K] bytes, Xs [T,K/bk]; W [E,N,K] bytes, Ws [E, N/bn, K/bk]; bias fp32 [E,N] or NULL (added to the fp32
 * accumulator before the routed weight, :702-715);
 * out bf16 bits [num_pairs, N].  Rows of `out` that no pair maps to are untouched.
 */
void oracle_grouped_block_gemm(const uint8_t *Xq, const float *Xs, const uint8_t *W, const float *Ws,
                               const int32_t *expert_to_token_index, const float *expert_to_weights,
                               const int32_t *expert_token_num, int64_t num_pairs, int32_t num_experts,
                               int32_t topk_num, int64_t N, int64_t K, int32_t bn, int32_t bk,
                               int32_t mul_routed_weight, const float *bias, uint16_t *out) {
    init_lut();
    int64_t KB = (K + bk - 1) / bk, NB = (N + bn - 1) / bn;
    for (int32_t e = 0; e < num_experts; ++e) {
        const uint8_t *We = W + (int64_t)e * N * K;
        const float *Wse = Ws + (int64_t)e * NB * KB;
        for (int32_t j = 0; j < expert_token_num[e]; ++j) {
            int32_t idx = expert_to_token_index[(int64_t)e * num_pairs + j];
            int64_t row = idx / topk_num;
            float rw = expert_to_weights[(int64_t)e * num_pairs + j];
            for (int64_t n = 0; n < N; ++n) {
                volatile float v = gemm_element_f32(Xq + row * K, Xs + row * KB, 1, We + n * K,
                                                    Wse + (n / bn) * KB, 1, K, bk);
                if (bias) v = v + bias[(int64_t)e * N + n];
                if (mul_routed_weight) v = v * rw;
                out[(int64_t)idx * N + n] = oracle_f32_to_bf16(v);
            }
        }
    }
}

/*
 * silu_and_mul on the "blocked" layout (fused_moe/moe_silu_and_mul.py:9-93):
 * in  bf16 [M, 2*H] = [gate | up];  out bf16 [M, H]
 *     g = gate.to(f32); out = (g / (1 + exp(-g))).to(bf16) * up      (product taken in bf16)
 */
void oracle_silu_and_mul(const uint16_t *in, int64_t M, int64_t H, uint16_t *out) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t h = 0; h < H; ++h) {
            float g = oracle_bf16_to_f32(in[m * 2 * H + h]);
            float u = oracle_bf16_to_f32(in[m * 2 * H + H + h]);
            volatile float sg = g / (1.0f + expf(-g));
            float gb = oracle_bf16_to_f32(oracle_f32_to_bf16(sg));
            out[m * H + h] = oracle_f32_to_bf16(gb * u);
        }
}

/*
 * The other forms of the same kernel (moe_silu_and_mul.py:46-71): interleaved input [g0,u0,g1,u1,...] and the
 * limit/alpha variant
 *     g = min(gate.f32, limit); u = clamp(up, -limit, limit)    (up stays bf16: the bound is bf16(limit))
 *     gate = (1 / (1 + exp(-g * alpha)) * g).to(bf16);  out = (u + 1) * gate   (both in bf16 arithmetic)
 * The reference has no test of these forms: pinned against float64 only ("parity unpinned" by the reference).
 */
void oracle_silu_and_mul_ex(const uint16_t *in, int64_t M, int64_t H, int32_t interleaved, int32_t use_limit,
                            float limit, float alpha, uint16_t *out) {
    const float lb = oracle_bf16_to_f32(oracle_f32_to_bf16(limit));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t h = 0; h < H; ++h) {
            const uint16_t *row = in + m * 2 * H;
            float g = oracle_bf16_to_f32(interleaved ? row[2 * h] : row[h]);
            float u = oracle_bf16_to_f32(interleaved ? row[2 * h + 1] : row[H + h]);
            if (!use_limit) {
                volatile float sg = g / (1.0f + expf(-g));
                float gb = oracle_bf16_to_f32(oracle_f32_to_bf16(sg));
                out[m * H + h] = oracle_f32_to_bf16(gb * u);
                continue;
            }
            if (g > limit) g = limit;
            if (u < -lb) u = -lb;
            if (u > lb) u = lb;
            volatile float sig = 1.0f / (1.0f + expf(-g * alpha));
            volatile float sg = sig * g;
            float gb = oracle_bf16_to_f32(oracle_f32_to_bf16(sg));
            float up1 = oracle_bf16_to_f32(oracle_f32_to_bf16(u + 1.0f));
            out[m * H + h] = oracle_f32_to_bf16(up1 * gb);
        }
}

/* moe_sum_reduce (fused_moe/moe_sum_reduce.py:8-108): out[t,h] = bf16( sum_k in[t,k,h] ), fp32 accumulate
 * in ascending k. */
void oracle_moe_sum_reduce(const uint16_t *in, int64_t T, int32_t topk, int64_t H, uint16_t *out) {
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            float acc = 0.0f;
            for (int32_t k = 0; k < topk; ++k) acc += oracle_bf16_to_f32(in[(t * topk + k) * H + h]);
            out[t * H + h] = oracle_f32_to_bf16(acc);
        }
}

/* weight_dequant (models/deepseek2/triton_kernel/weight_dequant.py:9-59): out[n,k] = bf16( f32(q[n,k]) * s[n/block, k/block] ). */
void oracle_block_weight_dequant(const uint8_t *q, const float *s, int64_t N, int64_t K, int32_t block, uint16_t *out) {
    const int64_t kb = (K + block - 1) / block;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            volatile float y = oracle_e4m3fn_to_f32(q[n * K + k]) * s[(n / block) * kb + k / block];
            out[n * K + k] = oracle_f32_to_bf16(y);
        }
}

/*
 * Replays, on the CPU, the exact operation sequence the HIP quantizer uses in place of two IEEE
 * divisions (csrc/quant_core.hpp: quant_chunk/quot), for every bf16 group maximum with bit pattern in
 * [amax_lo, amax_hi) stepping by `step`, against every bf16 element of either sign with |x| <= amax
 * (and every |x| < eps when the eps floor applies).  Returns how many (amax, x) pairs give a byte or a
 * scale different from the IEEE closed form above.  Zero for the whole range means the kernel's
 * shortcut is exact; it must stay in step with the kernel source.
 */
int64_t oracle_fast_quant_mismatches(uint32_t amax_lo, uint32_t amax_hi, uint32_t step) {
    const float eps = 1e-10f, c448 = 1.0f / 448.0f;
    int64_t bad = 0;
    for (uint32_t ab = amax_lo; ab < amax_hi && ab <= 0x7f7fu; ab += step) {
        float amax = oracle_bf16_to_f32((uint16_t)ab);
        uint32_t xmax = ab;
        if (!(amax > eps)) {
            if (ab != 0) continue;       /* every maximum below eps gives the same scale: test it once, */
            amax = eps;
            xmax = 0x2edbu;              /* against every bf16 magnitude below 1e-10 */
        }
        volatile float s_ref = amax / 448.0f;
        /* kernel: scale */
        float q0 = amax * c448;
        float s = fmaf(fmaf(-q0, 448.0f, amax), c448, q0);
        if (f32_to_bits(s) != f32_to_bits(s_ref)) { ++bad; continue; }
        volatile float r = 1.0f / s;
        for (uint32_t xb = 0; xb <= xmax; ++xb) {
            for (uint32_t sign = 0; sign <= 0x8000u; sign += 0x8000u) {
                float x = oracle_bf16_to_f32((uint16_t)(xb | sign));
                /* reference */
                volatile float y = x / s_ref;
                float cl = y;
                if (cl > 448.0f) cl = 448.0f;
                if (cl < -448.0f) cl = -448.0f;
                uint8_t want = oracle_f32_to_e4m3fn(cl);
                /* kernel */
                float y0 = x * r;
                float e = fmaf(-y0, s, x);
                float y1 = fmaf(e, r, y0);
                float fixed = bits_to_f32((f32_to_bits(y1) & 0x7fffffffu) | (f32_to_bits(x) & 0x80000000u));
                uint8_t got = oracle_f32_to_e4m3fn(fixed);
                if ((got & 0x7f) == 0x7f) got = (uint8_t)((got & 0x80) | 0x7e); /* the hardware cast saturates */
                if (got != want) ++bad;
            }
        }
    }
    return bad;
}

/* Bulk helpers so tests can sweep millions of values without a Python loop. */
void oracle_f32_to_e4m3fn_array(const float *x, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_e4m3fn(x[i]);
}
void oracle_e4m3fn_to_f32_array(const uint8_t *x, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_e4m3fn_to_f32(x[i]);
}
void oracle_f32_to_bf16_array(const float *x, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16(x[i]);
}

"""Pins the CPU oracle (oracle/fp8_oracle.c) against facts it does not itself compute:
known-answer bytes, torch's own float8 cast, the reference's torch closed forms, special cases whose answer
the arithmetic fixes, and brute force in float64."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H


# ---- the e4m3fn cast -------------------------------------------------------------------------------------
KAT = [  # (value, byte): RTNE, subnormals, no saturation (measured facts about the float8_e4m3fn format)
    (0.0, 0x00), (1.0, 0x38), (448.0, 0x7E), (449.0, 0x7E), (464.0, 0x7E), (465.0, 0x7F), (480.0, 0x7F),
    (1000.0, 0x7F), (-1000.0, 0xFF), (2.0 ** -10, 0x00), (2.0 ** -9, 0x01), (1.5 * 2.0 ** -9, 0x02),
    (17.0, 0x58), (18.0, 0x59), (19.0, 0x5A), (-1.0, 0xB8), (2.0 ** -6, 0x08), (0.875 * 2.0 ** -6, 0x07),
    (240.0, 0x77), (-0.0, 0x80),
]


def test_e4m3_known_answers():
    vals = np.array([v for v, _ in KAT], np.float32)
    got = oracle.f32_to_e4m3fn(vals)
    assert got.tolist() == [b for _, b in KAT]
    assert oracle.f32_to_e4m3fn(np.array([np.nan], np.float32))[0] & 0x7F == 0x7F


def test_e4m3_decode_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    mine = oracle.e4m3fn_to_f32(codes)
    theirs = tr.fp8_from_bits(codes).float().numpy()
    ok = ~np.isnan(theirs)
    assert np.array_equal(mine[ok], theirs[ok]) and np.isnan(mine[~ok]).all()
    # every finite code survives a round trip
    assert np.array_equal(oracle.f32_to_e4m3fn(mine[ok]), codes[ok])


def test_e4m3_cast_matches_torch_everywhere_it_matters():
    bits = np.arange(65536, dtype=np.uint16)
    x = tr.bf16_from_bits(bits).float()
    finite = ~torch.isnan(x)
    assert np.array_equal(oracle.f32_to_e4m3fn(x.numpy())[finite.numpy()],
                          tr.bits_of(x.to(torch.float8_e4m3fn))[finite.numpy()])
    # dense sweep of fp32 patterns over [2^-12, 1024), both signs (every 61st pattern)
    u = np.arange(0x39800000, 0x44800000, 61, dtype=np.uint32)
    for sign in (0, 0x80000000):
        f = (u | np.uint32(sign)).view(np.float32)
        assert np.array_equal(oracle.f32_to_e4m3fn(f), tr.bits_of(torch.from_numpy(f.copy()).to(torch.float8_e4m3fn)))
    # exact ties between neighbouring codes go to the even code
    codes = np.arange(0, 0x7E, dtype=np.uint8)
    lo, hi = oracle.e4m3fn_to_f32(codes), oracle.e4m3fn_to_f32(codes + 1)
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    got = oracle.f32_to_e4m3fn(mid)
    assert np.array_equal(got, np.where(codes % 2 == 0, codes, codes + 1))


def test_bf16_rounding_matches_torch():
    g = H.gen(3)
    x = torch.randn(200000, generator=g) * torch.exp2(torch.randint(-30, 30, (200000,), generator=g).float())
    assert np.array_equal(oracle.f32_to_bf16(x.numpy()), tr.bits_of(x.to(torch.bfloat16)))
    ties = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001], np.uint32).view(np.float32)
    assert oracle.f32_to_bf16(ties).tolist() == [0x3F80, 0x3F82, 0x3F80, 0x3F81]


# ---- the activation quantizer --------------------------------------------------------------------------
@pytest.mark.parametrize("M,K,kw", [(32, 4096, {}), (64, 1024, {"outliers": True, "zero_row": True}), (3, 128, {})])
def test_group_quant_equals_torch_closed_form(M, K, kw):
    x = H.activations(M, K, seed=M + K, **kw)
    q_t, s_t = tr.group_quant(x)
    q_c, s_c = oracle.group_quant_fp8(tr.bits_of(x))
    assert np.array_equal(tr.bits_of(s_t), s_c.view(np.uint32))
    assert np.array_equal(tr.bits_of(q_t), q_c)


@pytest.mark.parametrize("M,K,group", [(4, 4096, 4096), (5, 1024, 64), (3, 120, 24), (2, 100, 100)])
def test_group_quant_other_group_sizes_equal_torch_closed_form(M, K, group):
    """The group size is a parameter of the reference's kernel; the oracle follows the same closed form for any."""
    x = H.activations(M, K, seed=M + K + group, outliers=True)
    q_t, s_t = tr.group_quant(x, group=group)
    q_c, s_c = oracle.group_quant_fp8(tr.bits_of(x), group=group)
    assert np.array_equal(tr.bits_of(s_t), s_c.view(np.uint32))
    assert np.array_equal(tr.bits_of(q_t), q_c)


def test_group_quant_special_cases():
    # all-zero group: eps floor, scale bits of fp32(1e-10)/448, bytes zero
    z = np.zeros((1, 128), np.uint16)
    q, s = oracle.group_quant_fp8(z)
    assert s.view(np.uint32)[0, 0] == 0x2A7B5123 and not q.any()
    assert np.float32(1e-10).view(np.uint32) == 0x2EDBE6FF
    # group maximum 448 * 2^k: scale is exactly 2^k and the bytes are the exact cast of x / 2^k
    for k in (-20, -3, 0, 5, 40):
        vals = np.array([448.0, -448.0, 1.0, 17.0, 18.0, 19.0, 0.3125, -2.0 ** -9, 2.0 ** -10, 100.0] + [0.0] * 118,
                        np.float32) * np.float32(2.0 ** k)
        xb = oracle.f32_to_bf16(vals).reshape(1, 128)
        assert np.array_equal(oracle.bf16_to_f32(xb).ravel(), vals), "test values must be bf16-exact"
        q, s = oracle.group_quant_fp8(xb)
        assert s[0, 0] == np.float32(2.0 ** k)
        assert np.array_equal(q[0], oracle.f32_to_e4m3fn(vals / np.float32(2.0 ** k)))
        assert q[0, 0] == 0x7E and q[0, 1] == 0xFE


def test_group_quant_invariants():
    x = H.activations(256, 2048, seed=12, outliers=True)
    xb = tr.bits_of(x)
    q, s = oracle.group_quant_fp8(xb)
    xf = oracle.bf16_to_f32(xb).reshape(256, 16, 128)
    qf = oracle.e4m3fn_to_f32(q).reshape(256, 16, 128)
    assert not ((q & 0x7F) == 0x7F).any()                                  # never the NaN code
    assert np.array_equal(q >> 7, xb >> 15)                                # sign bit preserved
    # the group maximum lands on +-448
    am = np.abs(xf).argmax(-1)
    top = np.take_along_axis(q.reshape(256, 16, 128), am[..., None], -1)[..., 0]
    assert np.all((top & 0x7F) == 0x7E)
    # monotone inside a group
    order = np.argsort(xf, axis=-1)
    assert np.all(np.diff(np.take_along_axis(qf, order, -1), axis=-1) >= 0)
    # rounding error of the dequantised value is at most half an e4m3 ulp of the quotient (plus fp32 slack)
    y = xf / s[..., None]
    ulp = np.where(np.abs(y) < 2.0 ** -6, 2.0 ** -9, 2.0 ** (np.floor(np.log2(np.maximum(np.abs(y), 1e-30))) - 3))
    assert np.all(np.abs(qf - y) <= ulp / 2 * (1 + 1e-6))


def test_group_quant_column_major_layout():
    x = H.activations(10, 512, seed=13)
    q1, s1 = oracle.group_quant_fp8(tr.bits_of(x))
    q2, s2 = oracle.group_quant_fp8(tr.bits_of(x), column_major=True)
    assert s2.strides == (4, 40) and np.array_equal(s1, s2) and np.array_equal(q1, q2)


def test_kernel_division_shortcut_is_exact():
    """The HIP quantizer replaces x/s by a multiply and two fused multiply-adds.  Replaying those operations on
    the CPU for EVERY (bf16 group maximum, bf16 element of either sign) pair gives the IEEE bytes and scales."""
    assert oracle.fast_quant_mismatches(0, 0x7F80, 1) == 0


# ---- the weight quantizer ------------------------------------------------------------------------------
@pytest.mark.parametrize("N,K", [(256, 384), (200, 300), (128, 128)])
def test_weight_quant_equals_torch_closed_form(N, K):
    w = H.weights(N, K, seed=N)
    q_t, s_t = tr.block_weight_quant(w)
    q_c, s_c = oracle.block_weight_quant(w.float().numpy())
    assert np.array_equal(tr.bits_of(s_t), s_c.view(np.uint32))
    assert np.array_equal(tr.bits_of(q_t), q_c)


def test_weight_quant_quirk():
    """Stored scale is amax/448 but the divisor is scale + 1e-6: the quotient of the block maximum stays
    below 448 (here by about half a percent) before the cast rounds it."""
    w = H.weights(128, 128, seed=5)
    q, s = oracle.block_weight_quant(w.float().numpy())
    amax = float(w.float().abs().max())
    assert s[0, 0] == np.float32(amax) / np.float32(448.0)
    top = np.abs(oracle.e4m3fn_to_f32(q)).max()
    expect = amax / (float(s[0, 0]) + 1e-6)
    assert top == oracle.e4m3fn_to_f32(oracle.f32_to_e4m3fn(np.array([expect], np.float32)))[0]
    assert 440 < expect < 447.9
    qz, sz = oracle.block_weight_quant(np.zeros((128, 128), np.float32))
    assert sz[0, 0] == 0 and not qz.any()


# ---- the block-scaled GEMM -----------------------------------------------------------------------------
def _rand_problem(M, N, K, seed):
    x = H.activations(M, K, seed=seed)
    q, s = oracle.group_quant_fp8(tr.bits_of(x))
    wq, ws = oracle.block_weight_quant(H.weights(N, K, seed=seed + 1).float().numpy())
    return q, s, wq, ws


def test_gemm_brute_force_float64():
    M, N, K = 5, 130, 256
    q, s, wq, ws = _rand_problem(M, N, K, 40)
    # dequantise in fp32 (as the reference's check does), multiply-accumulate in float64
    a = (oracle.e4m3fn_to_f32(q) * np.repeat(s, 128, 1)).astype(np.float64)
    b = (oracle.e4m3fn_to_f32(wq) * np.repeat(np.repeat(ws, 128, 0)[:N], 128, 1)).astype(np.float64)
    want = a @ b.T
    got64 = oracle.dequant_matmul_sampled(q, s, wq, ws, np.arange(M), np.arange(N))
    assert np.allclose(got64, want, rtol=1e-12, atol=0)
    bits, c32 = oracle.block_gemm(q, s, wq, ws, want_f32=True)
    assert np.abs(c32 - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(bits, oracle.f32_to_bf16(c32))
    # sampling picks the right rows/columns
    sub = oracle.dequant_matmul_sampled(q, s, wq, ws, [4, 1], [129, 0, 64])
    assert np.array_equal(sub, got64[[4, 1]][:, [129, 0, 64]])


def test_gemm_unit_scales_reduce_to_integer_matmul():
    g = np.random.default_rng(41)
    M, N, K = 7, 140, 384
    a = g.integers(-8, 9, (M, K)).astype(np.float32)
    b = g.integers(-8, 9, (N, K)).astype(np.float32)
    _, c32 = oracle.block_gemm(oracle.f32_to_e4m3fn(a), np.ones((M, 3), np.float32), oracle.f32_to_e4m3fn(b),
                               np.ones((2, 3), np.float32), want_f32=True)
    assert np.array_equal(c32, a @ b.T)  # integers: exact in fp32


def test_gemm_scales_enter_per_block_and_per_operand():
    """A transposed or mis-indexed scale must fail here: distinct power-of-two scales per (row, k-block) and
    per (n-block, k-block), integer payloads, so the expected result is exact."""
    g = np.random.default_rng(42)
    M, N, K = 4, 256, 256
    a = g.integers(-4, 5, (M, K)).astype(np.float32)
    b = g.integers(-4, 5, (N, K)).astype(np.float32)
    As = 2.0 ** g.integers(-3, 4, (M, 2)).astype(np.float32)
    Bs = 2.0 ** g.integers(-3, 4, (2, 2)).astype(np.float32)
    want = np.zeros((M, N))
    for kb in range(2):
        blk = a[:, kb * 128:(kb + 1) * 128] @ b[:, kb * 128:(kb + 1) * 128].T
        want += blk * As[:, kb:kb + 1] * np.repeat(Bs[:, kb], 128)[None, :]
    _, c32 = oracle.block_gemm(oracle.f32_to_e4m3fn(a), As, oracle.f32_to_e4m3fn(b), Bs, want_f32=True)
    assert np.array_equal(c32, want.astype(np.float32))


def test_gemm_matches_torch_dequant_matmul_cpu_reference_config():
    """The reference's CPU-runnable case: M=32, N=K=4096, seed 0 (fp32 dequant + matmul, bf16 out)."""
    x = H.activations(32, 4096, seed=0)
    xq, xs = tr.group_quant(x)
    wq, ws = tr.block_weight_quant(H.weights(4096, 4096, seed=0))
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    bits = oracle.block_gemm(tr.bits_of(xq), xs.numpy(), tr.bits_of(wq), ws.numpy())
    got = tr.bf16_from_bits(bits).float()
    cos, rel = H.gemm_metrics(got, ref)
    assert cos >= 0.99999 and rel <= 2 ** -8, (cos, rel)   # two fp32 summation orders + one bf16 rounding


# ---- routing tables and the grouped GEMM -----------------------------------------------------------------
def test_moe_align_fused_reference_golden():
    """Vectors of unit_tests/common/fused_moe/test_grouped_fused_moe.py:80-126 (bincount / nonzero form)."""
    ids = np.array([[0, 1, 2], [0, 3, 1], [3, 1, 4]], np.int32)
    w = np.array([[0.3, 0.7, 0.1], [0.2, 0.8, 0.4], [0.5, 0.6, 0.9]], np.float32)
    idx, ew, cnt = oracle.moe_align_fused(ids, w, 5)
    assert cnt.tolist() == [2, 3, 1, 2, 1]
    assert idx[0, :2].tolist() == [0, 3] and idx[1, :3].tolist() == [1, 5, 7] and idx[3, :2].tolist() == [4, 6]
    assert np.allclose(ew[1, :3], [0.7, 0.4, 0.6])
    ids = (np.arange(128 * 17, dtype=np.int32).reshape(128, 17) % 5)
    idx, ew, cnt = oracle.moe_align_fused(ids, np.arange(ids.size, dtype=np.float32), 5)
    flat = ids.ravel()
    assert np.array_equal(cnt, np.bincount(flat, minlength=5))
    for e in range(5):
        want = np.nonzero(flat == e)[0]
        assert np.array_equal(idx[e, :cnt[e]], want) and np.array_equal(ew[e, :cnt[e]], want.astype(np.float32))


def test_moe_align1_demo_of_the_reference():
    """The worked example in the reference's moe_align1 docstring (grouped_fused_moe.py:160-190)."""
    idx, ew, cnt = oracle.moe_align_fused(np.array([[0, 1], [1, 3]], np.int32),
                                          np.array([[0.3, 0.7], [0.2, 0.8]], np.float32), 4)
    assert cnt.tolist() == [1, 2, 0, 1]
    assert idx[0, 0] == 0 and idx[1, :2].tolist() == [1, 2] and idx[3, 0] == 3
    assert np.allclose(ew[1, :2], [0.7, 0.2]) and np.isclose(ew[3, 0], 0.8)


def test_moe_align2_reference_golden():
    """unit_tests/common/fused_moe/test_grouped_fused_moe.py:219-258."""
    t = oracle.moe_align2(100, [8, 0, 60, 16], 16)
    assert t.shape[0] == 10
    assert t[:, 0].tolist() == [0, 2, 2, 2, 2, 3, -1, -1, -1, -1]
    assert t[:6, 1].tolist() == [0, 0, 1, 2, 3, 0]
    assert t[:6, 2].tolist() == [0, 8, 24, 40, 56, 68]
    assert t[:6, 3].tolist() == [8, 16, 16, 16, 12, 16]
    t = oracle.moe_align2(8, [8] + [0] * 9, 16)
    assert t.shape[0] == 8 and t[0, 0] == 0 and np.all(t[1:, 0] == -1)


def test_grouped_gemm_is_a_per_expert_loop_of_the_dense_oracle():
    T, E, topk, N, K = 24, 5, 3, 140, 256
    ids, tw = H.routing(T, E, topk, seed=50)
    idx, ew, cnt = oracle.moe_align_fused(ids.numpy(), tw.numpy(), E)
    xq, xs = oracle.group_quant_fp8(tr.bits_of(H.activations(T, K, seed=51)))
    Wq = np.empty((E, N, K), np.uint8)
    Ws = np.empty((E, 2, 2), np.float32)
    for e in range(E):
        Wq[e], Ws[e] = oracle.block_weight_quant(H.weights(N, K, seed=60 + e).float().numpy())
    for mul in (False, True):
        out = oracle.grouped_block_gemm(xq, xs, Wq, Ws, idx, ew, cnt, topk, mul)
        flat = ids.numpy().ravel()
        for pair in range(T * topk):
            e, row = flat[pair], pair // topk
            _, c32 = oracle.block_gemm(xq[row:row + 1], xs[row:row + 1], Wq[e], Ws[e], want_f32=True)
            if mul:
                c32 = c32 * tw.numpy().ravel()[pair]
            assert np.array_equal(out[pair], oracle.f32_to_bf16(c32[0]))


def test_grouped_gemm_bias_term():
    """The per-expert bias (grouped_fused_moe.py:702-715: added to the fp32 accumulator, then the routed weight):
    a zero bias is no bias; with all-zero activations the output is bf16(bias * routed weight) exactly; and in
    general it equals the unbiased fp32 result plus the bias, in fp32, times the weight."""
    T, E, topk, N, K = 20, 4, 2, 140, 256
    ids, tw = H.routing(T, E, topk, seed=52)
    idx, ew, cnt = oracle.moe_align_fused(ids.numpy(), tw.numpy(), E)
    xq, xs = oracle.group_quant_fp8(tr.bits_of(H.activations(T, K, seed=53)))
    Wq = np.empty((E, N, K), np.uint8)
    Ws = np.empty((E, 2, 2), np.float32)
    for e in range(E):
        Wq[e], Ws[e] = oracle.block_weight_quant(H.weights(N, K, seed=70 + e).float().numpy())
    bias = torch.randn((E, N), generator=H.gen(54)).numpy().astype(np.float32)
    flat_e, flat_w = ids.numpy().ravel(), tw.numpy().ravel()
    for mul in (False, True):
        plain = oracle.grouped_block_gemm(xq, xs, Wq, Ws, idx, ew, cnt, topk, mul)
        assert np.array_equal(oracle.grouped_block_gemm(xq, xs, Wq, Ws, idx, ew, cnt, topk, mul,
                                                        bias=np.zeros_like(bias)), plain)
        zq, zs = oracle.group_quant_fp8(np.zeros((T, K), np.uint16))
        only = oracle.grouped_block_gemm(zq, zs, Wq, Ws, idx, ew, cnt, topk, mul, bias=bias)
        want = bias[flat_e] * (flat_w[:, None] if mul else np.float32(1.0))
        assert np.array_equal(only, oracle.f32_to_bf16(want.astype(np.float32)))
        got = oracle.grouped_block_gemm(xq, xs, Wq, Ws, idx, ew, cnt, topk, mul, bias=bias)
        for pair in range(T * topk):
            e, row = flat_e[pair], pair // topk
            _, c32 = oracle.block_gemm(xq[row:row + 1], xs[row:row + 1], Wq[e], Ws[e], want_f32=True)
            c32 = c32[0] + bias[e]
            if mul:
                c32 = c32 * flat_w[pair]
            assert np.array_equal(got[pair], oracle.f32_to_bf16(c32.astype(np.float32)))


# ---- the steps between and after the two expert GEMMs --------------------------------------------------------
def test_silu_and_mul_special_values():
    """silu(0) = 0, silu(g) = g for large g (1 + exp(-g) rounds to 1), silu(g) = -0 for g << 0, silu(1) known."""
    H2 = 8
    gate = torch.tensor([0.0, 20.0, 64.0, -100.0, 1.0, -1.0, 3.0, 88.0]).to(torch.bfloat16)
    up = torch.tensor([3.0, 0.5, -2.0, 7.0, 1.0, 1.0, 1.0, 1.0]).to(torch.bfloat16)
    x = torch.cat([gate, up]).reshape(1, 2 * H2)
    got = tr.bf16_from_bits(oracle.silu_and_mul(tr.bits_of(x))).float().reshape(-1)
    assert got[0] == 0.0 and got[1] == 10.0 and got[2] == -128.0 and got[3] == 0.0
    # silu(1) = 0.7310585..., silu(-1) = -0.2689414..., silu(3) = 2.8577223...: rounded to bf16
    for i, v in ((4, 0.7310585786300049), (5, -0.2689414213699951), (6, 2.857722300624436)):
        assert got[i] == torch.tensor(v).to(torch.bfloat16).float()
    assert got[7] == 88.0


def test_silu_and_mul_matches_torch_float64_rounding():
    """Against silu evaluated in float64 and rounded once to fp32 then bf16: the oracle's fp32 evaluation may
    differ by an fp32 ulp before the bf16 rounding, which flips at most a handful of bf16 results by one ulp."""
    x = H.activations(64, 1024, seed=70)
    x = (x.float() * 3).to(torch.bfloat16)
    g, u = x[:, :512].double(), x[:, 512:]
    a = (g / (1 + torch.exp(-g))).float().to(torch.bfloat16)
    want = tr.bits_of((a.float() * u.float()).to(torch.bfloat16)).astype(np.int32)
    got = oracle.silu_and_mul(tr.bits_of(x)).astype(np.int32)
    diff = np.abs(got - want)
    assert diff.max() <= 1 or np.all((got[diff > 1] & 0x7fff) < 0x80)   # beyond one ulp only between tiny values
    assert (diff != 0).mean() < 1e-3


@pytest.mark.parametrize("layout", ["blocked", "interleaved"])
@pytest.mark.parametrize("limit,alpha", [(None, None), (7.0, 1.702), (3.3, 1.0)])
def test_silu_and_mul_other_forms_match_float64(layout, limit, alpha):
    """The interleaved layout and the limit/alpha form (moe_silu_and_mul.py:46-71), against float64 with the same
    rounding points: gate to bf16, up + 1 to bf16, product to bf16; the clamp bound of `up` is limit rounded to bf16
    (3.3 is not a bf16 value).  The reference holds no vectors for these forms."""
    x = (H.activations(48, 512, seed=71).float() * 4).to(torch.bfloat16)
    xin = x if layout == "blocked" else torch.stack([x[:, :256], x[:, 256:]], dim=-1).reshape(48, 512).contiguous()
    g, u = x[:, :256].double(), x[:, 256:].double()
    if limit is None:
        a = (g / (1 + torch.exp(-g))).float().to(torch.bfloat16)
        want = (a.float() * u.float()).to(torch.bfloat16)
    else:
        lb = float(torch.tensor(limit).to(torch.bfloat16))
        g = g.clamp(max=float(np.float32(limit)))
        u = u.clamp(-lb, lb)
        a = ((1.0 / (1.0 + torch.exp(-(g.float() * np.float32(alpha)).double()))) * g).float().to(torch.bfloat16)
        want = ((u + 1.0).float().to(torch.bfloat16).float() * a.float()).to(torch.bfloat16)
    got = oracle.silu_and_mul_ex(tr.bits_of(xin), layout, limit, alpha).astype(np.int32)
    wantb = tr.bits_of(want).astype(np.int32)
    diff = np.abs(got - wantb)
    assert diff.max() <= 1 or np.all((got[diff > 1] & 0x7fff) < 0x80)
    assert (diff != 0).mean() < 2e-3
    if limit is None and layout == "blocked":
        assert np.array_equal(got, oracle.silu_and_mul(tr.bits_of(x)).astype(np.int32))
    if limit is not None:   # the clamp is active and visible
        big = torch.full((1, 4), 100.0).to(torch.bfloat16)
        pair = big if layout == "blocked" else big
        out = tr.bf16_from_bits(oracle.silu_and_mul_ex(tr.bits_of(pair), layout, limit, alpha)).float()
        lbv = float(torch.tensor(limit).to(torch.bfloat16))
        gate = float(np.float32(limit)) / (1.0 + np.exp(-float(np.float32(limit)) * alpha))
        assert torch.allclose(out, torch.full_like(out, (lbv + 1.0) * gate), rtol=2e-2)


def test_moe_sum_reduce_exact_and_ordered():
    # integers: every partial sum is exact, any order gives the same answer
    g = H.gen(71)
    y = torch.randint(-64, 64, (6, 8, 128), generator=g).to(torch.bfloat16)
    got = tr.bf16_from_bits(oracle.moe_sum_reduce(tr.bits_of(y)))
    assert torch.equal(got, y.float().sum(1).to(torch.bfloat16))
    # order matters in fp32: 2^24 + 1 - 2^24 summed left to right is 0, not 1
    z = torch.zeros((1, 3, 8), dtype=torch.float32)
    z[0, 0], z[0, 1], z[0, 2] = 2.0 ** 24, 1.0, -(2.0 ** 24)
    got = tr.bf16_from_bits(oracle.moe_sum_reduce(tr.bits_of(z.to(torch.bfloat16))))
    assert torch.all(got.float() == 0.0)
    # torch closed form
    y = H.activations(6 * 4, 128, seed=71).reshape(6, 4, 128)
    want = y[:, 0].float()
    for k in range(1, 4):
        want = want + y[:, k].float()
    got = tr.bf16_from_bits(oracle.moe_sum_reduce(tr.bits_of(y)))
    assert torch.equal(got, want.to(torch.bfloat16))


def test_block_weight_dequant_closed_form_and_round_trip():
    w = H.weights(200, 300, seed=72)
    q, s = tr.block_weight_quant(w)
    want = (q.float() * s.repeat_interleave(128, 0)[:200].repeat_interleave(128, 1)[:, :300]).to(torch.bfloat16)
    got = tr.bf16_from_bits(oracle.block_weight_dequant(tr.bits_of(q), s.numpy()))
    assert torch.equal(got, want)
    # inverse of the quantizer up to the e4m3 step (2^-4 relative, half of it after rounding) plus the bf16 step
    rel = (got.float() - w.float()).abs() / w.float().abs().clamp_min(1e-3)
    assert rel.max() < 0.07


def test_fused_experts_composition_against_dense_float():
    """The oracle's routed-expert FFN against the plain per-token loop over dequantized weights in fp32
    (the structure of fused_experts_impl_ref, unit_tests/common/fused_moe/test_deepep.py:59-140)."""
    T, Hd, I, E, topk = 12, 256, 128, 6, 2
    x = H.activations(T, Hd, seed=73)
    w1 = H.weights(E * 2 * I, Hd, seed=74).reshape(E, 2 * I, Hd)
    w2 = H.weights(E * Hd, I, seed=75).reshape(E, Hd, I)
    q1 = [tr.block_weight_quant(w1[e]) for e in range(E)]
    q2 = [tr.block_weight_quant(w2[e]) for e in range(E)]
    ids, tw = H.routing(T, E, topk, seed=76)
    out = oracle.fused_experts(
        tr.bits_of(x), np.stack([tr.bits_of(q) for q, _ in q1]), np.stack([s.numpy() for _, s in q1]),
        np.stack([tr.bits_of(q) for q, _ in q2]), np.stack([s.numpy() for _, s in q2]), ids.numpy(), tw.numpy())
    got = tr.bf16_from_bits(out).float()
    want = torch.zeros((T, Hd))
    for t in range(T):
        for k in range(topk):
            e = int(ids[t, k])
            d1, d2 = tr.dequant(*q1[e], 128, 128), tr.dequant(*q2[e], 128, 128)
            h = x[t].float() @ d1.T
            a = torch.nn.functional.silu(h[:I]) * h[I:]
            want[t] += tw[t, k] * (a @ d2.T)
    assert tr.cosine(got, want) > 0.999
    assert (got - want).abs().max() / want.abs().max() < 0.05


# ---- activation quantizer: other input dtypes, non-finite groups ---------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_group_quant_f32_entry_equals_torch_closed_form(dtype):
    """The reference widens any input to fp32 first (fp8act_quant_kernel.py:52); torch's closed form does the same."""
    g = H.gen(91)
    x = (torch.randn((48, 1024), generator=g) * torch.exp2(torch.randint(-12, 12, (48, 8, 1), generator=g).float())
         .repeat_interleave(128, -1).reshape(48, 1024)).to(dtype)
    x[5] = 0.0
    q_t, s_t = tr.group_quant(x)
    q_c, s_c = oracle.group_quant_fp8_f32(x.float().numpy())
    assert np.array_equal(tr.bits_of(s_t), s_c.view(np.uint32))
    assert np.array_equal(tr.bits_of(q_t), q_c)
    if dtype == torch.bfloat16:
        q_b, s_b = oracle.group_quant_fp8(tr.bits_of(x))
        assert np.array_equal(q_b, q_c) and np.array_equal(s_b.view(np.uint32), s_c.view(np.uint32))


def test_group_quant_non_finite_groups_follow_the_stated_rule():
    """Outside the reference's contract.  The rule of this build: a group holding NaN or +-Inf gets scale NaN and
    bytes 0x7F | sign; the other groups of the row are quantized as usual."""
    x = H.activations(4, 384, seed=92).float()
    clean_q, clean_s = oracle.group_quant_fp8_f32(x.numpy())
    x[0, 3] = float("nan")
    x[1, 200] = float("inf")
    x[2, 383] = float("-inf")
    q, s = oracle.group_quant_fp8_f32(x.numpy())
    su = s.view(np.uint32)
    assert su[0, 0] == 0x7FC00000 and su[1, 1] == 0x7FC00000 and su[2, 2] == 0x7FC00000
    neg = (x.numpy().view(np.uint32) >> 31).astype(np.uint8)
    for (r, g) in [(0, 0), (1, 1), (2, 2)]:
        sl = slice(128 * g, 128 * g + 128)
        assert np.array_equal(q[r, sl], 0x7F | (neg[r, sl] << 7))
    keep = np.ones((4, 3), bool)
    keep[0, 0] = keep[1, 1] = keep[2, 2] = False
    assert np.array_equal(su[keep], clean_s.view(np.uint32)[keep])
    assert np.array_equal(q.reshape(4, 3, 128)[keep], clean_q.reshape(4, 3, 128)[keep])
    assert np.array_equal(q[3], clean_q[3])


def test_fused_experts_composition_is_exact_when_every_step_is():
    """Integer payloads and power-of-two scales make both GEMMs exact, so the only inexact steps left are the
    SiLU (checked value by value against float64 here) and the group quantizer of its output (torch's closed
    form).  A float64 evaluation with the reference's rounding points
    (fused_moe/grouped_fused_moe.py:1048-1113: bf16 after each GEMM and after silu_and_mul, fp32 sum over the
    slots in ascending order) must then equal the oracle bit for bit."""
    T, Hd, I, E, topk = 10, 256, 256, 5, 2
    g = H.gen(93)
    # activations: small integers, one 448 per group so that every activation scale is exactly 1
    x = torch.randint(-2, 3, (T, Hd), generator=g).float()
    x[:, ::128] = 448.0
    x_b = x.to(torch.bfloat16)
    xq_t, xs_t = tr.group_quant(x_b)
    assert torch.all(xs_t == 1.0) and torch.equal(xq_t.float(), x)
    # weights: sparse {-1, 0, 1} payloads (zero against the 448 columns), power-of-two block scales
    def payload(*shape):
        w = torch.randint(-1, 2, shape, generator=g).float() * (torch.rand(shape, generator=g) < 0.25)
        return w
    w1 = payload(E, 2 * I, Hd)
    w1[:, :, ::128] = 0.0
    w2 = payload(E, Hd, I)
    w1_s = torch.exp2(torch.randint(-2, 2, (E, 2 * I // 128, Hd // 128), generator=g).float())
    w2_s = torch.exp2(torch.randint(-3, 1, (E, Hd // 128, I // 128), generator=g).float())
    w1_q, w2_q = w1.to(torch.float8_e4m3fn), w2.to(torch.float8_e4m3fn)
    ids, tw = H.routing(T, E, topk, seed=94)
    # routed weights with few mantissa bits keep the last product exact enough to be rounded once
    tw = (tw * 16).round().clamp_min(1) / 16

    out = oracle.fused_experts(tr.bits_of(x_b), tr.bits_of(w1_q), w1_s.numpy(), tr.bits_of(w2_q), w2_s.numpy(),
                               ids.numpy(), tw.numpy())
    got = tr.bf16_from_bits(out)

    d1 = (w1.double().reshape(E, 2 * I // 128, 128, Hd // 128, 128) * w1_s.double()[:, :, None, :, None]).reshape(E, 2 * I, Hd)
    slots = torch.zeros((T, topk, Hd), dtype=torch.bfloat16)
    seen_gate = set()
    for t in range(T):
        for k in range(topk):
            e = int(ids[t, k])
            h1 = (d1[e] @ x.double()[t])                      # exact: integers times powers of two
            h1_b = h1.to(torch.bfloat16)
            assert torch.equal(h1_b.double(), h1), "first GEMM must be exact in bf16 for this test"
            gate, up = h1_b[:I].double(), h1_b[I:].double()
            seen_gate.update(gate.tolist())
            act = ((gate / (1.0 + torch.exp(-gate))).to(torch.bfloat16).double() * up).to(torch.bfloat16)
            aq, asc = tr.group_quant(act.reshape(1, I))
            acc = torch.zeros(Hd, dtype=torch.float64)
            for kb in range(I // 128):
                dot = w2[e][:, 128 * kb:128 * kb + 128].double() @ aq[0, 128 * kb:128 * kb + 128].double()
                acc = (acc.float() + (dot * asc[0, kb].double()).float() *
                       w2_s[e, :, kb].repeat_interleave(128).float()).double()   # fp32 running sum per block
            slots[t, k] = (acc.float() * tw[t, k]).to(torch.bfloat16)
    # the oracle's SiLU (libm expf in fp32) against float64 on every gate value that occurred
    gv = torch.tensor(sorted(seen_gate), dtype=torch.float64)
    pair = torch.stack([gv, torch.ones_like(gv)], 0).reshape(1, -1).to(torch.bfloat16)   # [gate | up = 1]
    silu_c = tr.bf16_from_bits(oracle.silu_and_mul(tr.bits_of(pair.reshape(1, 2 * gv.numel()))))
    assert torch.equal(silu_c[0].double(), (gv / (1.0 + torch.exp(-gv))).to(torch.bfloat16).double())
    want = slots.float().sum(dim=1) if topk == 1 else None
    acc = torch.zeros((T, Hd), dtype=torch.float32)
    for k in range(topk):
        acc += slots[:, k].float()
    want = acc.to(torch.bfloat16)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


# ---- the two-step routing tables (moe_align, moe_align1) ------------------------------------------------------
MOE_ALIGN_IDS = [[0, 1, 2], [0, 3, 1], [3, 1, 4]]
MOE_ALIGN_GOLD = [  # unit_tests/common/fused_moe/test_grouped_fused_moe.py:26-47
    [1, 0, 0, 1, 0, 0, 0, 0, 0],
    [0, 1, 0, 0, 0, 1, 0, 1, 0],
    [0, 0, 1, 0, 0, 0, 0, 0, 0],
    [0, 0, 0, 0, 1, 0, 1, 0, 0],
    [0, 0, 0, 0, 0, 0, 0, 0, 1],
]
MOE_ALIGN1_INFO = [[1, 0, 0, 0], [0, 1, 1, 0], [0, 0, 0, 1], [0, 0, 0, 0]]
MOE_ALIGN1_W = [[0.3, 0.7], [0.2, 0.8]]
MOE_ALIGN1_GOLD_INFO = [[0, 0, 0, 0], [1, 2, 1, 0], [3, 0, 0, 1], [0, 0, 0, 0]]   # same file :50-77
MOE_ALIGN1_GOLD_W = [[0.3, 0, 0, 0], [0.7, 0.2, 0, 0], [0.8, 0, 0, 0], [0, 0, 0, 0]]
MOE_ALIGN1_GOLD_CNT = [1, 2, 1, 0]


def test_moe_align_reference_golden():
    out = oracle.moe_align(np.array(MOE_ALIGN_IDS, np.int32), 5)
    assert out.tolist() == MOE_ALIGN_GOLD


def test_moe_align1_reference_golden():
    info, w, cnt = oracle.moe_align1(MOE_ALIGN1_INFO, MOE_ALIGN1_W, np.zeros((4, 4), np.float32))
    assert info.tolist() == MOE_ALIGN1_GOLD_INFO
    assert cnt.tolist() == MOE_ALIGN1_GOLD_CNT
    assert np.allclose(w, np.array(MOE_ALIGN1_GOLD_W, np.float32))


def test_moe_align_then_align1_equals_the_fused_form():
    ids, tw = H.routing(300, 12, 4, seed=95)
    mask = oracle.moe_align(ids.numpy(), 12)
    info, w, cnt = oracle.moe_align1(mask, tw.numpy(), np.zeros(mask.shape, np.float32))
    idx_f, w_f, cnt_f = oracle.moe_align_fused(ids.numpy(), tw.numpy(), 12)
    assert np.array_equal(cnt, cnt_f)
    for e in range(12):
        assert np.array_equal(info[e, :cnt[e]], idx_f[e, :cnt[e]]) and np.array_equal(w[e, :cnt[e]], w_f[e, :cnt[e]])

"""GPU parity of the element-wise MoE steps (silu_and_mul, fused silu+quant, moe_sum_reduce, weight_dequant)
against the CPU oracle.

Integer/byte bars: moe_sum_reduce and weight_dequant are bit-exact; the fused silu+quant kernel is bit-exact
against the GPU's own silu_and_mul followed by the oracle quantizer.  silu_and_mul itself goes through exp() and a
division: the kernel and the oracle may differ by an fp32 ulp or two before the first bf16 rounding, so the bar there
is "fewer than 0.1 % of the elements differ from the oracle, and each of those is what the reference's own sequence
gives when bf16(silu(gate)) lands on the neighbouring bf16 value" - the product with `up` and its rounding are exact
in both (tiny magnitudes below 2^-100 are compared by value).
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _silu_close(got_bits: np.ndarray, want_bits: np.ndarray, x: torch.Tensor = None):
    """`x` (bf16 [M, 2H] = [gate | up], the blocked plain form): elements that differ from the oracle must equal
    bf16(a' * up) for a' one bf16 step beside the oracle's a = bf16(silu(gate)).  Without `x` (the other forms):
    at most one bf16 step apart."""
    got, want = got_bits.astype(np.int32), want_bits.astype(np.int32)
    diff = np.abs(got - want)
    tiny = ((got & 0x7FFF) < 0x0D80) & ((want & 0x7FFF) < 0x0D80)   # both |v| < 2^-100
    frac = float((diff != 0).mean())
    assert frac < 1e-3, f"{frac:.2e} of the elements differ"
    if x is None:
        assert np.all((diff <= 1) | tiny), f"max bf16 distance {diff[~tiny].max()}"
        return
    Hh = x.shape[1] // 2
    g, u = x[:, :Hh].double(), x[:, Hh:].float()
    a = (g / (1.0 + torch.exp(-g))).to(torch.bfloat16)
    a_bits = a.view(torch.int16).to(torch.int32)
    ok = torch.from_numpy((diff == 0) | tiny)
    for step in (-1, 1):
        beside = (a_bits + step).to(torch.int16).view(torch.bfloat16)
        cand = (beside.float() * u).to(torch.bfloat16).view(torch.int16).to(torch.int32)
        ok |= cand == torch.from_numpy(got).to(torch.int32).reshape(cand.shape).to(torch.int16).to(torch.int32)
    assert bool(ok.all()), f"{int((~ok).sum())} elements are not explained by a neighbouring bf16(silu(gate))"


@pytest.mark.parametrize("M,Hh", [(1, 128), (7, 2048), (64, 1024), (300, 1408), (33, 100), (5, 7)])
def test_silu_and_mul(hip, M, Hh):
    from lightllm_amd.fused_moe import silu_and_mul_fwd

    print(f"silu_and_mul M={M} H={Hh}", flush=True)
    x = (H.activations(M, 2 * Hh, seed=M + Hh).float() * 3).to(torch.bfloat16)
    out = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x.cuda(), out)
    torch.cuda.synchronize()
    _silu_close(tr.bits_of(out), oracle.silu_and_mul(tr.bits_of(x)), x)


def test_silu_and_mul_extremes_and_strided_input(hip):
    from lightllm_amd.fused_moe import silu_and_mul_fwd

    print("silu_and_mul extremes", flush=True)
    g = H.gen(3)
    M, Hh = 64, 256
    expo = torch.randint(-20, 8, (M, 2 * Hh), generator=g).float()
    x = (torch.randn((M, 2 * Hh), generator=g) * torch.exp2(expo)).to(torch.bfloat16)
    x[0, :8] = torch.tensor([0.0, -0.0, 200.0, -200.0, 88.0, -88.0, 1e-30, -1e30]).to(torch.bfloat16)
    wide = torch.zeros((M, 2 * Hh + 64), dtype=torch.bfloat16)
    wide[:, : 2 * Hh] = x
    xin = wide.cuda()[:, : 2 * Hh]          # row stride 2H + 64
    out = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(xin, out)
    torch.cuda.synchronize()
    _silu_close(tr.bits_of(out), oracle.silu_and_mul(tr.bits_of(x)), x)
    assert torch.isfinite(out.float()).all()


def test_silu_and_mul_non_finite_gates(hip):
    """gate / (1 + exp(-gate)) of the reference (moe_silu_and_mul.py:33-38): a NaN gate and a -inf gate (-inf / inf)
    give NaN, a +inf gate gives +inf; products with an infinite or NaN up follow IEEE.  Same NaN positions and the
    same infinities as the oracle; the other elements as in every other test."""
    from lightllm_amd.fused_moe import silu_and_mul_fwd

    print("silu_and_mul non-finite", flush=True)
    M, Hh = 4, 256
    x = H.activations(M, 2 * Hh, seed=99).clone()
    x[0, 3] = float("nan")
    x[0, 40] = float("-inf")
    x[1, 7] = float("inf")
    x[1, 8] = float("inf")
    x[1, Hh + 8] = -1.5               # +inf gate times a negative up
    x[2, Hh + 100] = float("inf")     # finite gate, infinite up
    x[3, Hh + 5] = float("nan")
    out = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x.cuda(), out)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    want = tr.bf16_from_bits(oracle.silu_and_mul(tr.bits_of(x))).float().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.isnan(want).sum() >= 3
    assert np.array_equal(np.isinf(got), np.isinf(want)) and np.isinf(want).sum() >= 3
    assert np.array_equal(got[np.isinf(want)], want[np.isinf(want)])
    fin = np.isfinite(want)
    assert np.abs(got[fin] - want[fin]).max() <= 2 ** -7 * np.abs(want[fin]).max()


@pytest.mark.parametrize("layout", ["blocked", "interleaved"])
@pytest.mark.parametrize("limit,alpha", [(None, None), (7.0, 1.702), (3.3, 1.0)])
@pytest.mark.parametrize("M,Hh", [(5, 72), (300, 1024)])
def test_silu_and_mul_other_forms(hip, layout, limit, alpha, M, Hh):
    """The interleaved layout and the clamped limit/alpha form against the oracle's restatement of
    moe_silu_and_mul.py:46-71 (the reference holds no vectors for them): within one bf16 ulp on a few elements."""
    from lightllm_amd.fused_moe import silu_and_mul_fwd

    print(f"silu_and_mul layout={layout} limit={limit} alpha={alpha} M={M} H={Hh}", flush=True)
    x = (H.activations(M, 2 * Hh, seed=M + Hh + 1).float() * 4).to(torch.bfloat16)
    out = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x.cuda(), out, layout=layout, limit=limit, alpha=alpha)
    torch.cuda.synchronize()
    _silu_close(tr.bits_of(out), oracle.silu_and_mul_ex(tr.bits_of(x), layout, limit, alpha))


def test_silu_and_mul_argument_checks(hip):
    from lightllm_amd.fused_moe import silu_and_mul_fwd

    x = torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda")
    out = torch.empty((4, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        silu_and_mul_fwd(x, out, layout="rowwise")
    with pytest.raises(AssertionError):
        silu_and_mul_fwd(x, out, limit=7.0)


@pytest.mark.parametrize("M,Hh", [(1, 128), (9, 256), (64, 2048), (777, 1024)])
def test_fused_silu_quant_equals_two_steps(hip, M, Hh):
    from lightllm_amd.fused_moe import silu_and_mul_fwd, silu_and_mul_post_quant_fwd

    print(f"silu+quant M={M} H={Hh}", flush=True)
    x = (H.activations(M, 2 * Hh, seed=5 * M + Hh, outliers=True).float() * 2).to(torch.bfloat16).cuda()
    mid = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x, mid)
    q = torch.empty((M, Hh), dtype=torch.float8_e4m3fn, device="cuda")
    s = torch.empty((M, Hh // 128), dtype=torch.float32, device="cuda")
    silu_and_mul_post_quant_fwd(x, q, s)
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(mid))
    assert np.array_equal(tr.bits_of(s), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(q), q_ref)
    # and against the oracle end to end, in value: scales within an fp32-of-bf16 ulp, dequantized within an e4m3 step
    q_o, s_o = oracle.silu_and_mul_group_quant(tr.bits_of(x))
    assert np.allclose(s.cpu().numpy(), s_o, rtol=2 ** -7, atol=0)
    dq = tr.fp8_from_bits(q_o).float() * torch.from_numpy(s_o).repeat_interleave(128, 1)
    got = q.float().cpu() * s.cpu().repeat_interleave(128, 1)
    assert (got - dq).abs().max() <= 0.07 * dq.abs().max()


def test_fused_silu_quant_non_finite_products(hip):
    """A SiLU product that is NaN or infinite poisons its own 128-element group only, exactly as the stand-alone
    quantizer does with the bf16 products of silu_and_mul (scale = quiet NaN, bytes = e4m3fn NaN with the sign)."""
    from lightllm_amd.fused_moe import silu_and_mul_fwd, silu_and_mul_post_quant_fwd

    print("silu+quant non-finite", flush=True)
    M, Hh = 6, 512
    x = H.activations(M, 2 * Hh, seed=77).clone()
    x[1, 5] = float("inf")            # gate +inf: silu = inf, product inf * up
    x[2, 130] = float("nan")          # gate NaN
    x[3, Hh + 300] = float("-inf")    # up -inf
    x[4, 400] = float("-inf")         # gate -inf: silu = -0 * ... (NaN with a finite up only through 0 * inf)
    x = x.cuda()
    mid = torch.empty((M, Hh), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x, mid)
    q = torch.empty((M, Hh), dtype=torch.float8_e4m3fn, device="cuda")
    s = torch.empty((M, Hh // 128), dtype=torch.float32, device="cuda")
    silu_and_mul_post_quant_fwd(x, q, s)
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(mid))
    assert np.array_equal(tr.bits_of(s), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(q), q_ref)
    bad = ~torch.isfinite(mid.float()).cpu().numpy().reshape(M, Hh // 128, 128).all(axis=2)
    assert bad.sum() >= 4 and np.array_equal(np.isnan(s.cpu().numpy()), bad)


def test_fused_silu_quant_column_major_scales(hip):
    from lightllm_amd.fused_moe import silu_and_mul_post_quant_fwd

    print("silu+quant column-major scales", flush=True)
    M, Hh = 40, 512
    x = H.activations(M, 2 * Hh, seed=11).cuda()
    q = torch.empty((M, Hh), dtype=torch.float8_e4m3fn, device="cuda")
    s_rm = torch.empty((M, Hh // 128), dtype=torch.float32, device="cuda")
    s_cm = torch.empty((Hh // 128, M), dtype=torch.float32, device="cuda").t()
    silu_and_mul_post_quant_fwd(x, q, s_rm)
    q2 = torch.empty_like(q)
    silu_and_mul_post_quant_fwd(x, q2, s_cm)
    torch.cuda.synchronize()
    assert torch.equal(s_rm, s_cm.contiguous()) and torch.equal(q.view(torch.uint8), q2.view(torch.uint8))


@pytest.mark.parametrize("E,T,hidden", [(3, 1, 256), (4, 5, 512), (5, 3, 2048), (2, 64, 1024)])
def test_masked_post_quant(hip, E, T, hidden):
    """Shapes of the reference's test (unit_tests/common/fused_moe/test_moe_silu_and_mul_mix_quant_ep.py:26-78)."""
    from lightllm_amd.fused_moe import silu_and_mul_fwd, silu_and_mul_masked_post_quant_fwd

    print(f"masked silu+quant E={E} T={T} hidden={hidden}", flush=True)
    x = H.activations(E * T, hidden, seed=E * 100 + T).reshape(E, T, hidden).cuda()
    out = torch.empty((E, T, hidden // 2), dtype=torch.float8_e4m3fn, device="cuda")
    sc = torch.empty((E, T, hidden // 2 // 128), dtype=torch.float32, device="cuda")
    masked_m = torch.full((E,), T, dtype=torch.int32, device="cuda")
    silu_and_mul_masked_post_quant_fwd(x, out, sc, 128, masked_m)
    mid = torch.empty((E * T, hidden // 2), dtype=torch.bfloat16, device="cuda")
    silu_and_mul_fwd(x.view(-1, hidden), mid)
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(mid))
    assert np.array_equal(tr.bits_of(out).reshape(E * T, -1), q_ref)
    assert np.array_equal(tr.bits_of(sc).reshape(E * T, -1), s_ref.view(np.uint32))


def test_masked_post_quant_skips_padded_rows(hip):
    """The reference's second test (same file :81-108): rows at or past masked_m[e] stay as they were."""
    from lightllm_amd.fused_moe import silu_and_mul_masked_post_quant_fwd

    print("masked silu+quant padded rows", flush=True)
    E, T, hidden = 3, 4, 256
    masked = [0, 2, T]
    masked_m = torch.tensor(masked, dtype=torch.int32, device="cuda")
    x = H.activations(E * T, hidden, seed=9).reshape(E, T, hidden).cuda()
    out = torch.empty((E, T, hidden // 2), dtype=torch.float8_e4m3fn, device="cuda")
    sc = torch.empty((E, T, 1), dtype=torch.float32, device="cuda")
    out.fill_(1.0)
    sc.fill_(7.0)
    silu_and_mul_masked_post_quant_fwd(x, out, sc, 128, masked_m)
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.silu_and_mul_group_quant(tr.bits_of(x.view(-1, hidden)))
    for e, n in enumerate(masked):
        assert torch.equal(out[e, n:].float(), torch.ones_like(out[e, n:], dtype=torch.float32))
        assert torch.equal(sc[e, n:], torch.full_like(sc[e, n:], 7.0))
        if n:
            assert np.allclose(sc[e, :n].cpu().numpy().reshape(n, 1), s_ref[e * T: e * T + n], rtol=2 ** -7)


@pytest.mark.parametrize("T,topk,Hd", [(1, 1, 128), (6, 4, 128), (33, 8, 7168), (17, 6, 2048), (5, 3, 100), (9, 2, 7)])
def test_moe_sum_reduce_bit_exact(hip, T, topk, Hd):
    from lightllm_amd.fused_moe import moe_sum_reduce

    print(f"moe_sum_reduce T={T} topk={topk} H={Hd}", flush=True)
    x = H.activations(T * topk, Hd, seed=T + topk + Hd, outliers=True).reshape(T, topk, Hd)
    out = torch.empty((T, Hd), dtype=torch.bfloat16, device="cuda")
    moe_sum_reduce(x.cuda(), out)
    torch.cuda.synchronize()
    assert np.array_equal(tr.bits_of(out), oracle.moe_sum_reduce(tr.bits_of(x)))


@pytest.mark.parametrize("N,K", [(128, 128), (256, 512), (200, 304), (130, 100), (576, 7168)])
def test_weight_dequant_bit_exact(hip, N, K):
    from lightllm_amd.quantization import weight_dequant

    print(f"weight_dequant N={N} K={K}", flush=True)
    q, s = H.quantized_weights(N, K, seed=N + K)
    y = weight_dequant(q.cuda(), s.cuda())
    torch.cuda.synchronize()
    assert y.dtype == torch.bfloat16 and y.shape == (N, K)
    assert np.array_equal(tr.bits_of(y), oracle.block_weight_dequant(tr.bits_of(q), s.numpy()))


def test_weight_dequant_every_byte(hip):
    """All 256 e4m3fn bytes (NaN codes included) times a few scales."""
    from lightllm_amd.quantization import weight_dequant

    print("weight_dequant all bytes", flush=True)
    q = torch.arange(256, dtype=torch.uint8).repeat(128, 1).contiguous()      # [128, 256] -> two scale blocks
    s = torch.tensor([[0.0123, 3.5e-5]], dtype=torch.float32)
    y = weight_dequant(q.view(torch.float8_e4m3fn).cuda(), s.cuda())
    torch.cuda.synchronize()
    got, want = tr.bits_of(y), oracle.block_weight_dequant(q.numpy(), s.numpy())
    nan = (want & 0x7FFF) > 0x7F80
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7FFF) > 0x7F80)

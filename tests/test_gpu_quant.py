"""GPU parity of per_token_group_quant_fp8 against the CPU oracle: bytes and scale bits must be identical."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _run(x: torch.Tensor, **kw):
    from lightllm_amd.quantization import per_token_group_quant_fp8

    xq, xs = per_token_group_quant_fp8(x.cuda(), 128, **kw)
    torch.cuda.synchronize()
    return xq, xs


def _check(x: torch.Tensor, xq, xs):
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(x))
    q = tr.bits_of(xq)
    s = tr.bits_of(xs.contiguous())
    nq = int((q != q_ref).sum())
    ns = int((s != s_ref.view(np.uint32)).sum())
    assert ns == 0, f"{ns} scale words differ"
    assert nq == 0, f"{nq} of {q.size} fp8 bytes differ"


@pytest.mark.parametrize("M,K", [(1, 128), (1, 4096), (8, 4096), (32, 4096), (64, 14336), (257, 7168), (33, 384), (4096, 2048)])
def test_bit_exact_normal(hip, M, K):
    print(f"quant M={M} K={K}", flush=True)
    x = H.activations(M, K, seed=M * 131 + K)
    _check(x, *_run(x))


def test_bit_exact_outliers_zero_row(hip):
    print("quant outliers 2048x7168", flush=True)
    x = H.activations(2048, 7168, seed=4, outliers=True, zero_row=True)
    xq, xs = _run(x)
    _check(x, xq, xs)
    # the all-zero row: eps floor -> scale bits of fp32(1e-10)/448, all bytes zero
    assert np.all(tr.bits_of(xs[0].contiguous()) == 0x2A7B5123)
    assert np.all(tr.bits_of(xq[0].contiguous()) == 0)


def test_wide_dynamic_range(hip):
    """Groups whose magnitudes span the whole bf16 range, including subnormal inputs and values below eps."""
    print("quant dynamic range", flush=True)
    g = H.gen(7)
    M, K = 512, 1024
    expo = torch.randint(-140, 120, (M, K // 128, 1), generator=g).float()
    x = (torch.randn((M, K // 128, 128), generator=g) * torch.exp2(expo)).reshape(M, K).to(torch.bfloat16)
    _check(x, *_run(x))


def test_every_bf16_value(hip):
    """Every finite bf16 pattern as an element, against several group maxima."""
    print("quant all bf16 patterns", flush=True)
    bits = np.arange(65536, dtype=np.uint16)
    finite = bits[(bits & 0x7F80) != 0x7F80]
    vals = tr.bf16_from_bits(finite)  # 65280 values
    n = vals.numel() // 127 * 127
    rows = []
    for top in [448.0, 1.0, 3.0e38, 1e-3, 7.25, 1e-20]:
        body = vals[:n].reshape(-1, 127).clone()
        body = torch.where(body.abs().float() <= top, body, torch.zeros_like(body))
        lead = torch.full((body.shape[0], 1), top, dtype=torch.bfloat16)
        rows.append(torch.cat([lead, body], dim=1))
    x = torch.cat(rows, dim=0).contiguous()
    _check(x, *_run(x))


def test_column_major_scales(hip):
    print("quant column-major scales", flush=True)
    x = H.activations(130, 1024, seed=9)
    xq, xs = _run(x, column_major_scales=True, scale_tma_aligned=True)
    assert xs.shape == (130, 8) and xs.stride() == (1, 132)
    _check(x, xq, xs)


def test_into_caller_buffers(hip):
    from lightllm_amd.quantization import lightllm_per_token_group_quant_fp8

    x = H.activations(48, 512, seed=11).cuda()
    xq = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    xs = torch.empty((4, 48), dtype=torch.float32, device="cuda").t()  # column-major view
    assert lightllm_per_token_group_quant_fp8(x, 128, xq, xs) is None
    torch.cuda.synchronize()
    _check(x.cpu(), xq, xs)


@pytest.mark.parametrize("eps", [1e-4, 3.0, 1e-30])
def test_other_eps_through_the_caller_buffer_entry(hip, eps):
    """lightllm_per_token_group_quant_fp8 hands its eps to the kernel (fp8act_quant_kernel.py:63-113).  Any value
    other than 1e-10 takes the kernel with true divisions: groups whose amax lies below the floor (scale = eps/448,
    no bf16 value), groups above it, an all-zero group, and both scale layouts."""
    from lightllm_amd.quantization import lightllm_per_token_group_quant_fp8

    print(f"quant eps={eps}", flush=True)
    g = H.gen(17)
    M, K = 96, 1024
    expo = torch.randint(-40, 4, (M, K // 128, 1), generator=g).float()
    x = (torch.randn((M, K // 128, 128), generator=g) * torch.exp2(expo)).reshape(M, K)
    x[3, 128:256] = 0.0
    x = x.to(torch.bfloat16)
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(x), 128, eps)
    below = int((s_ref == np.float32(eps) / np.float32(448.0)).sum())
    if eps >= 1e-4:
        assert 0 < below, "the case must hold groups below the floor"
    if eps == 1e-4:
        assert below < s_ref.size, "and groups above it"
    for col_major in (False, True):
        xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device="cuda")
        xs = torch.empty((K // 128, M), dtype=torch.float32, device="cuda").t() if col_major else \
            torch.empty((M, K // 128), dtype=torch.float32, device="cuda")
        lightllm_per_token_group_quant_fp8(x.cuda(), 128, xq, xs, eps=eps)
        torch.cuda.synchronize()
        assert np.array_equal(tr.bits_of(xq), q_ref)
        assert np.array_equal(tr.bits_of(xs.contiguous()), s_ref.view(np.uint32))


def test_full_size_properties(hip):
    """The bandwidth config [16384,7168] with outliers and a zero row: bit-exact on a row sample, and
    size-independent properties on the whole tensor."""
    print("quant full size 16384x7168", flush=True)
    x = H.activations(16384, 7168, seed=0, outliers=True, zero_row=True)
    xq, xs = _run(x)
    rows = np.r_[0:64, 8000:8064, 16320:16384]
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(x)[rows])
    assert np.array_equal(tr.bits_of(xq)[rows], q_ref)
    assert np.array_equal(tr.bits_of(xs.contiguous())[rows], s_ref.view(np.uint32))
    qb = xq.view(torch.uint8)
    assert int(((qb & 0x7F) == 0x7F).sum()) == 0, "NaN code produced"
    # every non-zero group holds its maximum as +-448
    top = (qb & 0x7F).view(16384, 56, 128).amax(dim=-1)
    nonzero = x.cuda().view(16384, 56, 128).abs().amax(dim=-1) > 1e-10
    assert bool((top[nonzero] == 0x7E).all())
    # signs survive
    sign_in = x.cuda().view(torch.int16) < 0
    sign_out = (qb & 0x80) != 0
    assert bool((sign_out == sign_in).all())
    # the scale is the group amax over 448 (IEEE division, evaluated by torch on the CPU)
    amax = x.float().view(16384, 56, 128).abs().amax(dim=-1).clamp_min(1e-10)
    assert torch.equal(xs.cpu(), amax / 448.0)


def test_preconditions(hip):
    from lightllm_amd.quantization import per_token_group_quant_fp8

    with pytest.raises(AssertionError):
        per_token_group_quant_fp8(torch.zeros((4, 100), dtype=torch.bfloat16, device="cuda"), 128)
    with pytest.raises(AssertionError):
        per_token_group_quant_fp8(torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda")[:, ::2], 64)
    xq, xs = per_token_group_quant_fp8(torch.zeros((0, 256), dtype=torch.bfloat16, device="cuda"), 128)
    assert xq.shape == (0, 256) and xs.shape == (0, 2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("M,K", [(1, 128), (33, 384), (257, 7168), (64, 14336)])
def test_bit_exact_fp16_fp32_activations(hip, dtype, M, K):
    """The reference widens any input dtype to fp32 (fp8act_quant_kernel.py:52); so does the oracle."""
    print(f"quant {dtype} M={M} K={K}", flush=True)
    g = H.gen(M * 7 + K)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    x[:, ::97] *= 37.0
    if M > 1:
        x[1] = 0.0
    x = x.to(dtype)
    xq, xs = _run(x)
    q_ref, s_ref = oracle.group_quant_fp8_f32(x.float().numpy())
    assert np.array_equal(tr.bits_of(xs.contiguous()), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(xq), q_ref)


def test_fp32_wide_dynamic_range(hip):
    """fp32 groups spanning subnormals to 1e38, and values that are not bf16-representable."""
    g = H.gen(21)
    M, K = 256, 1024
    expo = torch.randint(-140, 120, (M, K // 128, 1), generator=g).float()
    x = (torch.randn((M, K // 128, 128), generator=g) * torch.exp2(expo)).reshape(M, K).contiguous()
    xq, xs = _run(x)
    q_ref, s_ref = oracle.group_quant_fp8_f32(x.numpy())
    assert np.array_equal(tr.bits_of(xs.contiguous()), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(xq), q_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_non_finite_groups_are_poisoned(hip, dtype):
    """One NaN, one +Inf and one -Inf group among finite ones: scale NaN, bytes 0x7F | sign; the finite groups
    of the same rows are untouched (the reference leaves this case undefined; the oracle states this build's rule)."""
    x = H.activations(8, 512, seed=13).float()
    x[1, 130] = float("nan")
    x[2, 5] = float("inf")
    x[3, 300] = float("-inf")
    x[4, 384] = float("nan")
    x[4, 385] = float("inf")
    x = x.to(dtype)
    xq, xs = _run(x)
    q_ref, s_ref = oracle.group_quant_fp8_f32(x.float().numpy())
    q, s = tr.bits_of(xq), tr.bits_of(xs.contiguous())
    assert np.array_equal(q, q_ref)
    assert np.array_equal(s, s_ref.view(np.uint32))
    assert s[1, 1] == 0x7FC00000 and s[2, 0] == 0x7FC00000 and s[3, 2] == 0x7FC00000 and s[4, 3] == 0x7FC00000
    assert np.all((q[1, 128:256] & 0x7F) == 0x7F) and np.all((q[1, :128] & 0x7F) != 0x7F)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M,K,group", [(7, 4096, 4096), (33, 14336, 14336), (5, 1024, 64), (9, 768, 256), (4, 120, 24),
                                       (3, 100, 100), (6, 7168, 512)])
def test_other_group_sizes(hip, dtype, M, K, group):
    """The reference's kernel takes any group size that divides K (fp8act_quant_kernel.py:18-60; its other callers
    quantize per token, group = K): bit-exact against the oracle, groups that are not a multiple of 8 elements and a
    poisoned group included; column-major scales as well."""
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"quant group={group} {dtype} M={M} K={K}", flush=True)
    g = H.gen(M + K + group)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    x[:, ::53] *= 29.0
    x[1] = 0.0
    x[2, K // 2] = float("inf")
    x = x.to(dtype)
    q_ref, s_ref = oracle.group_quant_fp8_f32(x.float().numpy(), group=group)
    xq, xs = per_token_group_quant_fp8(x.cuda(), group)
    torch.cuda.synchronize()
    assert xs.shape == (M, K // group)
    assert np.array_equal(tr.bits_of(xs.contiguous()), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(xq), q_ref)
    xq2, xs2 = per_token_group_quant_fp8(x.cuda(), group, column_major_scales=True)
    torch.cuda.synchronize()
    assert np.array_equal(tr.bits_of(xs2.contiguous()), s_ref.view(np.uint32)) and np.array_equal(tr.bits_of(xq2), q_ref)

"""GPU parity of the masked / contiguous grouped GEMM entry points (the layouts LightLLM's expert-parallel path
hands to DeepGEMM) against the per-expert dense oracle.  DeepGEMM itself is a third-party wheel that is not
part of the reference tree, so the expected values are the block-scaled GEMM oracle applied expert by expert
(the structure of fused_experts_impl_ref, unit_tests/common/fused_moe/test_deepep.py:59-140)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _weights(E, N, K, seed):
    qs = [H.quantized_weights(N, K, seed=seed + e) for e in range(E)]
    return torch.stack([q for q, _ in qs]).contiguous(), torch.stack([s for _, s in qs]).contiguous()


def _quant(x):
    q, s = oracle.group_quant_fp8(tr.bits_of(x))
    return tr.fp8_from_bits(q), torch.from_numpy(s)


def _expert_ref(xq_rows, xs_rows, wq_e, ws_e):
    bits = oracle.block_gemm(tr.bits_of(xq_rows), xs_rows.numpy(), tr.bits_of(wq_e), ws_e.numpy())
    return tr.bf16_from_bits(bits).float()


def _close(got, ref):
    cos, rel = H.gemm_metrics(got, ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


@pytest.mark.parametrize("E,T,N,K,masked", [(4, 40, 384, 512, [0, 7, 40, 33]), (3, 300, 256, 1024, [300, 1, 129])])
def test_masked_layout(hip, E, T, N, K, masked):
    from lightllm_amd.fused_moe import _deepgemm_grouped_fp8_nt_masked

    print(f"masked grouped gemm E={E} T={T} N={N} K={K}", flush=True)
    x = H.activations(E * T, K, seed=E + T)
    xq, xs = _quant(x)
    wq, ws = _weights(E, N, K, seed=T)
    out = torch.full((E, T, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    mm = torch.tensor(masked, dtype=torch.int32, device="cuda")
    _deepgemm_grouped_fp8_nt_masked((xq.view(E, T, K).cuda(), xs.view(E, T, -1).cuda()), (wq.cuda(), ws.cuda()), out,
                                    mm, max(masked))
    torch.cuda.synchronize()
    got = out.float().cpu()
    for e, n in enumerate(masked):
        assert torch.isnan(got[e, n:]).all(), "rows past masked_m must stay untouched"
        if n:
            _close(got[e, :n], _expert_ref(xq[e * T: e * T + n], xs[e * T: e * T + n], wq[e], ws[e]))


def test_contiguous_layout(hip):
    from lightllm_amd.fused_moe import deepgemm_grouped_fp8_nt_contiguous

    print("contiguous grouped gemm", flush=True)
    E, N, K = 5, 384, 512
    blocks = [2, 2, 0, -1, 4, 4, 4, 1, -1]          # expert of every 128-row block (-1 = padding block)
    m_idx = torch.tensor(blocks, dtype=torch.int32).repeat_interleave(128)
    m_idx[128 * 7 + 100:128 * 8] = -1               # a partly filled block
    rows = m_idx.numel()
    x = H.activations(rows, K, seed=31)
    xq, xs = _quant(x)
    wq, ws = _weights(E, N, K, seed=32)
    out = torch.full((rows, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    deepgemm_grouped_fp8_nt_contiguous((xq.cuda(), xs.cuda()), (wq.cuda(), ws.cuda()), out, m_idx.cuda())
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isnan(got[m_idx < 0]).all()
    for e in range(E):
        sel = torch.nonzero(m_idx == e).flatten()
        if sel.numel():
            _close(got[sel], _expert_ref(xq[sel], xs[sel], wq[e], ws[e]))


def test_masked_group_gemm_ffn(hip):
    """gate/up GEMM -> fused SiLU-mul + quant -> down GEMM on the masked layout, against the oracle's steps."""
    from lightllm_amd.fused_moe import masked_group_gemm

    print("masked_group_gemm", flush=True)
    E, T, Hd, I = 3, 24, 256, 128
    masked = [24, 0, 9]
    x = H.activations(E * T, Hd, seed=41)
    xq, xs = _quant(x)
    w1q, w1s = _weights(E, 2 * I, Hd, seed=42)
    w2q, w2s = _weights(E, Hd, I, seed=52)
    mm = torch.tensor(masked, dtype=torch.int32, device="cuda")
    out = masked_group_gemm((xq.view(E, T, Hd).cuda(), xs.view(E, T, -1).cuda()), mm, torch.bfloat16, w1q.cuda(),
                            w1s.cuda(), w2q.cuda(), w2s.cuda(), expected_m=16)
    torch.cuda.synchronize()
    assert out.shape == (E, T, Hd) and out.dtype == torch.bfloat16
    for e, n in enumerate(masked):
        if not n:
            continue
        r = slice(e * T, e * T + n)
        h1 = oracle.block_gemm(tr.bits_of(xq[r]), xs[r].numpy(), tr.bits_of(w1q[e]), w1s[e].numpy())
        aq, asc = oracle.silu_and_mul_group_quant(h1)
        ref = tr.bf16_from_bits(oracle.block_gemm(aq, asc, tr.bits_of(w2q[e]), w2s[e].numpy())).float()
        got = out[e, :n].float().cpu()
        assert tr.cosine(got, ref) >= 0.9999
        assert (got - ref).abs().max() <= 2e-2 * ref.abs().max()

"""The routed-expert configuration at its full size: 4096 tokens, top-8 of 256 experts, Zipf(1.1) routing,
gate/up GEMM N=4096 K=7168 and down GEMM N=7168 K=2048 (topk_num=1, routed weight multiplied in, input
[32768, 2048]) - the two launches of fused_experts_impl
(lightllm/common/basemodel/triton_kernel/fused_moe/grouped_fused_moe.py:1067-1112).

Every routed row of both GEMMs is compared with the torch fp32 dequant-matmul of its expert on the GPU, a sample
of entries with the float64 CPU oracle, and the whole layer with the oracle's restatement of the reference
sequence on a token subset.  Weights are quantized expert by expert, so their bf16 form never exists whole
(11.3 GB of e4m3 bytes stay resident)."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu

T, TOPK, E, HID, INTER = 4096, 8, 256, 7168, 2048


def _expert_weights(N, K, seed):
    """e4m3fn [E,N,K] + fp32 [E,N/128,K/128]: N(0,0.02) bf16 weights through the library's load-time quantizer
    (bit-exact against the oracle in test_gpu_weight_quant.py), one expert at a time."""
    from lightllm_amd.quantization import mm_weight_quant

    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(seed)
    for e in range(E):
        w = (torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32) * 0.02).to(torch.bfloat16)
        wq[e], ws[e] = mm_weight_quant(w)
    return wq, ws


@pytest.fixture(scope="module")
def routed():
    from lightllm_amd.fused_moe import moe_align_fused

    ids, tw = H.routing(T, E, TOPK, seed=5)
    P = T * TOPK
    idx = torch.empty((E, P), dtype=torch.int32, device="cuda")
    w = torch.empty((E, P), dtype=torch.float32, device="cuda")
    cnt = torch.empty((E,), dtype=torch.int32, device="cuda")
    moe_align_fused(idx, w, cnt, ids.cuda(), tw.cuda())
    torch.cuda.synchronize()
    counts = cnt.cpu().numpy()
    assert counts.sum() == P and np.array_equal(counts, np.bincount(ids.numpy().ravel(), minlength=E))
    # the shape of the raggedness this configuration is about: a few experts with thousands of rows, most small
    assert counts.max() > 2000 and (counts <= 64).sum() > 128
    return {"ids": ids, "tw": tw, "idx": idx, "w": w, "cnt": cnt, "counts": counts}


def _check_every_row(out, xq, xs, wq, ws, routed, topk_num, mul_w, rng):
    """out [P,N] against fp32 dequant-matmul per expert (all rows) and float64 oracle entries (sampled)."""
    idx_h, w_h = routed["idx"].cpu(), routed["w"].cpu()
    assert not torch.isnan(out.float()).any(), "a routed row was not written"
    worst_cos, worst_rel = 1.0, 0.0
    for e in range(E):
        n_e = int(routed["counts"][e])
        if n_e == 0:
            continue
        pairs = idx_h[e, :n_e].long().cuda()
        rows = pairs // topk_num
        ref = tr.dequant_matmul(xq[rows], xs[rows], wq[e], ws[e], out_dtype=torch.float32)
        if mul_w:
            ref = ref * w_h[e, :n_e].cuda()[:, None]
        cos, rel = H.gemm_metrics(out[pairs].float(), ref)
        worst_cos, worst_rel = min(worst_cos, cos), max(worst_rel, rel)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (e, n_e, cos, rel)
    # float64 oracle on sampled (row, column) entries of a few experts of every size class
    order = np.argsort(routed["counts"])
    for e in [int(order[-1]), int(order[len(order) // 2]), int(order[np.searchsorted(routed["counts"][order], 1)])]:
        n_e = int(routed["counts"][e])
        pick = rng.choice(n_e, size=min(n_e, 6), replace=False)
        pairs = idx_h[e, :n_e].long()[pick]
        rows = (pairs // topk_num).cuda()
        cols = np.sort(rng.choice(wq.shape[1], size=48, replace=False))
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows]), xs[rows].cpu().numpy(), tr.bits_of(wq[e]),
                                              ws[e].cpu().numpy(), np.arange(len(pick)), cols)
        if mul_w:
            ref64 = ref64 * w_h[e, :n_e].numpy()[pick][:, None].astype(np.float64)
        got = out[pairs.cuda()][:, torch.from_numpy(cols).cuda()].float().cpu().numpy()
        assert np.abs(got - ref64).max() <= 1e-2 * np.abs(ref64).max(), e
    return worst_cos, worst_rel


@pytest.mark.parametrize("block_m", [None, 64])
def test_gate_up_gemm_full_size(hip, routed, block_m):
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"routed experts gate_up full size block_m={block_m}", flush=True)
    wq, ws = _expert_weights(2 * INTER, HID, seed=11)
    x = H.activations(T, HID, seed=12).cuda()
    P = T * TOPK
    out = torch.full((P, 2 * INTER), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, x, None, routed["cnt"], routed["idx"], routed["w"], wq, ws, TOPK, out,
                   mul_routed_weight=False, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m} if block_m else None)
    torch.cuda.synchronize()
    xq, xs = per_token_group_quant_fp8(x, 128)
    cos, rel = _check_every_row(out, xq, xs, wq, ws, routed, TOPK, False, np.random.default_rng(1))
    print(f"  worst expert: cosine {cos:.6f} max-rel {rel:.2e}", flush=True)


@pytest.mark.parametrize("block_m", [None, 64])
def test_down_gemm_full_size(hip, routed, block_m):
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"routed experts down full size block_m={block_m}", flush=True)
    wq, ws = _expert_weights(HID, INTER, seed=13)
    P = T * TOPK
    act = H.activations(P, INTER, seed=14).cuda()          # stands for the quantized SiLU products
    xq, xs = per_token_group_quant_fp8(act, 128)
    out = torch.full((P, HID), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, xq, xs, routed["cnt"], routed["idx"], routed["w"], wq, ws, 1, out,
                   mul_routed_weight=True, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m} if block_m else None)
    torch.cuda.synchronize()
    cos, rel = _check_every_row(out, xq, xs, wq, ws, routed, 1, True, np.random.default_rng(2))
    print(f"  worst expert: cosine {cos:.6f} max-rel {rel:.2e}", flush=True)


def test_fused_experts_full_width(hip):
    """fused_experts_impl at H=7168, I=2048, E=256 on 512 tokens; the oracle's restatement of the reference
    sequence on 6 of those tokens (the FFN is independent per token; the experts those tokens use are compacted
    so that the CPU side holds 48 experts at most)."""
    from lightllm_amd.fused_moe import fused_experts_impl

    print("fused_experts full width", flush=True)
    tokens = 512
    w1q, w1s = _expert_weights(2 * INTER, HID, seed=21)
    w2q, w2s = _expert_weights(HID, INTER, seed=22)
    x = H.activations(tokens, HID, seed=23)
    ids, tw = H.routing(tokens, E, TOPK, seed=24)
    out = fused_experts_impl(x.cuda(), w1q, w2q, tw.cuda(), ids.cuda(), inplace=False, use_fp8_w8a8=True,
                             w1_scale=w1s, w2_scale=w2s)
    torch.cuda.synchronize()
    assert out.shape == x.shape and not torch.isnan(out.float()).any()
    sub = np.array([0, 1, 100, 255, 256, 511])
    used, inv = np.unique(ids.numpy()[sub], return_inverse=True)
    ids_sub = inv.reshape(len(sub), TOPK).astype(np.int32)
    sel = torch.from_numpy(used).long().cuda()
    want = tr.bf16_from_bits(oracle.fused_experts(
        tr.bits_of(x[sub]), tr.bits_of(w1q[sel]), w1s[sel].cpu().numpy(), tr.bits_of(w2q[sel]),
        w2s[sel].cpu().numpy(), ids_sub, tw.numpy()[sub])).float()
    got = out[torch.from_numpy(sub).cuda()].float().cpu()
    assert tr.cosine(got, want) >= 0.9999
    assert (got - want).abs().max() <= 2e-2 * want.abs().max()

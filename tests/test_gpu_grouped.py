"""GPU parity of the routing tables and the grouped (per-expert) block-FP8 GEMM."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _align(topk_ids, topk_weights, E):
    from lightllm_amd.fused_moe import moe_align_fused

    P = topk_ids.numel()
    idx = torch.full((E, P), -7, dtype=torch.int32, device="cuda")
    w = torch.full((E, P), -7.0, dtype=torch.float32, device="cuda")
    cnt = torch.empty((E,), dtype=torch.int32, device="cuda")
    moe_align_fused(idx, w, cnt, topk_ids.cuda(), topk_weights.cuda())
    torch.cuda.synchronize()
    return idx, w, cnt


def _check_align(topk_ids, topk_weights, E):
    """The reference test's bincount / nonzero oracle (unit_tests/common/fused_moe/test_grouped_fused_moe.py:80-112),
    in the ordered form, plus the C oracle for the whole table."""
    idx, w, cnt = _align(topk_ids, topk_weights, E)
    flat = topk_ids.flatten().long()
    assert torch.equal(cnt.cpu(), torch.bincount(flat, minlength=E).to(torch.int32))
    o_idx, o_w, o_cnt = oracle.moe_align_fused(topk_ids.numpy(), topk_weights.numpy(), E)
    assert np.array_equal(cnt.cpu().numpy(), o_cnt)
    idx, w = idx.cpu().numpy(), w.cpu().numpy()
    for e in range(E):
        c = o_cnt[e]
        assert np.array_equal(idx[e, :c], o_idx[e, :c])
        assert np.array_equal(w[e, :c], o_w[e, :c])
        assert np.all(idx[e, c:] == -7), "wrote past the expert's count"


def test_moe_align_fused_reference_vectors(hip):
    print("moe_align_fused", flush=True)
    ids = torch.tensor([[0, 1, 2], [0, 3, 1], [3, 1, 4]], dtype=torch.int32)
    w = torch.tensor([[0.3, 0.7, 0.1], [0.2, 0.8, 0.4], [0.5, 0.6, 0.9]], dtype=torch.float32)
    _check_align(ids, w, 5)
    ids = (torch.arange(128 * 17, dtype=torch.int32).reshape(128, 17) % 5).contiguous()
    _check_align(ids, torch.arange(ids.numel(), dtype=torch.float32).reshape(128, 17), 5)
    base = torch.tensor([[0, 1, 2], [0, 3, 1], [3, 1, 4], [2, 0, 4]], dtype=torch.int32)
    ids = base.repeat(1281, 1)[:5121].contiguous()
    _check_align(ids, torch.arange(ids.numel(), dtype=torch.float32).reshape(5121, 3), 257)
    ids = (torch.arange(5121 * 8, dtype=torch.int32).reshape(5121, 8) % 257).contiguous()
    _check_align(ids, torch.arange(ids.numel(), dtype=torch.float32).reshape(5121, 8), 257)


def test_moe_align_and_align1_reference_vectors(hip):
    """Golden vectors of the reference's test_moe_align / test_moe_align1 (test_grouped_fused_moe.py:26-77), then
    the two-step form against the oracle at sizes that span several 4096-pair steps and every padding."""
    import oracle
    from lightllm_amd.fused_moe import moe_align, moe_align1

    print("moe_align / moe_align1", flush=True)
    ids = torch.tensor([[0, 1, 2], [0, 3, 1], [3, 1, 4]], dtype=torch.int32, device="cuda")
    out = torch.full((5, 9), 7, dtype=torch.int32, device="cuda")
    moe_align(ids, out)
    assert out.cpu().tolist() == [
        [1, 0, 0, 1, 0, 0, 0, 0, 0], [0, 1, 0, 0, 0, 1, 0, 1, 0], [0, 0, 1, 0, 0, 0, 0, 0, 0],
        [0, 0, 0, 0, 1, 0, 1, 0, 0], [0, 0, 0, 0, 0, 0, 0, 0, 1]]
    info = torch.tensor([[1, 0, 0, 0], [0, 1, 1, 0], [0, 0, 0, 1], [0, 0, 0, 0]], dtype=torch.int32, device="cuda")
    tw = torch.tensor([[0.3, 0.7], [0.2, 0.8]], dtype=torch.float32, device="cuda")
    cnt = torch.zeros((4,), dtype=torch.int32, device="cuda")
    wout = torch.zeros((4, 4), dtype=torch.float32, device="cuda")
    moe_align1(info, tw, wout, cnt, 2)
    assert cnt.cpu().tolist() == [1, 2, 1, 0]
    assert info.cpu().tolist() == [[0, 0, 0, 0], [1, 2, 1, 0], [3, 0, 0, 1], [0, 0, 0, 0]]
    assert torch.allclose(wout.cpu(), torch.tensor([[0.3, 0, 0, 0], [0.7, 0.2, 0, 0], [0.8, 0, 0, 0], [0, 0, 0, 0]]))
    for (T, E, topk, seed) in [(1, 3, 2, 1), (300, 12, 4, 2), (5121, 257, 8, 3), (4097, 2, 1, 4)]:
        ids_c, tw_c = H.routing(T, E, topk, seed=seed)
        mask = torch.empty((E, T * topk), dtype=torch.int32, device="cuda")
        moe_align(ids_c.cuda(), mask)
        mask_ref = oracle.moe_align(ids_c.numpy(), E)
        assert np.array_equal(mask.cpu().numpy(), mask_ref)
        wout = torch.zeros((E, T * topk), dtype=torch.float32, device="cuda")
        cnt = torch.empty((E,), dtype=torch.int32, device="cuda")
        moe_align1(mask, tw_c.cuda(), wout, cnt, topk)
        info_ref, w_ref, cnt_ref = oracle.moe_align1(mask_ref, tw_c.numpy(), np.zeros(mask_ref.shape, np.float32))
        assert np.array_equal(cnt.cpu().numpy(), cnt_ref)
        assert np.array_equal(mask.cpu().numpy(), info_ref)          # in place, tails included
        assert np.array_equal(wout.cpu().numpy(), w_ref)


def test_moe_align2_reference_vectors(hip):
    """Golden vectors of the reference's test_moe_align2 (test_grouped_fused_moe.py:219-258)."""
    from lightllm_amd.fused_moe import moe_align2

    print("moe_align2", flush=True)
    cnt = torch.tensor([8, 0, 60, 16], dtype=torch.int32, device="cuda")
    t = moe_align2(100, cnt, block_m=16).cpu()
    assert t.shape[0] == min(100, -(-(100 + 4 * 15) // 16))
    assert t[:, 0].tolist() == [0, 2, 2, 2, 2, 3, -1, -1, -1, -1]
    assert t[:6, 1].tolist() == [0, 0, 1, 2, 3, 0]
    assert t[:6, 2].tolist() == [0, 8, 24, 40, 56, 68]
    assert t[:6, 3].tolist() == [8, 16, 16, 16, 12, 16]      # tokens per block (derived column)
    cnt = torch.zeros((10,), dtype=torch.int32, device="cuda")
    cnt[0] = 8
    t = moe_align2(8, cnt, block_m=16).cpu()
    assert t.shape[0] == 8 and t[0, 0] == 0 and bool((t[1:, 0] == -1).all())


def _grouped_case(T, E, topk, N, K, block_m, mul_w, seed):
    from lightllm_amd.fused_moe import grouped_matmul, moe_align2
    from lightllm_amd.quantization import per_token_group_quant_fp8

    ids, tw = H.routing(T, E, topk, seed=seed)
    idx, w, cnt = _align(ids, tw, E)
    x = H.activations(T, K, seed=seed + 1).cuda()
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, -(-N // 128), K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=seed + 10 + e, device="cuda")
    P = T * topk
    out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, x, None, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=mul_w, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m} if block_m else None)
    torch.cuda.synchronize()
    xq, xs = per_token_group_quant_fp8(x, 128)
    ref_bits = oracle.grouped_block_gemm(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy(),
                                         idx.cpu().numpy(), w.cpu().numpy(), cnt.cpu().numpy(), topk, mul_w)
    ref = tr.bf16_from_bits(ref_bits).float()
    got = out.float().cpu()
    assert not torch.isnan(got).any(), "a routed row was not written"
    cos, rel = H.gemm_metrics(got, ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    assert (got - ref).abs().max() <= ref.abs().max() * 2 ** -7


@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("block_m,T,E,N,K", [(16, 40, 12, 384, 512), (64, 300, 6, 200, 256), (128, 700, 5, 384, 512),
                                             (256, 900, 5, 640, 1152), (256, 2048, 64, 1160, 1152)])
def test_grouped_bias_vs_oracle(hip, bias_dtype, block_m, T, E, N, K):
    """The per-expert bias [E, N] (grouped_fused_moe.py:702-707) in every tile that has an epilogue of its own: the
    ring tiles, the 256-row ping-pong tile and (last case: more tiles than compute units) the 64x512 streaming
    tile; with and without the routed weight, an n tail, every bias dtype.  bf16 / fp16 biases are widened
    exactly, so the oracle gets their fp32 values."""
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"grouped bias dtype={bias_dtype} block_m={block_m} T={T} E={E} N={N} K={K}", flush=True)
    topk = 2
    ids, tw = H.routing(T, E, topk, seed=T + E)
    idx, w, cnt = _align(ids, tw, E)
    x = H.activations(T, K, seed=T).cuda()
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, -(-N // 128), K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=900 + e, device="cuda")
    bias = (torch.randn((E, N), generator=H.gen(N)) * 0.5).to(bias_dtype)
    xq, xs = per_token_group_quant_fp8(x, 128)
    P = T * topk
    for mul_w in (False, True):
        out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        grouped_matmul(P, x, None, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=mul_w, use_fp8_w8a8=True,
                       run_config={"BLOCK_SIZE_M": block_m}, bias=bias.cuda())
        torch.cuda.synchronize()
        ref_bits = oracle.grouped_block_gemm(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy(),
                                             idx.cpu().numpy(), w.cpu().numpy(), cnt.cpu().numpy(), topk, mul_w,
                                             bias=bias.float().numpy())
        ref = tr.bf16_from_bits(ref_bits).float()
        got = out.float().cpu()
        assert not torch.isnan(got).any(), "a routed row was not written"
        cos, rel = H.gemm_metrics(got, ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
        assert (got - ref).abs().max() <= ref.abs().max() * 2 ** -7
    # a zero bias gives the bits of the launch without one
    plain = torch.empty((P, N), dtype=torch.bfloat16, device="cuda")
    zero = torch.empty((P, N), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, x, None, cnt, idx, w, wq, ws, topk, plain, mul_routed_weight=True, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m})
    grouped_matmul(P, x, None, cnt, idx, w, wq, ws, topk, zero, mul_routed_weight=True, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m}, bias=torch.zeros((E, N), dtype=bias_dtype, device="cuda"))
    torch.cuda.synchronize()
    routed = idx.cpu()[0, : int(cnt.cpu()[0])].long()
    if routed.numel():
        # (-0 + 0 = +0: compare values, then bits wherever the plain result is not a negative zero)
        a, b = plain.cpu()[routed], zero.cpu()[routed]
        assert torch.equal(a.float(), b.float())


@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128])
@pytest.mark.parametrize("mul_w,topk", [(False, 4), (True, 1)])
def test_grouped_vs_oracle(hip, block_m, mul_w, topk):
    print(f"grouped block_m={block_m} mul_w={mul_w} topk={topk}", flush=True)
    _grouped_case(T=96 if topk > 1 else 300, E=12, topk=topk, N=384, K=512, block_m=block_m, mul_w=mul_w, seed=70)


@pytest.mark.parametrize("mul_w,topk,T,E", [(False, 4, 200, 7), (True, 1, 900, 5), (False, 2, 40, 9)])
def test_grouped_256_row_blocks_vs_oracle(hip, mul_w, topk, T, E):
    """The 256x256 ping-pong tile in grouped mode: experts with fewer than 64, 64-128,
    128-256 and more than 256 rows, so that every combination of skipped half tiles occurs; N tail (640 % 256)."""
    print(f"grouped block_m=256 mul_w={mul_w} topk={topk} T={T} E={E}", flush=True)
    _grouped_case(T=T, E=E, topk=topk, N=640, K=2048, block_m=256, mul_w=mul_w, seed=75)
    _grouped_case(T=T, E=E, topk=topk, N=640, K=1152, block_m=256, mul_w=mul_w, seed=76)   # K/128 = 9: partial scale chunk


@pytest.mark.parametrize("mul_w,topk,T", [(False, 4, 512), (True, 1, 2048)])
def test_grouped_small_block_tile_tails(hip, mul_w, topk, T):
    """More tiles than compute units, so the 256-row launch sorts the blocks by size and runs those of at most 64
    rows on the 64x512 streaming tile: 64 experts with Zipf routing (most blocks small, a few large), an n tail
    inside the last 512-wide pair (1160 = 2 * 512 + 136), K/128 = 9 (partial scale chunk)."""
    print(f"grouped small-block tile mul_w={mul_w} topk={topk} T={T}", flush=True)
    _grouped_case(T=T, E=64, topk=topk, N=1160, K=1152, block_m=256, mul_w=mul_w, seed=77)


@pytest.mark.parametrize("T,E,topk,what", [(1500, 40, 1, "only small blocks"), (3000, 6, 2, "only large blocks"),
                                           (2100, 30, 1, "blocks of exactly 64 and 65 rows")])
def test_grouped_two_queues_degenerate(hip, T, E, topk, what):
    """The launch with two work queues when one of them is empty, and at the boundary between them: uniform routing
    (zipf_s = 0) gives every expert about the same count; the third case forces counts of 64, 65, 128 and 129 rows.
    N = 3072 makes more tiles than compute units in every case."""
    from lightllm_amd.fused_moe import grouped_matmul, moe_align_fused
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"grouped two queues: {what}", flush=True)
    N, K = 3072, 512
    if "exactly" in what:
        counts = ([64, 65, 128, 129, 1, 63] * 5)[:E]
        ids = torch.cat([torch.full((c,), e, dtype=torch.int32) for e, c in enumerate(counts)])
        T = ids.numel()
        ids = ids[torch.randperm(T, generator=H.gen(3))].reshape(T, 1).contiguous()
        tw = torch.rand((T, 1), generator=H.gen(4)).float()
    else:
        ids, tw = H.routing(T, E, topk, seed=41, zipf_s=0.0)
    P = T * topk
    idx = torch.empty((E, P), dtype=torch.int32, device="cuda")
    w = torch.empty((E, P), dtype=torch.float32, device="cuda")
    cnt = torch.empty((E,), dtype=torch.int32, device="cuda")
    moe_align_fused(idx, w, cnt, ids.cuda(), tw.cuda())
    counts_h = cnt.cpu().numpy()
    if "small" in what:
        assert counts_h.max() <= 64
    if "large" in what:
        assert counts_h.min() > 64
    x = H.activations(T, K, seed=42).cuda()
    xq, xs = per_token_group_quant_fp8(x, 128)
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=500 + e, device="cuda")
    out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, xq, xs, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=True, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": 256})
    torch.cuda.synchronize()
    assert not torch.isnan(out.float()).any(), "a routed row was not written"
    idx_h, w_h = idx.cpu(), w.cpu()
    for e in range(E):
        n_e = int(counts_h[e])
        if n_e == 0:
            continue
        pairs = idx_h[e, :n_e].long().cuda()
        ref = tr.dequant_matmul(xq[pairs // topk], xs[pairs // topk], wq[e], ws[e], out_dtype=torch.float32)
        ref = ref * w_h[e, :n_e].cuda()[:, None]
        cos, rel = H.gemm_metrics(out[pairs].float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (e, n_e, cos, rel)


def test_grouped_persistent_launch_matches_one_workgroup_per_tile(hip, monkeypatch):
    """The 256-row launch with the workspace counters (persistent, tiles handed out per XCD) against the same
    kernel without a workspace (one workgroup per tile): about 600 tiles of mixed cost, identical bits, counter
    words zero afterwards.  A sample of rows is checked against the torch fp32 dequant-matmul of its expert."""
    from lightllm_amd import _lib
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print("grouped persistent vs per-tile launch", flush=True)
    T, E, topk, N, K = 2048, 24, 4, 4096, 1024
    ids, tw = H.routing(T, E, topk, seed=95)
    idx, w, cnt = _align(ids, tw, E)
    x = H.activations(T, K, seed=96).cuda()
    xq, xs = per_token_group_quant_fp8(x, 128)
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=100 + e, device="cuda")
    P = T * topk

    def run():
        out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        grouped_matmul(P, xq, xs, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=False, use_fp8_w8a8=True,
                       run_config={"BLOCK_SIZE_M": 256})
        torch.cuda.synchronize()
        return out

    persistent = [run() for _ in range(2)]
    counters = _lib.workspace(xq.device, _lib.WS_COUNTER_BYTES)[:64]
    assert not bool(counters.any())
    with monkeypatch.context() as mp:
        mp.setattr(_lib, "workspace", lambda *a, **k: None)
        once = run()
    assert not torch.isnan(once.float()).any()
    for out in persistent:
        assert torch.equal(out.view(torch.int16), once.view(torch.int16))
    cnt_h, idx_h = cnt.cpu(), idx.cpu()
    for e in range(0, E, 5):
        pairs = idx_h[e, : int(cnt_h[e])].long()[:64].cuda()
        ref = tr.dequant_matmul(xq[pairs // topk], xs[pairs // topk], wq[e], ws[e], out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(once[pairs].float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (e, cos, rel)


def test_grouped_random_shapes(hip):
    """Sixteen seeded random routed batches (tokens, experts, top-k, N with a tail, K with and without chunked
    scale fetches, every row-block size that the shape allows, routed weight on and off): every routed row against
    the torch fp32 dequant-matmul of its expert."""
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    rng = np.random.default_rng(97)
    for case in range(16):
        T = int(rng.integers(1, 700))
        E = int(rng.integers(1, 20))
        topk = int(rng.integers(1, min(E, 4) + 1))
        N = int(rng.integers(1, 12)) * 64 + int(rng.choice([0, 8, 40]))
        K = int(rng.choice([128, 384, 1024, 2048]))
        blocks = [16, 32, 64, 128, 256]
        block_m = int(rng.choice(blocks))
        mul_w = bool(rng.integers(0, 2)) and topk == 1
        print(f"grouped random case {case}: T={T} E={E} topk={topk} N={N} K={K} block_m={block_m} mul_w={mul_w}", flush=True)
        ids, tw = H.routing(T, E, topk, seed=500 + case)
        idx, w, cnt = _align(ids, tw, E)
        x = H.activations(T, K, seed=600 + case).cuda()
        xq, xs = per_token_group_quant_fp8(x, 128)
        wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
        ws = torch.empty((E, -(-N // 128), K // 128), dtype=torch.float32, device="cuda")
        for e in range(E):
            wq[e], ws[e] = H.quantized_weights(N, K, seed=700 + 31 * case + e, device="cuda")
        P = T * topk
        out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        grouped_matmul(P, xq, xs, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=mul_w, use_fp8_w8a8=True,
                       run_config={"BLOCK_SIZE_M": block_m})
        torch.cuda.synchronize()
        assert not torch.isnan(out.float()).any(), "a routed row was not written"
        cnt_h, idx_h, w_h = cnt.cpu(), idx.cpu(), w.cpu()
        for e in range(E):
            n_e = int(cnt_h[e])
            if n_e == 0:
                continue
            pairs = idx_h[e, :n_e].long().cuda()
            ref = tr.dequant_matmul(xq[pairs // topk], xs[pairs // topk], wq[e], ws[e], out_dtype=torch.float32)
            if mul_w:
                ref = ref * w_h[e, :n_e].cuda()[:, None]
            cos, rel = H.gemm_metrics(out[pairs].float(), ref)
            assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (case, e, cos, rel)


def test_grouped_empty_and_single_token_experts(hip):
    """More experts than tokens: most experts get no rows, some one row; N tail (200 % 128 != 0)."""
    print("grouped sparse experts", flush=True)
    _grouped_case(T=5, E=40, topk=2, N=200, K=256, block_m=None, mul_w=False, seed=80)


@pytest.mark.parametrize("block_m", [None, 256])
def test_grouped_deepseek_shape_sampled(hip, block_m):
    """The routed-expert config at a reduced expert count (16 of 256 experts, same N/K, Zipf routing):
    every routed row is checked against the torch fp32 dequant-matmul of its expert."""
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"grouped dsv3-shaped block_m={block_m}", flush=True)
    T, E, topk, N, K = 1024, 16, 8, 4096, 7168
    ids, tw = H.routing(T, E, topk, seed=90)
    idx, w, cnt = _align(ids, tw, E)
    x = H.activations(T, K, seed=91).cuda()
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=100 + e, device="cuda")
    P = T * topk
    out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_matmul(P, x, None, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=False, use_fp8_w8a8=True,
                   run_config={"BLOCK_SIZE_M": block_m} if block_m else None)
    torch.cuda.synchronize()
    xq, xs = per_token_group_quant_fp8(x, 128)
    dx = tr.dequant(xq, xs, 1, 128)
    pair_expert = ids.flatten().cuda().long()
    for e in range(E):
        rows = torch.nonzero(pair_expert == e).flatten()
        if rows.numel() == 0:
            continue
        ref = dx[rows // topk] @ tr.dequant(wq[e], ws[e], 128, 128).T
        cos, rel = H.gemm_metrics(out[rows].float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (e, cos, rel)


@pytest.mark.parametrize("block_m", [16, 64, 128, 256])
def test_grouped_fp16_output(hip, block_m):
    """out in fp16 (`accumulator.to(compute_type)`, grouped_fused_moe.py:717): every row-block size, the 256-row launch
    with enough tiles for the small-block tile; against the bf16 launch and the torch fp32 dequant-matmul per expert."""
    from lightllm_amd.fused_moe import grouped_matmul
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print(f"grouped fp16 out block_m={block_m}", flush=True)
    T, E, topk, N, K = 700, 40, 4, 1160, 1152
    ids, tw = H.routing(T, E, topk, seed=31)
    idx, w, cnt = _align(ids, tw, E)
    x = H.activations(T, K, seed=32).cuda()
    xq, xs = per_token_group_quant_fp8(x, 128)
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, -(-N // 128), K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=300 + e, device="cuda")
    P = T * topk
    outs = {}
    for dt in (torch.float16, torch.bfloat16):
        out = torch.full((P, N), float("nan"), dtype=dt, device="cuda")
        grouped_matmul(P, xq, xs, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=True, use_fp8_w8a8=True,
                       run_config={"BLOCK_SIZE_M": block_m})
        torch.cuda.synchronize()
        assert not torch.isnan(out.float()).any()
        outs[dt] = out
    a, b = outs[torch.float16].float(), outs[torch.bfloat16].float()
    assert (a - b).abs().max() <= 2 ** -8 * b.abs().max()
    cnt_h, idx_h, w_h = cnt.cpu(), idx.cpu(), w.cpu()
    for e in range(0, E, 7):
        n_e = int(cnt_h[e])
        if n_e == 0:
            continue
        pairs = idx_h[e, :n_e].long().cuda()
        ref = tr.dequant_matmul(xq[pairs // topk], xs[pairs // topk], wq[e], ws[e], out_dtype=torch.float32)
        ref = ref * w_h[e, :n_e].cuda()[:, None]
        cos, rel = H.gemm_metrics(a[pairs], ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (e, cos, rel)

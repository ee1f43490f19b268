"""The entry points enqueue kernels only (no allocation, no host synchronisation, counters left zero), so a captured
HIP graph of the quantizer + GEMM, and of the grouped GEMM, replays to the eager result every time."""
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def _replay_matches(fn_eager, make_graph_outputs, replays=4):
    """fn_eager() -> tensor; make_graph_outputs() -> (graph, output tensor).  Eager work and synchronisations sit
    between the replays, and the output is poisoned before each one."""
    expect = fn_eager().clone()
    graph, out = make_graph_outputs()
    for r in range(replays):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), expect.view(torch.int16)), f"replay {r}"
        again = fn_eager()                      # eager launches between replays share the stream's workspace
        assert torch.equal(again.view(torch.int16), expect.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(4096, 12288, 1024), (8, 4096, 14336), (32, 4096, 14336), (200, 640, 8192), (100, 4096, 14336), (200, 4096, 14336)])
def test_quant_and_gemm_under_graph_capture(hip, M, N, K):
    """Persistent 256x256 launch (768 tiles), split-K stream launch, split-K 128x128 launch, the 256-weight-row
    stream with its second launch that adds the partial sums."""
    from lightllm_amd.quantization import lightllm_per_token_group_quant_fp8, w8a8_block_fp8_matmul

    print(f"graph capture gemm M={M} N={N} K={K}", flush=True)
    x = H.activations(M, K, seed=5).cuda()
    wq, ws = H.quantized_weights(N, K, seed=6, device="cuda")
    xq = torch.empty((M, K), dtype=torch.float8_e4m3fn, device="cuda")
    xs = torch.empty((M, K // 128), dtype=torch.float32, device="cuda")

    def step(out):
        lightllm_per_token_group_quant_fp8(x, 128, xq, xs)
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), out, [128, 128])
        return out

    eager_out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def capture():
        out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(out)                            # first call on this stream allocates its workspace: before capture
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                step(out)
        torch.cuda.current_stream().wait_stream(side)
        return g, out

    _replay_matches(lambda: step(eager_out), capture)


def test_grouped_gemm_under_graph_capture(hip):
    from lightllm_amd.fused_moe import grouped_matmul, moe_align_fused
    from lightllm_amd.quantization import per_token_group_quant_fp8

    print("graph capture grouped gemm", flush=True)
    T, E, topk, N, K = 1536, 24, 4, 4096, 1024       # more tiles than compute units: persistent, both work queues
    ids, tw = H.routing(T, E, topk, seed=15)
    P = T * topk
    idx = torch.empty((E, P), dtype=torch.int32, device="cuda")
    w = torch.empty((E, P), dtype=torch.float32, device="cuda")
    cnt = torch.empty((E,), dtype=torch.int32, device="cuda")
    moe_align_fused(idx, w, cnt, ids.cuda(), tw.cuda())
    xq, xs = per_token_group_quant_fp8(H.activations(T, K, seed=16).cuda(), 128)
    wq = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device="cuda")
    ws = torch.empty((E, N // 128, K // 128), dtype=torch.float32, device="cuda")
    for e in range(E):
        wq[e], ws[e] = H.quantized_weights(N, K, seed=20 + e, device="cuda")

    def step(out, infos=None):
        return grouped_matmul(P, xq, xs, cnt, idx, w, wq, ws, topk, out, mul_routed_weight=False, use_fp8_w8a8=True,
                              reused_mblock_infos=infos, run_config={"BLOCK_SIZE_M": 256})

    eager_out = torch.empty((P, N), dtype=torch.bfloat16, device="cuda")
    infos = step(eager_out)                     # the schedule table is built once, outside the graph

    def capture():
        out = torch.empty((P, N), dtype=torch.bfloat16, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(out, infos)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                step(out, infos)
        torch.cuda.current_stream().wait_stream(side)
        return g, out

    def eager():
        step(eager_out, infos)
        return eager_out

    _replay_matches(eager, capture)


def test_graph_survives_workspace_regrowth(hip):
    """A graph captured at a split-K shape keeps the workspace address it was captured with.  A later eager call
    that needs a larger workspace must not free that buffer: the replay afterwards still has to give the eager
    result, and so does the large call."""
    from lightllm_amd import _lib
    from lightllm_amd.quantization import per_token_group_quant_fp8, w8a8_block_fp8_matmul

    print("graph capture across workspace regrowth", flush=True)
    M, N, K = 32, 4096, 14336                     # stream kernel, K split over CTAs: uses partials + counters
    xq, xs = per_token_group_quant_fp8(H.activations(M, K, seed=31).cuda(), 128)
    wq, ws = H.quantized_weights(N, K, seed=32, device="cuda")
    expect = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), expect, [128, 128])
    torch.cuda.synchronize()

    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), out, [128, 128])
        torch.cuda.synchronize()
        first_ws = _lib.workspace(xq.device, 1)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), out, [128, 128])
        # a call on the same stream that outgrows the workspace, then garbage written wherever the allocator
        # would have recycled a freed buffer
        bigger = _lib.workspace(xq.device, first_ws.numel() + (8 << 20))
        assert bigger.data_ptr() != first_ws.data_ptr()
        del first_ws
        junk = [torch.full((first_n,), 0x7F, dtype=torch.uint8, device="cuda") for first_n in (33 << 20, 33 << 20)]
        torch.cuda.synchronize()
        for r in range(3):
            out.fill_(float("nan"))
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), expect.view(torch.int16)), f"replay {r}"
            eager = torch.empty_like(out)
            w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), eager, [128, 128])   # now on the larger workspace
            torch.cuda.synchronize()
            assert torch.equal(eager.view(torch.int16), expect.view(torch.int16))
        del junk
    torch.cuda.current_stream().wait_stream(side)


def test_capture_after_a_warm_up_on_another_stream_allocates_nothing(hip):
    """The reference warms a shape up on the current stream and captures on the side stream that ``torch.cuda.graph``
    opens by itself (lightllm/common/basemodel/cuda_graph.py, _capture_decode).  The captured call must find the
    device's workspace sized by the warm-up: no buffer appears during the capture, the allocator hands out nothing,
    and every replay gives the eager result."""
    from lightllm_amd import _lib
    from lightllm_amd.quantization import per_token_group_quant_fp8, w8a8_block_fp8_matmul

    print("graph capture after a warm-up on the current stream", flush=True)
    M, N, K = 32, 4096, 14336                     # K shared between workgroups: partials + counters in the workspace
    xq, xs = per_token_group_quant_fp8(H.activations(M, K, seed=41).cuda(), 128)
    wq, ws = H.quantized_weights(N, K, seed=42, device="cuda")
    assert _lib.lib().mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_AUTO) > _lib.WS_COUNTER_BYTES
    expect = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), expect, [128, 128])          # the warm-up, current stream
    torch.cuda.synchronize()
    out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    buffers = {k: v.data_ptr() for k, v in _lib._workspaces.items()}
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):                                                  # torch's own capture stream
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), out, [128, 128])
        after = torch.cuda.memory_stats()["allocation.all.allocated"]
    assert after == before, "the captured call allocated device memory"
    assert {k: v.data_ptr() for k, v in _lib._workspaces.items()} == buffers
    for r in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), expect.view(torch.int16)), f"replay {r}"
        eager = torch.empty_like(out)
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), eager, [128, 128])
        torch.cuda.synchronize()
        assert torch.equal(eager.view(torch.int16), expect.view(torch.int16))


def test_reset_workspace_recovers_dirty_counters(hip):
    """Counter words left non-zero (as an aborted launch would) make a split-K launch wrong; the reset entry point
    restores the invariant."""
    from lightllm_amd import _lib
    from lightllm_amd.quantization import per_token_group_quant_fp8, w8a8_block_fp8_matmul

    M, N, K = 32, 4096, 14336
    xq, xs = per_token_group_quant_fp8(H.activations(M, K, seed=33).cuda(), 128)
    wq, ws = H.quantized_weights(N, K, seed=34, device="cuda")
    expect = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), expect, [128, 128])
    torch.cuda.synchronize()
    buf = _lib.workspace(xq.device, 1)
    buf[: _lib.WS_COUNTER_BYTES].view(torch.int32).fill_(1 << 20)   # no CTA will ever see itself as the last arrival
    _lib.reset_workspace(xq.device)
    out = torch.empty_like(expect)
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), out, [128, 128])
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), expect.view(torch.int16))
    assert int(buf[: _lib.WS_COUNTER_BYTES].view(torch.int32).abs().max()) == 0

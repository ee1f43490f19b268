"""GPU parity of w8a8_block_fp8_matmul.

Acceptance (stated by the task, form from the reference's in-file check,
quantization/fp8w8a8_block_gemm_kernel.py:213-223): against the fp32 dequant-then-matmul,
max|C - ref| / max|ref| <= 1e-2 and cosine >= 0.9999.  Small shapes are compared with the CPU oracle on the
whole matrix; full-size shapes with a float64 oracle on sampled rows/columns plus a torch fp32
dequant-matmul of the whole matrix on the GPU.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu

VARIANTS_BIG = ["tile256", "tile256x128", "tile128"]


def _prep(M, N, K, seed=0, device="cuda"):
    from lightllm_amd.quantization import per_token_group_quant_fp8

    x = H.activations(M, K, seed=seed).to(device)
    xq, xs = per_token_group_quant_fp8(x, 128)
    wq, ws = H.quantized_weights(N, K, seed=seed + 1, device=device)
    return xq, xs, wq, ws


def _run(xq, xs, wq, ws, variant=None, out=None):
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    M, N = xq.shape[0], wq.shape[0]
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=xq.device) if out is None else out
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), C, [128, 128], dtype=torch.bfloat16,
                          run_config={"variant": variant} if variant else None)
    torch.cuda.synchronize()
    return C


def _check_small(xq, xs, wq, ws, C):
    """Whole-matrix comparison with the CPU oracle (fp32 per-block order) and the acceptance metrics
    against float64 dequant-matmul."""
    M, N = C.shape
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy(),
                                          np.arange(M), np.arange(N))
    ref = torch.from_numpy(ref64)
    c = C.float().cpu()
    assert not torch.isnan(c).any(), "output holds unwritten (NaN) entries"
    cos, rel = H.gemm_metrics(c, ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    # bf16 rounding of an fp32 accumulation: within one bf16 ulp of the oracle's own bf16 result, relative to
    # the row scale (different but valid summation order)
    cb = tr.bf16_from_bits(oracle.block_gemm(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy())).float()
    err = (c - cb).abs().max() / cb.abs().max()
    assert err <= 2 ** -7, err


def test_cpu_reference_config_on_the_gpu(hip):
    """The CPU reference configuration (M = 32, N = K = 4096, seed 0: activations ~ N(0,1) quantized per 1x128
    group, weights ~ N(0, 0.02) block-quantized with the reference's load-time quantizer) through the HIP path
    with the kernel the shape table picks: the whole matrix against the oracle's fp32 per-block form and the
    float64 dequant-matmul."""
    from lightllm_amd.quantization import per_token_group_quant_fp8, w8a8_block_fp8_matmul, weight_quant

    print("gemm cpu-reference config M=32 N=4096 K=4096", flush=True)
    M, N, K = 32, 4096, 4096
    x = H.activations(M, K, seed=0)
    w = H.weights(N, K, seed=0)
    xq, xs = per_token_group_quant_fp8(x.cuda(), 128)
    wq, ws = weight_quant(w.cuda(), 128)
    # the operands themselves are the oracle's, bit for bit
    q_ref, s_ref = oracle.group_quant_fp8(tr.bits_of(x))
    wq_ref, ws_ref = oracle.block_weight_quant(w.float().numpy())
    assert np.array_equal(tr.bits_of(xq), q_ref) and np.array_equal(tr.bits_of(xs), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(wq), wq_ref) and np.array_equal(ws.cpu().numpy(), ws_ref)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), C, [128, 128]) is C
    torch.cuda.synchronize()
    _check_small(xq, xs, wq, ws, C)
    # and against the reference's own closed form on the CPU (fp8w8a8_block_gemm_kernel.py:213-217 in fp32)
    ref = tr.dequant_matmul(xq.cpu(), xs.cpu(), wq.cpu(), ws.cpu(), out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(C.float().cpu(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


@pytest.mark.parametrize("variant", [None, "tile256", "tile256x128", "tile128", "skinny", "rows128", "generic"])
@pytest.mark.parametrize("M,N,K", [(32, 512, 1024), (1, 256, 512), (64, 384, 2048), (17, 2112, 256)])
def test_small_vs_oracle(hip, M, N, K, variant):
    print(f"gemm small M={M} N={N} K={K} variant={variant}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + N + K, device="cuda")
    _check_small(xq, xs, wq, ws, _run(xq, xs, wq, ws, variant))


@pytest.mark.parametrize("variant", [None, "tile256", "tile256x128", "tile128", "generic"])
@pytest.mark.parametrize("M,N,K", [(300, 640, 1024), (129, 200, 128), (513, 136, 384)])
def test_ragged_edges(hip, M, N, K, variant):
    print(f"gemm edges M={M} N={N} K={K} variant={variant}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=3 * M + N + K, device="cuda")
    _check_small(xq, xs, wq, ws, _run(xq, xs, wq, ws, variant))


@pytest.mark.parametrize("M,N,K", [(256, 256, 1024), (257, 520, 1024), (700, 2112, 2048), (1024, 768, 3072)])
def test_pingpong_tile_equals_ring_tile(hip, M, N, K):
    """The ping-pong schedule (scales fetched in chunks of eight K steps) and the plain ring on the same 256x256 tile
    add the same products in the same order, so the two must agree bit for bit - with row-major scales (16-byte
    requests) and with column-major scales (strides (1, M): 4-byte requests)."""
    print(f"gemm ping-pong vs ring M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + K, device="cuda")
    c_pp = _run(xq, xs, wq, ws, "tile256")
    c_ring = _run(xq, xs, wq, ws, "tile256ring")
    assert torch.equal(c_pp.view(torch.int16), c_ring.view(torch.int16))
    xs_cm = xs.t().contiguous().t()
    assert xs_cm.stride() == (1, M) or M == 1
    c_cm = _run(xq, xs_cm, wq, ws, "tile256")
    assert torch.equal(c_cm.view(torch.int16), c_ring.view(torch.int16))
    if M * N <= 300 * 600:
        _check_small(xq, xs, wq, ws, c_pp)


@pytest.mark.parametrize("M,N,K", [(2048, 8448, 512), (2048, 8448, 256), (4096, 4352, 1024), (1024, 17152, 384),
                                   (2048, 8448 + 128, 512), (2048 - 8, 8448, 512)])
def test_pingpong_requests_run_on_across_tiles(hip, M, N, K):
    """Persistent launches (more tiles than compute units) of 256x256 tiles with an even number of K steps:
    the last two steps of a tile request the first two of the workgroup's next tile.  Short K ranges, so that a
    workgroup crosses several tile boundaries with two to eight steps between them; K/128 odd takes the plain path,
    and so do the boundaries next to the partial tiles of a ragged N or M.  Bit-equal to the ring kernel, and
    against the torch fp32 dequant-matmul."""
    print(f"gemm ping-pong across tiles M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + N + K, device="cuda")
    c_pp = _run(xq, xs, wq, ws, "tile256").clone()
    assert torch.equal(c_pp.view(torch.int16), _run(xq, xs, wq, ws, "tile256").view(torch.int16))
    c_ring = _run(xq, xs, wq, ws, "tile256ring")
    assert torch.equal(c_pp.view(torch.int16), c_ring.view(torch.int16)), (M, N, K)
    xs_cm = xs.t().contiguous().t()   # column-major scales: 4-byte scale requests
    assert torch.equal(_run(xq, xs_cm, wq, ws, "tile256").view(torch.int16), c_ring.view(torch.int16)), (M, N, K)
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(c_pp.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


@pytest.mark.parametrize("K", [128, 512, 1152, 1536, 2304, 7296])
def test_pingpong_tile_off_grid_k(hip, K):
    """K/128 not a multiple of 8 (the reference's own tuning list holds K = 512, 1152, 1536, 2304,
    test/kernel/deepseekv3_fp8_block_gemm_tuning.py:230-251): the last scale chunk is partial, rows of the scale
    matrix are not 16-byte aligned for odd K/128.  Bit-equal to the ring, persistent launch included."""
    for (M, N) in [(300, 520), (4096, 4096)]:
        print(f"gemm ping-pong off-grid K M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=K + M, device="cuda")
        c_pp = _run(xq, xs, wq, ws, "tile256")
        c_ring = _run(xq, xs, wq, ws, "tile256ring")
        assert torch.equal(c_pp.view(torch.int16), c_ring.view(torch.int16)), (M, N, K)
        if M * N <= 300 * 600:
            _check_small(xq, xs, wq, ws, c_pp)
        else:
            ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
            cos, rel = H.gemm_metrics(c_pp.float(), ref)
            assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


# (M, N, K): tiles that do not fill whole rounds of 256 compute units, so that the stream-K plan is taken: one
# round half empty (DeepSeek q_a+kv_a), a second round one eighth full, few tiles with a long K, ragged edges with
# a K that is not a multiple of 1024
# ... and shapes that take the panel split (every tile's K range in the same runs, one (m tile, run) pair per XCD):
# even and uneven runs, ragged edges, three runs over eight m tiles
STREAM_K_SHAPES = [(4096, 2112, 7168), (512, 36864, 7168), (1024, 7168, 18432), (1000, 8200, 4992), (500, 3000, 6400),
                   (2048, 2112, 7168), (300, 4096, 14336), (1000, 2048, 16384), (240, 7168, 18432),
                   (352, 7168, 16384)]


@pytest.mark.parametrize("M,N,K", STREAM_K_SHAPES)
def test_stream_k_launch(hip, M, N, K):
    """Stream-K: the K steps of all tiles are shared between the compute units - as one cut of the (tile, step)
    sequence, or as the panel split where the shape has one - and partial tiles are added through the workspace in K
    order by a second launch.  Against the torch fp32 dequant-matmul (whole matrix) and the float64 oracle
    (sample); identical bits on repeated launches whoever arrives last; counter words zero afterwards.  The shape
    table itself takes this launch only for the last shape (few tiles, long K)."""
    from lightllm_amd import _lib

    print(f"gemm stream-K M={M} N={N} K={K}", flush=True)
    need = hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_TILE256_STREAMK)
    assert need > _lib.WS_COUNTER_BYTES, "the shape must take the stream-K plan on this device"
    xq, xs, wq, ws = _prep(M, N, K, seed=M + N)
    first = _run(xq, xs, wq, ws, "tile256streamk").clone()
    for _ in range(3):
        assert torch.equal(_run(xq, xs, wq, ws, "tile256streamk").view(torch.int16), first.view(torch.int16))
    if (M, N, K) == STREAM_K_SHAPES[-1]:
        assert hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_AUTO) == need
        assert torch.equal(_run(xq, xs, wq, ws, None).view(torch.int16), first.view(torch.int16))
    counters = _lib.workspace(xq.device, need)[: _lib.WS_COUNTER_BYTES]
    assert not bool(counters.any())
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(first.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    # against the plain tile loop: same products, another summation order for the tiles that were split
    plain = _run(xq, xs, wq, ws, "tile256")
    assert (first.float() - plain.float()).abs().max() <= 2 ** -7 * plain.float().abs().max()
    rng = np.random.default_rng(M)
    rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 6)])
    cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 40)])
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                          ws.cpu().numpy(), np.arange(len(rows)), cols)
    got = first[rows][:, cols].float().cpu().double().numpy()
    assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * np.abs(ref64).max()


@pytest.mark.parametrize("M,N,K", [(4096, 16384, 1024), (4000, 16400, 1024), (1100, 16385, 1024)])
def test_persistent_launch_matches_one_workgroup_per_tile(hip, M, N, K):
    """With the workspace counters the ping-pong kernel is persistent (one workgroup per CU; from the third tile
    on a workgroup takes tiles from per-XCD atomic counters), without them every tile gets its own workgroup.
    About 1000 tiles (and fewer, with ragged M and N edges and an N that forces element-wise stores): same bits
    either way, on repeated launches, and the counter words are zero again afterwards."""
    from lightllm_amd import _lib

    print(f"gemm persistent vs per-tile launch M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=12)
    once = _run(xq, xs, wq, ws, "tile256once").clone()
    for _ in range(3):
        assert torch.equal(_run(xq, xs, wq, ws, "tile256").view(torch.int16), once.view(torch.int16))
    counters = _lib.workspace(xq.device, _lib.WS_COUNTER_BYTES)[:64]
    assert int(counters.to(torch.int32).sum()) == 0 and not bool(counters.any())
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(once.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


def test_pingpong_tile_random_shapes(hip):
    """Twenty seeded random shapes (ragged M and N edges, several K): ping-pong and ring tiles agree bit for bit,
    and a sample of entries agrees with the float64 oracle."""
    rng = np.random.default_rng(2024)
    for case in range(20):
        M = int(rng.integers(1, 1100))
        N = int(rng.integers(1, 300)) * 8
        K = int(rng.choice([1024, 2048, 3072]))
        print(f"gemm ping-pong random case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=1000 + case, device="cuda")
        c_pp = _run(xq, xs, wq, ws, "tile256")
        c_ring = _run(xq, xs, wq, ws, "tile256ring")
        assert torch.equal(c_pp.view(torch.int16), c_ring.view(torch.int16)), (M, N, K)
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 6)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c_pp[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)


def test_stream_kernel_random_shapes(hip):
    """Twenty-four seeded random decode-size shapes (every M class, N with and without a 64-row tail or a
    vector-store-friendly width, K from one to 72 steps so that single-CTA and split-K launches, staged and
    gathered scales all occur): the whole matrix against the torch fp32 dequant-matmul and a sample against the
    float64 oracle; the slow generic kernel must agree within one bf16 ulp of the row scale."""
    rng = np.random.default_rng(4711)
    for case in range(24):
        M = int(rng.choice([1, 2, 7, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64]))
        N = int(rng.integers(1, 400)) * int(rng.choice([1, 8, 16]))
        K = int(rng.choice([128, 256, 1024, 2048, 4096, 7168, 9216]))
        print(f"gemm stream random case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=3000 + case, device="cuda")
        c = _run(xq, xs, wq, ws, "skinny")
        assert not torch.isnan(c.float()).any()
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(c.float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (M, N, K, cos, rel)
        g = _run(xq, xs, wq, ws, "generic")
        assert (c.float() - g.float()).abs().max() <= ref.abs().max() * 2 ** -7, (M, N, K)
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 4)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)


def test_per_unit_stream_kernel(hip):
    """The weight stream cut into one share per compute unit (M <= 16, one workgroup of 8 waves per tile, whole K):
    every tile width of 1..5 row blocks - the 48- and 80-row tiles straddle two 128-row scale blocks, whose scales
    differ -, N tails that cut the last tile, the last block and the vector stores, 16 to 160 K steps, one or two
    activation loads per step (M <= 8 / M > 8), column-major activation scales, fp16 output; against the torch fp32
    dequant-matmul, the plain kernel and the float64 oracle, and bit-equal over repeated launches."""
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    rng = np.random.default_rng(4242)
    cus = _lib_cus()
    cases = []
    for tnw, frac in [(1, 1.0), (1, 0.88), (2, 1.0), (2, 0.855), (3, 0.9), (4, 1.0), (5, 0.9), (5, 1.0)]:
        blocks = int(cus * tnw * frac)
        for tail in (0, -4, -9):
            cases.append((int(rng.choice([1, 5, 8, 9, 16])), 16 * blocks + tail, int(rng.choice([2048, 4096, 7168, 18432, 20480]))))
    cases += [(8, 16 * cus, 14336), (16, 16 * cus, 14336), (1, 32 * cus, 2048)]
    for case, (M, N, K) in enumerate(cases):
        print(f"gemm per-unit stream case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=6000 + case, device="cuda")
        c = _run(xq, xs, wq, ws, "streamcu")
        assert not torch.isnan(c.float()).any()
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(c.float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (M, N, K, cos, rel)
        g = _run(xq, xs, wq, ws, "generic")
        assert (c.float() - g.float()).abs().max() <= ref.abs().max() * 2 ** -7, (M, N, K)
        assert torch.equal(c.view(torch.int16), _run(xq, xs, wq, ws, "streamcu").view(torch.int16))
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 4)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 60)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)
        if case % 5 == 0:
            assert torch.equal(c, _run(xq, xs.t().contiguous().t(), wq, ws, "streamcu"))
            h = torch.empty((M, N), dtype=torch.float16, device="cuda")
            w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), h, [128, 128], run_config={"variant": "streamcu"})
            torch.cuda.synchronize()
            assert (h.float() - ref).abs().max() <= ref.abs().max() * 2 ** -9
    # outside its limits the forced kernel is refused, and the table does not pick it
    xq, xs, wq, ws = _prep(17, 4096, 4096, seed=1, device="cuda")
    with pytest.raises(ValueError):
        _run(xq, xs, wq, ws, "streamcu")
    xq, xs, wq, ws = _prep(8, 1024, 4096, seed=1, device="cuda")
    with pytest.raises(ValueError):
        _run(xq, xs, wq, ws, "streamcu")


def _lib_cus():
    from lightllm_amd import _lib

    return _lib.device_info()["compute_units"]


def test_shared_activation_stream_kernel(hip):
    """The streaming kernel whose workgroup shares the activation block (M = 33..64): random shapes with N tails that
    cut a wave's rows, a workgroup's rows and the vector stores, K from one step to 128, against the torch fp32
    dequant-matmul, the first streaming kernel (same products, same order per output: bit-equal) and the float64
    oracle; and the shape the table sends there (N/128 about the number of compute units)."""
    rng = np.random.default_rng(815)
    cases = [(int(rng.integers(33, 65)), int(rng.integers(1, 300)) * int(rng.choice([1, 8, 16, 128])),
              int(rng.choice([128, 384, 1024, 4096, 7168, 16384]))) for _ in range(14)] + [(64, 28672, 4096), (40, 24576, 1536)]
    for case, (M, N, K) in enumerate(cases):
        print(f"gemm shared-activation stream case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=5000 + case, device="cuda")
        c = _run(xq, xs, wq, ws, "xshare")
        assert not torch.isnan(c.float()).any()
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(c.float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (M, N, K, cos, rel)
        if K <= 2048:   # the first kernel adds a wave's K steps first and the four waves' sums after: same only for few steps
            assert (c.float() - _run(xq, xs, wq, ws, "skinny").float()).abs().max() <= ref.abs().max() * 2 ** -7
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 4)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)
    # the table sends 33..64 rows there when N alone gives more 256-row tiles than compute units
    xq, xs, wq, ws = _prep(64, 66048, 1024, seed=77, device="cuda")
    assert torch.equal(_run(xq, xs, wq, ws, None).view(torch.int16), _run(xq, xs, wq, ws, "xshare").view(torch.int16))


def test_rows128_stream_kernel(hip):
    """The weight stream with the activation block in LDS (M <= 384; 256 weight rows per workgroup up to 128 rows,
    128 beyond, other widths where they make a single round): random shapes - every row-block
    count, N tails that cut a wave's rows, a workgroup's rows and the vector stores, K from one step (fewer
    steps than ring slots) to 144 so that whole-K and shared-K launches (second launch adds the partial sums) both
    occur - against the torch fp32 dequant-matmul, the float64 oracle on a sample and the 128x128 tile (same
    products in the same order when neither shares K: bit-equal); twice in a row (no state is left behind)."""
    from lightllm_amd import _lib

    rng = np.random.default_rng(2718)
    cases = [(int(rng.integers(1, 129)), int(rng.integers(1, 300)) * int(rng.choice([1, 8, 16, 32, 128])),
              int(rng.choice([128, 256, 384, 640, 1024, 2048, 4096, 7168, 18432]))) for _ in range(20)]
    cases += [(int(rng.integers(129, 385)), int(rng.integers(1, 300)) * int(rng.choice([1, 4, 8, 16, 128])),
               int(rng.choice([128, 256, 640, 1024, 2048, 7168, 18432]))) for _ in range(18)]
    cases += [(128, 256, 128), (65, 4096, 14336), (127, 2112, 7168), (80, 520, 2304), (256, 128, 128), (129, 7168, 2048),
              (100, 160 * 200 + 8, 640), (40, 192 * 230 - 3, 512), (128, 160 * 141, 256),   # 160- and 192-row workgroups
              (255, 2112, 7168), (144, 1000, 4096), (384, 640, 4096), (257, 136, 256), (383, 4100, 2048),
              # 129..208 rows, one round of 64- to 112-row workgroups (one 16-row block per wave) ...
              (130, 9100, 384), (192, 16384 - 7, 256), (208, 20000, 640), (150, 24576 - 1, 128), (176, 28672 - 20, 256),
              # ... or of 160- to 256-row ones (two blocks per wave) where N is wider
              (144, 36864 - 5, 256), (208, 45000, 128), (160, 52003, 256), (199, 65536 - 9, 128)]
    shared = 0
    for case, (M, N, K) in enumerate(cases):
        print(f"gemm rows128 case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=6000 + case, device="cuda")
        c = _run(xq, xs, wq, ws, "rows128").clone()
        assert not torch.isnan(c.float()).any()
        assert torch.equal(c, _run(xq, xs, wq, ws, "rows128"))
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(c.float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (M, N, K, cos, rel)
        t = _run(xq, xs, wq, ws, "tile128")
        split_here = _lib.lib().mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_ROWS128) > 0
        split_there = _lib.lib().mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_TILE128) > 0
        shared += split_here
        if not split_here and not split_there:
            assert torch.equal(c.view(torch.int16), t.view(torch.int16)), (M, N, K)
        else:
            assert (c.float() - t.float()).abs().max() <= ref.abs().max() * 2 ** -7, (M, N, K)
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 4)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)
    assert 4 <= shared <= len(cases) - 4, "both launch kinds must occur"


def test_rows128_column_major_scales(hip):
    print("gemm rows128 column-major scales", flush=True)
    xq, xs, wq, ws = _prep(100, 512, 2048, seed=78)
    xs_cm = xs.t().contiguous().t()
    C = _run(xq, xs_cm, wq, ws, "rows128")
    _check_small(xq, xs, wq, ws, C)
    assert torch.equal(C, _run(xq, xs, wq, ws, "rows128"))


@pytest.mark.parametrize("M,N,K", [(128, 36864, 7168), (100, 7168, 18432), (64, 7168, 16384), (65, 4096, 14336),
                                   (128, 2112, 7168), (200, 7168, 18432), (160, 28672, 4096), (129, 2112, 7168),
                                   (192, 36864, 7168), (208, 24576, 1536),
                                   (200, 6144, 4096), (384, 4096, 14336), (300, 7168, 16384), (48, 24576, 1536),
                                   (64, 28672, 4096), (24, 36864, 1024), (48, 10240, 8192), (64, 14336, 4096), (24, 7168, 18432), (32, 18432, 7168)])
def test_rows128_where_the_table_sends_it(hip, M, N, K):
    """Model linears with 33..384 rows that the shape table gives to the weight stream with the activation block in
    LDS."""
    print(f"gemm rows128 table shape M={M} N={N} K={K}", flush=True)
    _check_full(M, N, K, None, seed=M + N % 89)
    xq, xs, wq, ws = _prep(M, N, K, seed=1)
    assert torch.equal(_run(xq, xs, wq, ws, None).view(torch.int16), _run(xq, xs, wq, ws, "rows128").view(torch.int16))


def test_rows_tiled_over_m(hip):
    """The weight stream with the activation block in LDS, tiled over M as well (more than 384 rows on a narrow N, one
    round of tiles, K unshared): every row-block count 1..8 on three ring slots and 9..13 on two, 5-, 6-, 7- and
    8-wave workgroups, ragged last row tiles, N tails that cut a workgroup's rows and the vector stores, K from fewer
    steps than ring slots to 56 - against the torch fp32 dequant-matmul, the float64 oracle on a sample and the
    128x128 tile (same products in the same order when that does not share K: bit-equal); twice in a row."""
    from lightllm_amd import _lib

    rng = np.random.default_rng(31415)
    cases = [(512, 4096, 4096), (1000, 2112, 4096), (4096, 1024, 1536), (700, 3072, 7168), (3001, 576, 2048),
             (2048, 4096 - 24, 512), (401, 5120, 640), (4096, 2112, 7168), (1500, 1536 + 4, 256), (2500, 1000, 128),
             (6000, 1024, 384), (8192, 512, 1024), (1024, 2049, 2048), (3333, 3333, 384),
             # 7 row blocks; 9 on 7 waves; 11 on 6 waves; 13 on 5 waves (a single column of tiles)
             (3000, 2112, 1024), (5000, 1568, 512), (44000, 190, 256), (52000, 150, 128)]
    cases += [(int(rng.integers(385, 5000)), int(rng.integers(3, 160)) * int(rng.choice([1, 8, 32])),
               int(rng.choice([128, 256, 640, 1024, 2048, 4096]))) for _ in range(12)]
    lib = _lib.lib()
    seen = set()
    for case, (M, N, K) in enumerate(cases):
        print(f"gemm rows tiled over M case {case}: M={M} N={N} K={K}", flush=True)
        xq, xs, wq, ws = _prep(M, N, K, seed=6400 + case, device="cuda")
        try:
            c = _run(xq, xs, wq, ws, "rowsm").clone()
        except ValueError:
            continue                          # no one-round plan for this shape: a forced call is refused
        seen.add(case)
        assert not torch.isnan(c.float()).any()
        assert torch.equal(c, _run(xq, xs, wq, ws, "rowsm"))
        if case % 4 == 0:
            assert torch.equal(c, _run(xq, xs.t().contiguous().t(), wq, ws, "rowsm"))    # column-major activation scales
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        cos, rel = H.gemm_metrics(c.float(), ref)
        assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (M, N, K, cos, rel)
        t = _run(xq, xs, wq, ws, "tile128")
        if lib.mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_TILE128) == 0:
            assert torch.equal(c.view(torch.int16), t.view(torch.int16)), (M, N, K)
        else:
            assert (c.float() - t.float()).abs().max() <= ref.abs().max() * 2 ** -7, (M, N, K)
        rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 6)])
        cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
        ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                              ws.cpu().numpy(), np.arange(len(rows)), cols)
        got = c[rows][:, cols].float().cpu().double().numpy()
        assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * max(np.abs(ref64).max(), 1e-6)
    assert len(seen) >= 20 and set(range(18)) <= seen, sorted(seen)


@pytest.mark.parametrize("M,N,K", [(512, 4096, 4096), (1024, 2112, 7168), (2048, 4096, 4096), (768, 3584, 3584),
                                   (1024, 1024, 4096), (600, 5120, 5120)])
def test_rows_tiled_over_m_where_the_table_sends_it(hip, M, N, K):
    print(f"gemm rows tiled over M, table shape M={M} N={N} K={K}", flush=True)
    from lightllm_amd import _lib

    assert _lib.lib().mi355_block_fp8_gemm_variant(M, N, K) == _lib.GEMM_ROWS_MTILED
    _check_full(M, N, K, None, seed=M + N % 89)
    xq, xs, wq, ws = _prep(M, N, K, seed=1)
    assert torch.equal(_run(xq, xs, wq, ws, None).view(torch.int16), _run(xq, xs, wq, ws, "rowsm").view(torch.int16))


def test_unit_scales_is_plain_matmul(hip):
    """All scales 1: the result is the plain product of the fp8 values, exact in fp32 for K=128."""
    print("gemm unit scales", flush=True)
    g = H.gen(21)
    M, N, K = 48, 256, 128
    a = torch.randint(-8, 9, (M, K), generator=g).float().to(torch.float8_e4m3fn).cuda()
    b = torch.randint(-8, 9, (N, K), generator=g).float().to(torch.float8_e4m3fn).cuda()
    ones_a = torch.ones((M, 1), dtype=torch.float32, device="cuda")
    ones_b = torch.ones((2, 1), dtype=torch.float32, device="cuda")
    for variant in [None, "tile128", "tile256", "skinny", "rows128", "generic"]:
        C = _run(a, ones_a, b, ones_b, variant)
        ref = (a.float().cpu().double() @ b.float().cpu().double().T)
        # integers up to 128*64 = 8192 need 13 bits; bf16 keeps 8: compare after the same rounding
        assert torch.equal(C.cpu(), ref.float().to(torch.bfloat16)), variant


def test_one_hot_rows_pick_scaled_columns(hip):
    """A = one-hot rows with value 1: C[m,n] = As[m,kb] * Bs[n/128,kb] * B[n,k_m], one product, no sum."""
    print("gemm one-hot", flush=True)
    g = H.gen(22)
    M, N, K = 40, 384, 512
    wq, ws = H.quantized_weights(N, K, seed=23, device="cuda")
    ks = torch.randint(0, K, (M,), generator=g)
    a = torch.zeros((M, K), dtype=torch.float32)
    a[torch.arange(M), ks] = 1.0
    aq = a.to(torch.float8_e4m3fn).cuda()
    As = (torch.rand((M, K // 128), generator=g) + 0.5).cuda()
    for variant in [None, "tile128", "skinny", "rows128"]:
        C = _run(aq, As, wq, ws, variant)
        kb = (ks // 128).cuda()
        sa = As[torch.arange(M, device="cuda"), kb]                       # [M]
        sb = ws.repeat_interleave(128, 0)[:N][:, kb].T                      # [M,N]
        wv = wq.float()[:, ks.cuda()].T                                     # [M,N]
        ref = (wv * sa[:, None] * sb)
        got = C.float()
        # one fp32 product chain then a bf16 rounding: at most 1 bf16 ulp from either multiplication order
        assert torch.all((got - ref).abs() <= ref.abs() * 2 ** -7 + 1e-30), variant


@pytest.mark.parametrize("M,N,K", [(128, 512, 4096), (200, 640, 8192), (65, 256, 2048)])
def test_mid_m_split_k_tiles(hip, M, N, K):
    """Few 128x128 tiles and a long K: the tiled kernel shares the K range between CTAs.  (The shape table sends
    at most 128 rows with K >= 2048 to the 256-weight-row stream instead.)"""
    print(f"gemm mid-M split-K M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + K)
    C1 = _run(xq, xs, wq, ws, None).clone()
    C2 = _run(xq, xs, wq, ws, "tile128").clone()
    assert torch.equal(C1, _run(xq, xs, wq, ws, "rows128" if M <= 128 else "tile128"))
    assert torch.equal(C2, _run(xq, xs, wq, ws, "tile128"))
    assert (C1.float() - C2.float()).abs().max() <= C2.float().abs().max() * 2 ** -7
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(C1.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    rows, cols = np.arange(0, M, 7), np.arange(0, N, 5)
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy(), rows, cols)
    got = C1[rows][:, cols].float().cpu().double().numpy()
    assert np.abs(got - ref64).max() / np.abs(ref64).max() <= H.GEMM_MAX_REL


@pytest.mark.parametrize("M,N,K", [(768, 2112, 8192), (1024, 2112, 7168), (300, 520, 4096)])
def test_256x128_tiles_with_shared_k(hip, M, N, K):
    """256x128 tiles whose K range is shared between workgroups (few tiles, long K): against the torch fp32
    dequant-matmul, the float64 oracle on a sample and the 128x128 tiles; repeated calls agree bit for bit.  The
    shape table sends narrow-N shapes with many rows there."""
    from lightllm_amd import _lib

    print(f"gemm 256x128 split-K M={M} N={N} K={K}", flush=True)
    assert _lib.lib().mi355_block_fp8_gemm_workspace_bytes(M, N, K, _lib.GEMM_TILE256x128) > 0
    xq, xs, wq, ws = _prep(M, N, K, seed=M + K)
    C1 = _run(xq, xs, wq, ws, "tile256x128").clone()
    assert torch.equal(C1, _run(xq, xs, wq, ws, "tile256x128"))
    if M == 768:
        assert torch.equal(C1, _run(xq, xs, wq, ws, None))
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(C1.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    assert (C1.float() - _run(xq, xs, wq, ws, "tile128").float()).abs().max() <= ref.abs().max() * 2 ** -7
    rows, cols = np.arange(0, M, 37), np.arange(0, N, 11)
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq), xs.cpu().numpy(), tr.bits_of(wq), ws.cpu().numpy(), rows, cols)
    got = C1[rows][:, cols].float().cpu().double().numpy()
    assert np.abs(got - ref64).max() / np.abs(ref64).max() <= H.GEMM_MAX_REL


@pytest.mark.parametrize("M,N,K", [(512, 36864, 1024), (400, 36864 + 72, 2048), (768, 24576, 1536), (300, 36864, 2048),
                                   (1024, 36864, 1024)])
def test_rest_of_a_round_runs_as_its_own_launch(hip, M, N, K):
    """256x256 tiles that fill the device once (or twice) and leave a small rest: the table runs the rest (the last weight
    rows) as a second launch with the kernel its own shape gets.  Same products in the same order per output as
    the one-launch 256x256 tiles when that kernel does not share K, close to it otherwise; fp32 reference and
    float64 oracle as everywhere."""
    from lightllm_amd import _lib

    print(f"gemm rest-of-a-round split M={M} N={N} K={K}", flush=True)
    cus = _lib.device_info()["compute_units"]
    t256 = -(-M // 256) * -(-N // 256)
    rounds, rest = divmod(t256, cus)
    if not (rounds in (1, 2) and 0 < rest * 2 * rounds <= cus):
        pytest.skip("shape chosen for 256 compute units")
    xq, xs, wq, ws = _prep(M, N, K, seed=M + K)
    c = _run(xq, xs, wq, ws, None).clone()
    assert not torch.isnan(c.float()).any()
    assert torch.equal(c, _run(xq, xs, wq, ws, None))
    one = _run(xq, xs, wq, ws, "tile256")
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    if K // 128 < 16:
        assert torch.equal(c.view(torch.int16), one.view(torch.int16))
    else:
        assert (c.float() - one.float()).abs().max() <= ref.abs().max() * 2 ** -7
    cos, rel = H.gemm_metrics(c.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    rng = np.random.default_rng(M)
    rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 6)])
    cols = np.unique(np.r_[0, N - 1, N - 4096, N - 4097, rng.integers(0, N, 60)])
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                          ws.cpu().numpy(), np.arange(len(rows)), cols)
    got = c[rows][:, cols].float().cpu().double().numpy()
    assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * np.abs(ref64).max()


def test_split_k_is_deterministic_and_reusable(hip):
    """The split-K path reduces in a fixed order and leaves its workspace counters zero: repeated calls agree bit for bit."""
    print("gemm split-k determinism", flush=True)
    xq, xs, wq, ws = _prep(64, 4096, 14336, seed=31)
    outs = [_run(xq, xs, wq, ws, "skinny").clone() for _ in range(3)]
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(outs[0].float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)


def _check_full(M, N, K, variant, seed):
    xq, xs, wq, ws = _prep(M, N, K, seed=seed)
    C = _run(xq, xs, wq, ws, variant)
    assert not torch.isnan(C.float()).any()
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)     # torch fp32 on the GPU
    cos, rel = H.gemm_metrics(C.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (variant, cos, rel)
    del ref
    rng = np.random.default_rng(seed)
    rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 14)])
    cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 126)])
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                          ws.cpu().numpy(), np.arange(len(rows)), cols)
    got = C[rows][:, cols].float().cpu().double().numpy()
    scale = np.abs(ref64).max()
    assert np.abs(got - ref64).max() / scale <= H.GEMM_MAX_REL


@pytest.mark.parametrize("M", [1, 8, 32, 64])
@pytest.mark.parametrize("N,K", [(28672, 4096), (4096, 14336)])
def test_llama_decode_shapes(hip, M, N, K):
    print(f"gemm llama M={M} N={N} K={K}", flush=True)
    _check_full(M, N, K, None, seed=M + 5)


@pytest.mark.parametrize("M,N,K", [(64, 16384, 8192), (8, 16384, 8448), (20, 1024, 4736), (33, 2048, 7168)])
def test_stream_kernel_scale_staging(hip, M, N, K):
    """The M <= 64 kernel stages the activation scales of a CTA's K range in LDS when the range is short enough
    (59 steps at M > 32, else 64) and gathers them per step otherwise: both paths, an uneven K split (37 steps
    over 2 CTAs) and a 56-step range just under the limit."""
    print(f"gemm stream scale staging M={M} N={N} K={K}", flush=True)
    _check_full(M, N, K, "skinny", seed=M + 3)


def test_stream_kernel_column_major_scales(hip):
    print("gemm stream column-major scales", flush=True)
    xq, xs, wq, ws = _prep(24, 512, 2048, seed=77)
    xs_cm = xs.t().contiguous().t()
    C = _run(xq, xs_cm, wq, ws, "skinny")
    _check_small(xq, xs, wq, ws, C)
    assert torch.equal(C, _run(xq, xs, wq, ws, "skinny"))


@pytest.mark.parametrize("N,K,variant", [(36864, 7168, "tile256"), (7168, 18432, None), (2112, 7168, None),
                                         (2112, 7168, "tile256"), (7168, 18432, "tile256x128")])
def test_deepseek_prefill_shapes(hip, N, K, variant):
    print(f"gemm dsv3 M=4096 N={N} K={K} variant={variant}", flush=True)
    _check_full(4096, N, K, variant, seed=N % 97)


@pytest.mark.parametrize("bn,bk", [(64, 64), (128, 64), (32, 256), (64, 96)])
def test_other_block_sizes(hip, bn, bk):
    """Weight blocks other than 128x128 (the reference kernel takes any block_size, fp8w8a8_block_gemm_kernel.py:100-123):
    the plain kernel against the C oracle's fp32 per-block order (bit-equal bf16) and the float64 dequant-matmul,
    with an N tail inside a block and a partial last K block."""
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    print(f"gemm block sizes bn={bn} bk={bk}", flush=True)
    M, N, K = 37, 200, 3 * bk + bk // 2
    g = H.gen(900 + bn + bk)
    a = torch.randint(0, 256, (M, K), generator=g, dtype=torch.int32)
    b = torch.randint(0, 256, (N, K), generator=g, dtype=torch.int32)
    a[(a & 0x7F) == 0x7F] = 0x38       # no e4m3fn NaN bytes
    b[(b & 0x7F) == 0x7F] = 0xB8
    aq = a.to(torch.uint8).cuda().view(torch.float8_e4m3fn)
    bq = b.to(torch.uint8).cuda().view(torch.float8_e4m3fn)
    kb, nb = -(-K // bk), -(-N // bn)
    As = (torch.rand((M, kb), generator=g) * 0.02 + 0.001).cuda()
    Bs = (torch.rand((nb, kb), generator=g) * 0.02 + 0.001).cuda()
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(aq, bq.t(), As, Bs.t(), C, [bk, bn])
    torch.cuda.synchronize()
    want = oracle.block_gemm(tr.bits_of(aq), As.cpu().numpy(), tr.bits_of(bq), Bs.cpu().numpy(), bn=bn, bk=bk)
    got = C.view(torch.int16).cpu().numpy().view(np.uint16)
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(aq), As.cpu().numpy(), tr.bits_of(bq), Bs.cpu().numpy(),
                                          np.arange(M), np.arange(N), bn=bn, bk=bk)
    assert np.abs(C.float().cpu().double().numpy() - ref64).max() <= H.GEMM_MAX_REL * np.abs(ref64).max()
    # same fp32 order per block up to the order inside a block: within one bf16 ulp of the oracle's result
    wf = tr.bf16_from_bits(want).float()
    assert (C.float().cpu() - wf).abs().max() <= wf.abs().max() * 2 ** -7
    with pytest.raises(ValueError):
        w8a8_block_fp8_matmul(aq, bq.t(), As, Bs.t(), C, [bk, bn], run_config={"variant": "tile128"})


def test_generic_strides(hip):
    """B given as a contiguous [K,N] tensor (not the transposed weight view) and row-strided A-scales."""
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    print("gemm generic strides", flush=True)
    xq, xs, wq, ws = _prep(24, 256, 384, seed=41)
    Bkn = wq.t().contiguous()                 # strides (N,1)
    Bs_kn = ws.t().contiguous()
    xs_cm = xs.t().contiguous().t()           # column-major scales
    C = torch.empty((24, 256), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(xq, Bkn, xs_cm, Bs_kn, C, [128, 128])
    torch.cuda.synchronize()
    _check_small(xq, xs, wq, ws, C)
    C2 = _run(xq, xs_cm, wq, ws, "tile128")   # fast kernel with column-major activation scales
    _check_small(xq, xs, wq, ws, C2)


@pytest.mark.parametrize("variant,M,N,K", [("rows128", 100, 1000, 2048), ("rows128", 300, 640, 4096), ("rows128", 64, 160 * 150, 256),
                                           ("tile128", 200, 520, 4096), ("tile256", 300, 520, 1024), ("tile256x128", 768, 520, 4096),
                                           ("skinny", 20, 1000, 4096), ("streamcu", 12, 4096, 4096), ("xshare", 40, 4096, 1024), ("tile256streamk", 600, 1024, 8192),
                                           ("rowsm", 700, 1000, 2048), ("rowsm", 3000, 2112, 512), (None, 512, 36864, 256)])
def test_padded_rows_through_the_c_abi(hip, variant, M, N, K):
    """Operands whose rows are longer than they need be (lda > K, ldb_n > K, ldc > N, padded scale rows), as a
    caller that slices larger buffers passes them: every fast kernel against its own result on packed operands
    (same kernel, same order: bit-equal), and nothing written into the padding of C."""
    from lightllm_amd import _lib
    from lightllm_amd.quantization.fp8w8a8_block_gemm_kernel import _VARIANTS

    print(f"gemm padded rows variant={variant} M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + N)
    want = _run(xq, xs, wq, ws, variant).clone()
    xq_p = torch.zeros((M, K + 128), dtype=torch.uint8, device="cuda")
    xq_p[:, :K] = xq.view(torch.uint8)
    wq_p = torch.zeros((N, K + 256), dtype=torch.uint8, device="cuda")
    wq_p[:, :K] = wq.view(torch.uint8)
    xs_p = torch.zeros((M, K // 128 + 3), dtype=torch.float32, device="cuda")
    xs_p[:, :K // 128] = xs
    ws_p = torch.zeros((ws.shape[0], K // 128 + 5), dtype=torch.float32, device="cuda")
    ws_p[:, :K // 128] = ws
    out = torch.full((M, N + 8), 7.0, dtype=torch.bfloat16, device="cuda")
    code = _VARIANTS[variant]
    need = hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, code)
    wsp = torch.zeros(max(need, 16), dtype=torch.uint8, device="cuda")
    rc = hip.mi355_block_fp8_gemm(xq_p.data_ptr(), wq_p.data_ptr(), xs_p.data_ptr(), ws_p.data_ptr(), out.data_ptr(), M, N, K,
                                  xq_p.stride(0), 1, wq_p.stride(0), out.stride(0), xs_p.stride(0), 1, 1, ws_p.stride(0),
                                  128, 128, wsp.data_ptr(), wsp.numel(), code, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0, hip.mi355_error_string(rc)
    assert torch.equal(out[:, :N].contiguous().view(torch.int16), want.view(torch.int16))
    assert bool((out[:, N:] == 7.0).all())
    assert not bool(wsp[:_lib.WS_COUNTER_BYTES].any()) if need >= _lib.WS_COUNTER_BYTES else True


def test_preconditions(hip):
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    xq, xs, wq, ws = _prep(16, 256, 256, seed=51)
    C = torch.empty((16, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        w8a8_block_fp8_matmul(xq, wq.t(), xs[:, :1], ws.t(), C, [128, 128])
    with pytest.raises(AssertionError):
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), C.t(), [128, 128])
    with pytest.raises(AssertionError):
        w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), C, [128])


def test_quant_method_apply(hip):
    """The plug-in object end to end: quantize a bf16 weight, apply to bf16 activations."""
    from lightllm_amd.quantization import QUANTMETHODS

    print("quant method apply", flush=True)
    method = QUANTMETHODS.get("fp8w8a8-b128")
    pack, parts = method.create_weight([512, 256], 1024, torch.bfloat16, 0)
    w = H.weights(768, 1024, seed=61).cuda()
    method.load_weight(w, pack)
    assert pack.load_ok == [True, True, True] and parts[1].weight.shape == (256, 1024)
    x = H.activations(40, 1024, seed=62).cuda()
    out = method.apply(x, pack)
    torch.cuda.synchronize()
    ref = x.float() @ w.float().T
    cos = tr.cosine(out.float(), ref)
    assert out.shape == (40, 768) and cos > 0.999, cos     # quantization error of fp8 itself
    # and it is exactly the composition of the three kernels
    from lightllm_amd.quantization import per_token_group_quant_fp8

    xq, xs = per_token_group_quant_fp8(x, 128)
    C = _run(xq, xs, pack.weight, pack.weight_scale)
    assert torch.equal(C, out)
    # an fp16 model: fp16 activations are quantized as they are and the output comes back in fp16 (w8a8.py:507-529)
    x16 = x.to(torch.float16)
    out16 = method.apply(x16, pack)
    torch.cuda.synchronize()
    assert out16.dtype == torch.float16 and out16.shape == (40, 768)
    assert tr.cosine(out16.float(), ref) > 0.999


@pytest.mark.parametrize("variant,M,N,K", [("tile256", 300, 1000, 1152), ("tile256once", 512, 512, 1024), ("tile128", 130, 520, 512),
                                           ("tile256x128", 260, 300, 256), ("skinny", 9, 1000, 2048), ("skinny", 40, 4100, 4096),
                                           ("xshare", 50, 4096, 1024), ("tile256streamk", 1000, 2048, 16384),
                                           ("rows128", 100, 1000, 512), ("rows128", 128, 4104, 14336), ("rows128", 250, 1004, 4096),
                                           ("rowsm", 900, 1004, 1024), ("rowsm", 3000, 2112, 512),
                                           ("generic", 7, 130, 256), (None, 64, 28672, 4096), (None, 1024, 2112, 7168)])
def test_fp16_output(hip, variant, M, N, K):
    """C in fp16: the fp32 accumulator is cast to the dtype of C (fp8w8a8_block_gemm_kernel.py:78; LightLLM allocates C
    in the activations' dtype).  Every kernel against the same launch with bf16 output - the fp16 values must be the
    fp16 rounding of a number whose bf16 rounding is the bf16 result - and against the float64 oracle on a sample."""
    print(f"gemm fp16 out variant={variant} M={M} N={N} K={K}", flush=True)
    xq, xs, wq, ws = _prep(M, N, K, seed=M + N + K)
    c16 = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    from lightllm_amd.quantization import w8a8_block_fp8_matmul

    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), c16, [128, 128], dtype=torch.float16,
                          run_config={"variant": variant} if variant else None)
    torch.cuda.synchronize()
    cb = _run(xq, xs, wq, ws, variant)
    assert not torch.isnan(c16.float()).any()
    # same accumulator, two roundings: they agree to bf16 precision, and fp16 is the finer one
    assert (c16.float() - cb.float()).abs().max() <= 2 ** -8 * cb.float().abs().max()
    ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
    cos, rel = H.gemm_metrics(c16.float(), ref)
    assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)
    e16 = (c16.float() - ref).abs().mean()
    eb = (cb.float() - ref).abs().mean()
    assert e16 <= eb, (float(e16), float(eb))   # three more mantissa bits than bf16
    rng = np.random.default_rng(M)
    rows = np.unique(np.r_[0, M - 1, rng.integers(0, M, 4)])
    cols = np.unique(np.r_[0, N - 1, rng.integers(0, N, 30)])
    ref64 = oracle.dequant_matmul_sampled(tr.bits_of(xq[rows].contiguous()), xs[rows].cpu().numpy(), tr.bits_of(wq),
                                          ws.cpu().numpy(), np.arange(len(rows)), cols)
    got = c16[rows][:, cols].float().cpu().double().numpy()
    assert np.abs(got - ref64).max() <= H.GEMM_MAX_REL * np.abs(ref64).max()

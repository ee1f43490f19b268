"""mi355_block_fp8_gemm_noalloc (scratch inside the library's device image) against mi355_block_fp8_gemm (caller's
workspace), through the C ABI: same bits on two calls in a row, the second with a smaller input; sizes beyond the
fixed scratch are refused."""
import ctypes

import pytest
import torch

from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _operands(M, N, K, seed):
    from lightllm_amd.quantization import per_token_group_quant_fp8

    xq, xs = per_token_group_quant_fp8(H.activations(M, K, seed=seed).cuda(), 128)
    wq, ws = H.quantized_weights(N, K, seed=seed + 1, device="cuda")
    return xq, xs, wq, ws


def _call(lib, name, xq, xs, wq, ws, out, variant, workspace=None):
    M, K = xq.shape
    N = wq.shape[0]
    head = [xq.data_ptr(), wq.data_ptr(), xs.data_ptr(), ws.data_ptr(), out.data_ptr(), M, N, K,
            xq.stride(0), 1, wq.stride(0), out.stride(0), xs.stride(0), xs.stride(1), 1, ws.stride(0), 128, 128]
    stream = torch.cuda.current_stream().cuda_stream
    if name == "mi355_block_fp8_gemm":
        tail = [workspace.data_ptr() if workspace is not None else None,
                workspace.numel() if workspace is not None else 0, variant, stream]
    else:
        tail = [variant, stream]
    return getattr(lib, name)(*head, *tail)


# (M, N, K, variant): a K-split stream launch, a smaller one, a split-K 128x128 launch, a persistent 256x256 launch
CASES = [(32, 4096, 14336, 0), (24, 2048, 7168, 0), (200, 640, 8192, 2), (4096, 8192, 1024, 1)]


def test_noalloc_entry_point_matches_the_workspace_one(hip):
    from lightllm_amd import _lib

    for (M, N, K, variant) in CASES:
        print(f"noalloc gemm M={M} N={N} K={K} variant={variant}", flush=True)
        xq, xs, wq, ws = _operands(M, N, K, seed=M + N)
        need = hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, variant)
        assert need > 0, "the case must use the scratch"
        workspace = torch.zeros(need, dtype=torch.uint8, device="cuda")
        want = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert _call(hip, "mi355_block_fp8_gemm", xq, xs, wq, ws, want, variant, workspace) == 0
        for rep in range(2):
            got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
            assert _call(hip, "mi355_block_fp8_gemm_noalloc", xq, xs, wq, ws, got, variant) == 0
            torch.cuda.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K, variant, rep)
    # beyond the fixed scratch: a clear error, nothing launched
    M, N, K = 128, 7168, 18432
    need = hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, 2)
    assert need > _lib.WS_COUNTER_BYTES + (8 << 20)
    xq, xs, wq, ws = _operands(M, N, K, seed=3)
    out = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    rc = _call(hip, "mi355_block_fp8_gemm_noalloc", xq, xs, wq, ws, out, 2)
    torch.cuda.synchronize()
    assert rc == -7 and b"scratch" in hip.mi355_error_string(rc)
    assert not bool(out.any())
    # the shape table itself never fails for want of scratch: it takes a plan that fits.  The shapes after the
    # first are ones whose first choice (the weight stream with K shared) needs more than the scratch and whose
    # second is a stream-K plan that needs more still; every one of them must end in a kernel that runs - through
    # the scratch entry point and through the ordinary one without any workspace.
    for (M, N, K) in [(128, 7168, 18432), (200, 7168, 18432), (300, 4096, 14336), (384, 4096, 14336)]:
        print(f"noalloc AUTO M={M} N={N} K={K}", flush=True)
        assert hip.mi355_block_fp8_gemm_workspace_bytes(M, N, K, 0) > _lib.WS_COUNTER_BYTES + (8 << 20)
        xq, xs, wq, ws = _operands(M, N, K, seed=3 + M)
        out = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        ref = tr.dequant_matmul(xq, xs, wq, ws, out_dtype=torch.float32)
        for name in ("mi355_block_fp8_gemm_noalloc", "mi355_block_fp8_gemm_noalloc", "mi355_block_fp8_gemm"):
            out.fill_(float("nan"))
            assert _call(hip, name, xq, xs, wq, ws, out, 0) == 0, (name, M, N, K)
            torch.cuda.synchronize()
            cos, rel = H.gemm_metrics(out.float(), ref)
            assert cos >= H.GEMM_MIN_COS and rel <= H.GEMM_MAX_REL, (cos, rel)

"""Block-scaled FP8 GEMM: A scaled per 1x128 group, B per 128x128 block, fp32 accumulate, bf16 out.

Same name, arguments and layouts as
lightllm/common/basemodel/triton_kernel/quantization/fp8w8a8_block_gemm_kernel.py:127-192 of the reference;
the work is done by ``mi355_block_fp8_gemm`` (csrc/block_gemm.hip, csrc/gemm_tile.hpp).
"""
from typing import List, Optional

import torch

from .. import _lib

_VARIANTS = {
    None: _lib.GEMM_AUTO, "auto": _lib.GEMM_AUTO, "tile256": _lib.GEMM_TILE256, "tile128": _lib.GEMM_TILE128,
    "skinny": _lib.GEMM_SKINNY, "generic": _lib.GEMM_GENERIC, "tile256x128": _lib.GEMM_TILE256x128,
    "tile256ring": _lib.GEMM_TILE256_RING, "tile256once": _lib.GEMM_TILE256_ONCE,
    "tile256streamk": _lib.GEMM_TILE256_STREAMK, "xshare": _lib.GEMM_SKINNY_XSHARE, "rows128": _lib.GEMM_ROWS128, "streamcu": _lib.GEMM_SKINNY_CU, "rowsm": _lib.GEMM_ROWS_MTILED,
}


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def w8a8_block_fp8_matmul(
    A: torch.Tensor,
    B: torch.Tensor,
    Ascale: torch.Tensor,
    Bscale: torch.Tensor,
    C: torch.Tensor,
    block_size: List[int],
    dtype: torch.dtype = torch.bfloat16,
    run_config=None,
) -> torch.Tensor:
    """C = (A * Ascale) @ (B * Bscale), written into ``C`` and returned.

    A [M,K] e4m3fn contiguous; B [K,N] e4m3fn (LightLLM passes ``weight.t()``: strides (1,K));
    Ascale [M, K/128] fp32; Bscale [K/128, ceil(N/128)] fp32; C [M,N] bf16 or fp16 contiguous (the accumulator is
    cast to the dtype of ``C``).
    ``run_config`` may force a kernel: ``{"variant": "auto"|"tile256"|"tile256streamk"|"tile256x128"|"tile128"|
    "rows128"|"rowsm"|"xshare"|"skinny"|"streamcu"|"generic"}`` (plus the comparison variants "tile256ring" and
    "tile256once"); a forced kernel that cannot run the shape raises ``ValueError``.  The reference's tile
    dictionaries (BLOCK_M, ...) are accepted and ignored: the shape table is built in.
    """
    assert len(block_size) == 2
    block_k, block_n = block_size[0], block_size[1]
    assert A.shape[0] == Ascale.shape[0] and A.shape[-1] == B.shape[0]
    assert A.is_contiguous() and C.is_contiguous()
    M, K = A.shape
    _, N = B.shape
    assert _cdiv(K, block_k) == Ascale.shape[-1] and Ascale.shape[-1] == Bscale.shape[0]
    assert _cdiv(N, block_n) == Bscale.shape[1]
    assert C.shape[0] == M and C.shape[1] == N
    assert C.dtype in (torch.bfloat16, torch.float16), "the gfx950 kernels write bf16 or fp16"
    assert A.dtype == torch.float8_e4m3fn and B.dtype == torch.float8_e4m3fn
    assert Ascale.dtype == torch.float32 and Bscale.dtype == torch.float32
    _lib.require_cuda(A, B, Ascale, Bscale, C)
    variant = _lib.GEMM_AUTO
    if isinstance(run_config, dict) and "variant" in run_config:
        variant = _VARIANTS[run_config["variant"]]
    lib = _lib.lib()
    stream = _lib.stream_ptr(A.device)
    ws_ptr, ws_bytes = None, 0
    need = lib.mi355_block_fp8_gemm_workspace_bytes(M, N, K, variant)
    if need:
        ws = _lib.workspace(A.device, need, stream)
        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
    # the accumulator is cast to the dtype of C, like `accumulator.to(C.dtype.element_ty)` in the reference (:78)
    code = lib.mi355_block_fp8_gemm_dtype(
        A.data_ptr(), B.data_ptr(), Ascale.data_ptr(), Bscale.data_ptr(), C.data_ptr(), M, N, K,
        A.stride(0), B.stride(0), B.stride(1), C.stride(0),
        Ascale.stride(0), Ascale.stride(1), Bscale.stride(0), Bscale.stride(1),
        block_n, block_k, ws_ptr, ws_bytes, variant, _lib.DTYPE_CODES[C.dtype], stream,
    )
    _lib.check(code, "w8a8_block_fp8_matmul")
    return C

"""Load-time 128x128 block weight quantizer.

Same names and behaviour as
lightllm/common/basemodel/triton_kernel/quantization/fp8w8a8_block_quant_kernel.py:30-58 of the reference
(including its quirk: the stored scale is amax/448, the divisor is scale + 1e-6, no clamp);
the work is done by ``mi355_block_weight_quant_fp8`` (csrc/weight_quant.hip).
"""
from typing import Tuple

import torch

from .. import _lib

_DTYPES = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}


def mm_weight_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    assert x.is_contiguous(), "Input tensor must be contiguous"
    assert x.dtype in _DTYPES, f"unsupported weight dtype {x.dtype}"
    _lib.require_cuda(x)
    M, N = x.size()
    y_quant = torch.empty((M, N), dtype=torch.float8_e4m3fn, device=x.device)
    nbm, nbn = (M + block_size - 1) // block_size, (N + block_size - 1) // block_size
    s_scales = torch.empty((nbm, nbn), dtype=torch.float32, device=x.device)
    code = _lib.lib().mi355_block_weight_quant_fp8(
        x.data_ptr(), _DTYPES[x.dtype], y_quant.data_ptr(), s_scales.data_ptr(), M, N, block_size,
        _lib.stream_ptr(x.device),
    )
    _lib.check(code, "mm_weight_quant")
    return y_quant, s_scales


def weight_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    assert x.is_contiguous(), "Input tensor must be contiguous"
    if not x.is_cuda:
        x = x.cuda(torch.cuda.current_device())
    if x.dim() == 3:
        E, M, N = x.shape
        y_quant = torch.empty((E, M, N), dtype=torch.float8_e4m3fn, device=x.device)
        nbm, nbn = (M + block_size - 1) // block_size, (N + block_size - 1) // block_size
        s_scales = torch.empty((E, nbm, nbn), dtype=torch.float32, device=x.device)
        for i in range(E):
            y_quant[i], s_scales[i] = mm_weight_quant(x[i], block_size)
        return y_quant, s_scales
    return mm_weight_quant(x, block_size)

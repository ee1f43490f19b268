"""Inverse of the 128x128 block weight quantizer (load-time only).

Same name and arguments as ``weight_dequant`` of the reference
(lightllm/models/deepseek2/triton_kernel/weight_dequant.py:9-30); runs ``mi355_block_weight_dequant``.
"""
import torch

from .. import _lib


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """x e4m3fn [M, N], s fp32 [ceil(M/128), ceil(N/128)] -> bf16 [M, N] = x * s per block."""
    assert x.is_contiguous() and s.is_contiguous(), "Input tensors must be contiguous"
    assert x.dim() == 2 and s.dim() == 2, "Input tensors must have 2 dimensions"
    if block_size != 128:
        raise ValueError("weight_dequant: block_size must be 128 on gfx950")
    assert x.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    M, N = x.size()
    assert s.shape == ((M + 127) // 128, (N + 127) // 128)
    _lib.require_cuda(x, s)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    code = _lib.lib().mi355_block_weight_dequant(
        x.data_ptr(), s.data_ptr(), y.data_ptr(), M, N, block_size, _lib.stream_ptr(x.device)
    )
    _lib.check(code, "weight_dequant")
    return y

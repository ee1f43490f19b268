"""Activation quantizer: bf16 (fp16, fp32) -> float8_e4m3fn with one fp32 scale per 1x128 group.

Same names, arguments and tensor layouts as
lightllm/common/basemodel/triton_kernel/quantization/fp8act_quant_kernel.py (:63-113, :116-168, :216-236)
of the reference; the work is done by ``mi355_group_quant_fp8`` (csrc/group_quant.hip).
"""
from typing import Callable

import torch

from .. import _lib


def get_tma_aligned_size(x: int, element_size: int) -> int:
    """M padded so that a column of scales starts on a 16-byte boundary (reference :173-189)."""
    alignment = 16 // element_size
    return (x + alignment - 1) // alignment * alignment


def lightllm_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    x_q: torch.Tensor,
    x_s: torch.Tensor,
    eps: float = 1e-10,
    dtype: torch.dtype = torch.float8_e4m3fn,
):
    """Quantize ``x`` into the caller's ``x_q`` / ``x_s``; returns None.

    ``x_s`` is 2-D [M, K/group_size] with any strides: row-major and column-major are both written in place
    (the reference picks between them from ``x_s.is_contiguous()``, :83).
    """
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    assert dtype == torch.float8_e4m3fn, "only torch.float8_e4m3fn is supported"
    assert x.dtype in _lib.DTYPE_CODES, "activations must be bf16 (the fast path), fp16 or fp32"
    assert x_q.is_contiguous() and x_q.shape == x.shape and x_q.dtype == torch.float8_e4m3fn
    assert x_s.dtype == torch.float32
    _lib.require_cuda(x, x_q, x_s)
    xs_m, xs_n = x_s.shape  # 2-D like the reference (:84)
    K = x.shape[-1]
    M = x.numel() // K if K else 0
    assert xs_m == M and xs_n == K // group_size, "scale tensor shape must be [M, K // group_size]"
    code = _lib.lib().mi355_group_quant_fp8(
        x.data_ptr(), _lib.DTYPE_CODES[x.dtype], x_q.data_ptr(), x_s.data_ptr(), M, K, group_size, eps,
        x_s.stride(0), x_s.stride(1),
        _lib.stream_ptr(x.device),
    )
    _lib.check(code, "per_token_group_quant_fp8")
    return


def per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = torch.float8_e4m3fn,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    alloc_func: Callable = torch.empty,
):
    """-> (x_q, x_s).  Like the reference's own branch (:158-167) the floor is always 1e-10 and the output
    e4m3fn, whatever ``eps`` / ``dtype`` say; with both layout flags the scales come back as the [M, K/g]
    view of a [K/g, ceil4(M)] buffer (strides (1, ceil4(M))), written directly instead of transposed after."""
    x_q = alloc_func(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    groups = x.shape[-1] // group_size
    if column_major_scales and scale_tma_aligned:
        assert x.dim() == 2
        m = x.shape[0]
        padded = get_tma_aligned_size(m, 4)
        buf = alloc_func((groups, padded), device=x.device, dtype=torch.float32)
        x_s = buf.t()[:m]
    else:
        x_s = alloc_func(x.shape[:-1] + (groups,), device=x.device, dtype=torch.float32)
    x_s2 = x_s if x_s.dim() == 2 else x_s.view(-1, groups)
    lightllm_per_token_group_quant_fp8(x, group_size, x_q, x_s2, eps=1e-10, dtype=torch.float8_e4m3fn)
    return x_q, x_s


def tma_align_input_scale(input_scale: torch.Tensor) -> torch.Tensor:
    """Row-major [M, K/g] scales -> column-major view with M padded to 4 floats (reference :216-236).
    A strided copy; the quantizer can also write this layout directly."""
    assert input_scale.dim() == 2
    m, kdiv = input_scale.shape
    padded = get_tma_aligned_size(m, input_scale.element_size())
    output = torch.empty((kdiv, padded), dtype=input_scale.dtype, device=input_scale.device)
    output[:, :m].copy_(input_scale.t())
    return output.t()[:m]

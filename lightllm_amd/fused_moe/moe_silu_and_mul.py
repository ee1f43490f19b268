"""SiLU-and-mul between the two expert / FFN GEMMs.

Same name and arguments as ``silu_and_mul_fwd`` of the reference
(lightllm/common/basemodel/triton_kernel/fused_moe/moe_silu_and_mul.py:117-176); the work is done by
``mi355_silu_and_mul`` (the "blocked" [gate | up] layout without limit/alpha: the path the fp8 block-quantized
layers take, a streaming kernel) and ``mi355_silu_and_mul_ex`` (the "interleaved" layout and the clamped
limit/alpha variant, one element per lane).  The tanh-GELU switch of the reference is not implemented.
"""
import torch

from .. import _lib


def silu_and_mul_fwd(input: torch.Tensor, output: torch.Tensor, layout="blocked", limit=None, alpha=None,
                     run_config=None):
    """output[m, :] = bf16(silu(input[m, :H])) * input[m, H:], H = input.shape[-1] // 2; with ``limit``/``alpha``
    the clamped form (up + 1) * gate * sigmoid(alpha * gate); ``layout="interleaved"`` reads [g0, u0, g1, u1, ...].

    ``run_config`` (the reference's tile dictionary) is accepted and ignored.
    """
    assert input.stride(-1) == 1
    assert output.is_contiguous()
    assert (limit is None and alpha is None) or (limit is not None and alpha is not None)
    if layout not in ("blocked", "interleaved"):
        raise ValueError(f"silu_and_mul_fwd: unknown layout {layout!r}")
    assert input.dtype == torch.bfloat16 and output.dtype == torch.bfloat16
    assert input.ndim == 2 and output.ndim == 2
    size_m, size_n = input.shape[0], input.shape[-1] // 2
    assert output.shape[0] == size_m and output.shape[1] == size_n
    _lib.require_cuda(input, output)
    if layout == "blocked" and limit is None:
        code = _lib.lib().mi355_silu_and_mul(
            input.data_ptr(), output.data_ptr(), size_m, size_n, input.stride(0), output.stride(0),
            _lib.stream_ptr(input.device),
        )
    else:
        code = _lib.lib().mi355_silu_and_mul_ex(
            input.data_ptr(), output.data_ptr(), size_m, size_n, input.stride(0), output.stride(0),
            1 if layout == "interleaved" else 0, 0 if limit is None else 1,
            0.0 if limit is None else float(limit), 0.0 if alpha is None else float(alpha),
            _lib.stream_ptr(input.device),
        )
    _lib.check(code, "silu_and_mul_fwd")
    return

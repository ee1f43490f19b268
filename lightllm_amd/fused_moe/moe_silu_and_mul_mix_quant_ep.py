"""SiLU-and-mul fused with the 1x128 group quantizer.

``silu_and_mul_masked_post_quant_fwd`` has the name, arguments and layouts of the reference
(lightllm/common/basemodel/triton_kernel/fused_moe/moe_silu_and_mul_mix_quant_ep.py:78-141);
``silu_and_mul_post_quant_fwd`` is the same operation on a flat [M, 2H] tensor, used between the two
grouped GEMMs so that the bf16 intermediate never goes to memory.  Both run ``mi355_silu_and_mul_group_quant_fp8``
and give exactly the bytes and scales of silu_and_mul_fwd followed by per_token_group_quant_fp8.
"""
import torch

from .. import _lib


def silu_and_mul_masked_post_quant_fwd(input: torch.Tensor, output: torch.Tensor, output_scale: torch.Tensor,
                                       quant_group_size: int, masked_m: torch.Tensor):
    """input bf16 [expert_num, token_num_padded, hidden_dim]; output e4m3fn [.., .., hidden_dim // 2];
    output_scale fp32 [.., .., hidden_dim // 2 // 128]; masked_m int32 [expert_num] = rows in use per expert.
    Rows at or past masked_m[e] are left untouched in output and output_scale."""
    assert input.is_contiguous()
    assert output.dtype == torch.float8_e4m3fn
    assert output.is_contiguous()
    assert len(input.shape) == 3
    assert input.shape[0] == masked_m.shape[0]
    assert input.shape[-1] % 2 == 0
    size_n = input.shape[-1] // 2
    assert size_n % quant_group_size == 0
    if quant_group_size != 128:
        raise ValueError("silu_and_mul_masked_post_quant_fwd: quant_group_size must be 128 on gfx950")
    assert input.dtype == torch.bfloat16 and output_scale.dtype == torch.float32
    assert masked_m.dtype == torch.int32 and masked_m.is_contiguous()
    E, T, _ = input.shape
    assert output.shape == (E, T, size_n) and output_scale.shape == (E, T, size_n // quant_group_size)
    # the kernel walks the E*T rows as one table: the expert stride of the scales must be T row strides
    if E > 1 and T > 1 and output_scale.stride(0) != T * output_scale.stride(1):
        raise ValueError("silu_and_mul_masked_post_quant_fwd: output_scale rows of different experts must be "
                         "evenly spaced (stride(0) == token_num_padded * stride(1))")
    _lib.require_cuda(input, output, output_scale, masked_m)
    stride_m = output_scale.stride(1) if T > 1 else output_scale.stride(0)
    code = _lib.lib().mi355_silu_and_mul_group_quant_fp8(
        input.data_ptr(), output.data_ptr(), output_scale.data_ptr(), E * T, size_n, input.stride(1),
        quant_group_size, stride_m, output_scale.stride(2), masked_m.data_ptr(), T, _lib.stream_ptr(input.device),
    )
    _lib.check(code, "silu_and_mul_masked_post_quant_fwd")
    return


def silu_and_mul_post_quant_fwd(input: torch.Tensor, output: torch.Tensor, output_scale: torch.Tensor,
                                quant_group_size: int = 128):
    """input bf16 [M, 2H] (row stride free, unit column stride) -> output e4m3fn [M, H] contiguous,
    output_scale fp32 [M, H // 128] (any strides)."""
    assert input.ndim == 2 and input.stride(-1) == 1 and input.dtype == torch.bfloat16
    assert output.dtype == torch.float8_e4m3fn and output.is_contiguous()
    assert input.shape[-1] % 2 == 0
    size_m, size_n = input.shape[0], input.shape[-1] // 2
    assert size_n % quant_group_size == 0
    if quant_group_size != 128:
        raise ValueError("silu_and_mul_post_quant_fwd: quant_group_size must be 128 on gfx950")
    assert output.shape == (size_m, size_n)
    assert output_scale.dtype == torch.float32 and output_scale.shape == (size_m, size_n // quant_group_size)
    _lib.require_cuda(input, output, output_scale)
    code = _lib.lib().mi355_silu_and_mul_group_quant_fp8(
        input.data_ptr(), output.data_ptr(), output_scale.data_ptr(), size_m, size_n, input.stride(0),
        quant_group_size, output_scale.stride(0), output_scale.stride(1), None, 0, _lib.stream_ptr(input.device),
    )
    _lib.check(code, "silu_and_mul_post_quant_fwd")
    return

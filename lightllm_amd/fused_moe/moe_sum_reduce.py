"""Sum over the top-k slots after the second expert GEMM.

Same name and arguments as ``moe_sum_reduce`` of the reference
(lightllm/common/basemodel/triton_kernel/fused_moe/moe_sum_reduce.py:69-108); runs ``mi355_moe_sum_reduce``.
"""
from typing import Dict

import torch

from .. import _lib


def moe_sum_reduce(input: torch.Tensor, output: torch.Tensor, run_config: Dict = None):
    """output[t, :] = bf16(sum_k input[t, k, :]) with fp32 accumulation in ascending k.
    ``run_config`` (the reference's tile dictionary) is accepted and ignored."""
    assert input.is_contiguous()
    assert output.is_contiguous()
    token_num, topk_num, hidden_dim = input.shape
    assert output.shape[0] == token_num and output.shape[1] == hidden_dim
    assert input.dtype == torch.bfloat16 and output.dtype == torch.bfloat16
    _lib.require_cuda(input, output)
    code = _lib.lib().mi355_moe_sum_reduce(
        input.data_ptr(), output.data_ptr(), token_num, topk_num, hidden_dim, _lib.stream_ptr(input.device)
    )
    _lib.check(code, "moe_sum_reduce")
    return

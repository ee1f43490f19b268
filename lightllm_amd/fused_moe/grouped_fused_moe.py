"""Routed-expert (MoE) block-FP8 GEMM for ragged per-expert batches, plus its routing tables.

Same names, arguments and tensor layouts as
lightllm/common/basemodel/triton_kernel/fused_moe/grouped_fused_moe.py of the reference
(moe_align_fused :388-396, moe_align2 :452-477, grouped_matmul :771-989); the work is done by
``mi355_moe_align_fused``, ``mi355_moe_align2`` and ``mi355_grouped_block_fp8_gemm``.
Only the fp8 128x128-block branch exists here (use_fp8_w8a8=True with 3-D weight scales).
"""
from typing import Optional

import torch

from .. import _lib
from ..quantization.fp8act_quant_kernel import per_token_group_quant_fp8

_BLOCK_MS = (16, 32, 64, 128)


def moe_align_fused(expert_to_token_index, expert_to_weight, expert_token_num, topk_ids, topk_weights):
    """Bucket the flattened (token, slot) pairs of ``topk_ids`` [T, topk] by expert.

    Fills expert_to_token_index int32 [E, T*topk], expert_to_weight fp32 [E, T*topk] and
    expert_token_num int32 [E]; entries past an expert's count are left as they were.  Pair indices come
    out ascending inside every expert for every T (the reference only orders them for T <= 128).
    """
    assert topk_ids.is_contiguous() and topk_weights.is_contiguous()
    assert topk_ids.dtype == torch.int32 and topk_weights.dtype == torch.float32
    assert expert_to_token_index.is_contiguous() and expert_to_weight.is_contiguous()
    assert expert_to_token_index.dtype == torch.int32 and expert_to_weight.dtype == torch.float32
    assert expert_token_num.dtype == torch.int32 and expert_token_num.is_contiguous()
    pairs = topk_ids.numel()
    E = expert_token_num.shape[0]
    assert expert_to_token_index.shape == (E, pairs) and expert_to_weight.shape == (E, pairs)
    _lib.require_cuda(topk_ids, topk_weights, expert_to_token_index, expert_to_weight, expert_token_num)
    code = _lib.lib().mi355_moe_align_fused(
        topk_ids.data_ptr(), topk_weights.data_ptr(), pairs, E, expert_to_token_index.data_ptr(),
        expert_to_weight.data_ptr(), expert_token_num.data_ptr(), _lib.stream_ptr(topk_ids.device),
    )
    _lib.check(code, "moe_align_fused")
    return expert_to_token_index, expert_to_weight, expert_token_num


def moe_align2(token_num_mul_topk_num: int, exports_token_num: torch.Tensor, block_m: int):
    """Expert counts [E] -> schedule table int32 [max_blocks, 3] of (expert, m_index, token_start);
    rows past the last real block have expert = -1."""
    assert exports_token_num.dtype == torch.int32 and exports_token_num.is_contiguous()
    _lib.require_cuda(exports_token_num)
    E = exports_token_num.shape[0]
    lib = _lib.lib()
    rows = lib.mi355_moe_align2_rows(token_num_mul_topk_num, E, block_m)
    table = torch.empty((rows, 3), dtype=torch.int32, device=exports_token_num.device)
    code = lib.mi355_moe_align2(
        exports_token_num.data_ptr(), E, block_m, rows, table.data_ptr(), _lib.stream_ptr(table.device)
    )
    _lib.check(code, "moe_align2")
    return table


def grouped_matmul(
    token_num_mul_topk_num: int,
    token_inputs: torch.Tensor,
    token_input_scale: torch.Tensor,
    expert_to_token_num: torch.Tensor,
    expert_to_token_index: torch.Tensor,
    expert_to_weights: torch.Tensor,
    expert_weights: torch.Tensor,
    expert_to_weights_scale: torch.Tensor,
    topk_num: int,
    out: torch.Tensor,
    mul_routed_weight: bool,
    use_fp8_w8a8: bool,
    alloc_tensor_func=torch.empty,
    reused_mblock_infos=None,
    run_config: Optional[dict] = None,
    bias: Optional[torch.Tensor] = None,
):
    """out[idx] = blockscaled(quant(token_inputs[idx // topk_num]) @ expert_weights[e].T) [* routed weight]
    for every pair idx routed to expert e.  Returns (mblocks_to_tuple_info, BLOCK_SIZE_M) for reuse by the
    second GEMM of the layer, like the reference.

    token_inputs bf16 [T,K] (quantized here per 1x128 group, reference :862-875) or, as an extension,
    already-quantized e4m3fn with ``token_input_scale`` [T,K/128]; expert_weights e4m3fn [E,N,K];
    expert_to_weights_scale fp32 [E,N/128,K/128]; out bf16 [T*topk, N].
    """
    assert use_fp8_w8a8, "only the fp8 block-quantized branch is implemented on gfx950"
    assert bias is None, "per-expert bias is not supported by the fp8 block branch"
    expert_num, n, k = expert_weights.shape
    assert token_inputs.shape[1] == k
    assert expert_to_token_index.shape == expert_to_weights.shape
    assert token_inputs.is_contiguous()
    assert expert_to_token_num.is_contiguous()
    assert expert_to_weights.is_contiguous()
    assert expert_weights.is_contiguous()
    assert expert_to_weights_scale is not None and expert_to_weights_scale.ndim == 3
    assert expert_to_weights_scale.is_contiguous() and out.is_contiguous()
    # 128x128 weight blocks (the reference derives the block sizes from the two shapes, :814-816; the last
    # n block may be partial here)
    block_size_k = 128
    assert expert_to_weights_scale.shape[1] == (n + 127) // 128 and expert_to_weights_scale.shape[2] * 128 == k, (
        "weights must be 128x128 block-quantized"
    )
    assert out.dtype == torch.bfloat16 and out.shape[1] == n
    _lib.require_cuda(token_inputs, expert_weights, out)
    lib = _lib.lib()

    if token_inputs.dtype == torch.float8_e4m3fn:
        assert token_input_scale is not None and token_input_scale.is_contiguous()
    else:
        assert k % block_size_k == 0
        token_inputs, token_input_scale = per_token_group_quant_fp8(
            token_inputs, block_size_k, dtype=expert_weights.dtype, alloc_func=alloc_tensor_func
        )

    block_m = None
    if run_config is not None and run_config.get("BLOCK_SIZE_M") in _BLOCK_MS:
        block_m = run_config["BLOCK_SIZE_M"]
    if block_m is None:
        block_m = lib.mi355_grouped_block_m(token_num_mul_topk_num, expert_num, n, k)
    if reused_mblock_infos is not None and reused_mblock_infos[1] == block_m:
        table = reused_mblock_infos[0]
    else:
        table = moe_align2(token_num_mul_topk_num, expert_to_token_num, block_m)

    code = lib.mi355_grouped_block_fp8_gemm(
        token_inputs.data_ptr(), token_input_scale.data_ptr(), expert_weights.data_ptr(),
        expert_to_weights_scale.data_ptr(), expert_to_token_index.data_ptr(), expert_to_weights.data_ptr(),
        expert_to_token_num.data_ptr(), table.data_ptr(), table.shape[0], block_m, token_num_mul_topk_num,
        token_inputs.shape[0], expert_num, topk_num, n, k, 1 if mul_routed_weight else 0, out.data_ptr(),
        _lib.stream_ptr(out.device),
    )
    _lib.check(code, "grouped_matmul")
    return (table, block_m)

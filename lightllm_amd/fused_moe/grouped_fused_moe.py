"""Routed-expert (MoE) block-FP8 GEMM for ragged per-expert batches, plus its routing tables.

Same names, arguments and tensor layouts as
lightllm/common/basemodel/triton_kernel/fused_moe/grouped_fused_moe.py of the reference
(moe_align :64-98, moe_align1 :147-214, moe_align_fused :388-396, moe_align2 :452-477, grouped_matmul :771-989, fused_experts_impl :992-1115);
the work is done by ``mi355_moe_align_fused``, ``mi355_moe_align2`` and ``mi355_grouped_block_fp8_gemm``.
Only the fp8 128x128-block branch exists here (use_fp8_w8a8=True with 3-D weight scales).
"""
from typing import Optional

import torch

from .. import _lib
from ..quantization.fp8act_quant_kernel import lightllm_per_token_group_quant_fp8, per_token_group_quant_fp8
from .moe_silu_and_mul import silu_and_mul_fwd
from .moe_silu_and_mul_mix_quant_ep import silu_and_mul_post_quant_fwd
from .moe_sum_reduce import moe_sum_reduce

_BLOCK_MS = (16, 32, 64, 128, 256)
FFN_MOE_CHUNK_SIZE = 32 * 1024  # tokens per pass of fused_experts_impl (reference :34)


def moe_align(topk_ids: torch.Tensor, out: torch.Tensor):
    """out int32 [E, T*topk]: out[e, j] = 1 where the flattened pair j of ``topk_ids`` [T, topk] is routed to
    expert e, 0 elsewhere (reference :64-98; its zero fill is part of the kernel here)."""
    token_num, topk = topk_ids.shape
    assert out.shape[1] == token_num * topk, f"out shape {out.shape} topk_ids shape {topk_ids.shape} "
    assert topk_ids.is_contiguous()
    assert topk_ids.dtype == torch.int32 and out.dtype == torch.int32 and out.stride(1) == 1
    _lib.require_cuda(topk_ids, out)
    code = _lib.lib().mi355_moe_align(
        topk_ids.data_ptr(), token_num * topk, out.shape[0], out.data_ptr(), out.stride(0),
        _lib.stream_ptr(out.device),
    )
    _lib.check(code, "moe_align")


def moe_align1(experts_info: torch.Tensor, topk_weights: torch.Tensor, experts_weight_info: torch.Tensor,
               exports_token_num: torch.Tensor, topk: int):
    """Compacts the 0/1 table of ``moe_align`` in place into pair indices, with the weights and the per-expert
    counts (reference :147-214).  Entries past an expert's count keep what they held."""
    expert_num, token_num_mul_topk = experts_info.shape
    topk_num = topk_weights.shape[1]
    assert token_num_mul_topk <= FFN_MOE_CHUNK_SIZE * topk_num, "need split to handle seq len too long"
    assert exports_token_num.shape[0] == expert_num
    assert topk_weights.is_contiguous()
    assert experts_info.dtype == torch.int32 and experts_info.stride(1) == 1
    assert experts_weight_info.dtype == torch.float32 and experts_weight_info.stride(1) == 1
    assert experts_weight_info.shape == experts_info.shape
    assert exports_token_num.dtype == torch.int32 and exports_token_num.is_contiguous()
    assert topk_weights.dtype == torch.float32
    _lib.require_cuda(experts_info, topk_weights, experts_weight_info, exports_token_num)
    code = _lib.lib().mi355_moe_align1(
        experts_info.data_ptr(), experts_info.stride(0), topk_weights.data_ptr(), token_num_mul_topk, expert_num,
        experts_weight_info.data_ptr(), experts_weight_info.stride(0), exports_token_num.data_ptr(),
        _lib.stream_ptr(experts_info.device),
    )
    _lib.check(code, "moe_align1")


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
    """Expert counts [E] -> schedule table int32 [max_blocks, 4] of (expert, m_index, token_start,
    tokens in the block);
    rows past the last real block have expert = -1."""
    assert exports_token_num.dtype == torch.int32 and exports_token_num.is_contiguous()
    _lib.require_cuda(exports_token_num)
    E = exports_token_num.shape[0]
    lib = _lib.lib()
    rows = lib.mi355_moe_align2_rows(token_num_mul_topk_num, E, block_m)
    table = torch.empty((rows, 4), dtype=torch.int32, device=exports_token_num.device)
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
    expert_to_weights_scale fp32 [E,N/128,K/128]; out bf16 [T*topk, N]; ``bias`` [E, N] (bf16, fp16 or fp32) is
    added to the fp32 accumulator before the routed weight (reference :702-715).
    """
    assert use_fp8_w8a8, "only the fp8 block-quantized branch is implemented on gfx950"
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
    assert out.dtype in (torch.bfloat16, torch.float16) and out.shape[1] == n
    if bias is not None:
        assert bias.shape == (expert_num, n) and bias.stride(1) == 1 and bias.dtype in _lib.DTYPE_CODES
    _lib.require_cuda(token_inputs, expert_weights, out, bias)
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

    # the 256-row launch is persistent when it gets the (zero at rest) tile counters of this stream's workspace
    # (and, given room for the two block lists, runs the blocks of few rows on the weight-streaming tile)
    ws = _lib.workspace(out.device, lib.mi355_grouped_workspace_bytes(table.shape[0])) if block_m == 256 else None
    code = lib.mi355_grouped_block_fp8_gemm_bias(
        token_inputs.data_ptr(), token_input_scale.data_ptr(), expert_weights.data_ptr(),
        expert_to_weights_scale.data_ptr(), expert_to_token_index.data_ptr(), expert_to_weights.data_ptr(),
        expert_to_token_num.data_ptr(), table.data_ptr(), table.shape[0], block_m, token_num_mul_topk_num,
        token_inputs.shape[0], expert_num, topk_num, n, k, 1 if mul_routed_weight else 0, out.data_ptr(),
        ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, _lib.DTYPE_CODES[out.dtype],
        bias.data_ptr() if bias is not None else None, _lib.DTYPE_CODES[bias.dtype] if bias is not None else 0,
        bias.stride(0) if bias is not None else 0, _lib.stream_ptr(out.device),
    )
    _lib.check(code, "grouped_matmul")
    return (table, block_m)


def fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    inplace: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    w1_bias: Optional[torch.Tensor] = None,
    w2_bias: Optional[torch.Tensor] = None,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    alloc_tensor_func=torch.empty,
    run_config: Optional[dict] = None,
    layout="blocked",
    limit=None,
    alpha=None,
):
    """The routed-expert FFN: out[t] = sum_k w[t,k] * ( silu_mul( x[t] @ w1[e].T ) @ w2[e].T ),  e = topk_ids[t,k].

    hidden_states bf16 [T, H]; w1 e4m3fn [E, 2I, H] (gate rows then up rows), w2 e4m3fn [E, H, I];
    w1_scale / w2_scale fp32 128x128-block scales; topk_ids int32 [T, topk], topk_weights fp32 [T, topk].

    Same steps and the same results as the reference's sequence (routing tables, gate/up GEMM,
    silu_and_mul, quantize, down GEMM with the routed weight, sum over slots); the SiLU product is
    quantized where it is produced, so its bf16 form [T*topk, I] is never written to memory.
    """
    assert use_fp8_w8a8 and not use_int8_w8a16, "only the fp8 block-quantized branch is implemented on gfx950"
    fused_act = layout == "blocked" and limit is None and alpha is None   # else: silu_and_mul_fwd + quantizer
    assert hidden_states.shape[1] == w1.shape[2], "Hidden size mismatch"
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype == torch.bfloat16
    num_tokens, _ = hidden_states.shape
    E, N, _ = w1.shape
    assert N % 256 == 0 and w2.shape[2] == N // 2, "intermediate size must be a multiple of 128"
    topk_num = topk_ids.shape[1]
    M = min(num_tokens, FFN_MOE_CHUNK_SIZE)
    device, dtype = hidden_states.device, hidden_states.dtype

    # gate/up output and down output share one buffer, as in the reference: the first is dead once quantized
    shared13 = alloc_tensor_func((M, topk_num, max(N, w2.shape[1])), device=device, dtype=dtype)
    cache1 = shared13.view(-1)[: M * topk_num * N].view(M, topk_num, N)
    cache3 = shared13.view(-1)[: M * topk_num * w2.shape[1]].view(M, topk_num, w2.shape[1])
    cache2_q = alloc_tensor_func((M, topk_num, N // 2), device=device, dtype=torch.float8_e4m3fn)
    cache2_s = alloc_tensor_func((M, topk_num, N // 2 // 128), device=device, dtype=torch.float32)

    out_hidden_states = hidden_states if inplace else alloc_tensor_func(hidden_states.shape, device=device, dtype=dtype)

    for begin in range(0, num_tokens, FFN_MOE_CHUNK_SIZE):
        end = min(begin + FFN_MOE_CHUNK_SIZE, num_tokens)
        cur = hidden_states[begin:end]
        tokens = end - begin
        c1, c3 = cache1[:tokens], cache3[:tokens]
        c2_q, c2_s = cache2_q[:tokens], cache2_s[:tokens]
        cur_ids, cur_weights = topk_ids[begin:end], topk_weights[begin:end]
        pairs = cur_ids.numel()

        expert_to_tokens = torch.empty((E, pairs), dtype=torch.int32, device=device)
        expert_to_weights = torch.empty((E, pairs), dtype=torch.float32, device=device)
        expert_to_token_num = torch.empty((E,), dtype=torch.int32, device=device)
        moe_align_fused(expert_to_tokens, expert_to_weights, expert_to_token_num, cur_ids, cur_weights)

        reused = grouped_matmul(
            pairs, cur, a1_scale, expert_to_token_num, expert_to_tokens, expert_to_weights=expert_to_weights,
            expert_weights=w1, expert_to_weights_scale=w1_scale, topk_num=topk_num, out=c1.view(-1, N),
            mul_routed_weight=False, use_fp8_w8a8=True, alloc_tensor_func=alloc_tensor_func, run_config=run_config,
            bias=w1_bias,
        )
        if fused_act:
            silu_and_mul_post_quant_fwd(c1.view(-1, N), c2_q.view(-1, N // 2), c2_s.view(-1, N // 2 // 128))
        else:
            act = alloc_tensor_func((pairs, N // 2), device=device, dtype=dtype)
            silu_and_mul_fwd(c1.view(-1, N), act, layout=layout, limit=limit, alpha=alpha)
            lightllm_per_token_group_quant_fp8(act, 128, c2_q.view(-1, N // 2), c2_s.view(-1, N // 2 // 128))
        grouped_matmul(
            pairs, c2_q.view(-1, N // 2), c2_s.view(-1, N // 2 // 128), expert_to_token_num, expert_to_tokens,
            expert_to_weights=expert_to_weights, expert_weights=w2, expert_to_weights_scale=w2_scale, topk_num=1,
            out=c3.view(-1, w2.shape[1]), mul_routed_weight=True, use_fp8_w8a8=True,
            alloc_tensor_func=alloc_tensor_func, reused_mblock_infos=reused, run_config=run_config, bias=w2_bias,
        )
        moe_sum_reduce(c3, out_hidden_states[begin:end])
    return out_hidden_states


def inplace_fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    use_fp8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    w1_bias: Optional[torch.Tensor] = None,
    w2_bias: Optional[torch.Tensor] = None,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    layout: str = "blocked",
    alpha: Optional[float] = None,
    limit: Optional[float] = None,
) -> None:
    """`fused_experts_impl` writing the result over ``hidden_states`` (reference :1118-1154; there it is also
    registered as ``torch.ops.lightllm.inplace_fused_experts_impl``, which this package leaves to the host)."""
    fused_experts_impl(
        hidden_states, w1, w2, topk_weights, topk_ids, inplace=True, use_fp8_w8a8=use_fp8_w8a8,
        use_int8_w8a16=use_int8_w8a16, w1_bias=w1_bias, w2_bias=w2_bias, w1_scale=w1_scale, w2_scale=w2_scale,
        a1_scale=a1_scale, a2_scale=a2_scale, layout=layout, alpha=alpha, limit=limit,
    )


def outplace_fused_experts_impl(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    use_fp8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    w1_bias: Optional[torch.Tensor] = None,
    w2_bias: Optional[torch.Tensor] = None,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    layout: str = "blocked",
    alpha: Optional[float] = None,
    limit: Optional[float] = None,
) -> torch.Tensor:
    """`fused_experts_impl` into a new tensor (reference :1187-1223)."""
    return fused_experts_impl(
        hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, use_fp8_w8a8=use_fp8_w8a8,
        use_int8_w8a16=use_int8_w8a16, w1_bias=w1_bias, w2_bias=w2_bias, w1_scale=w1_scale, w2_scale=w2_scale,
        a1_scale=a1_scale, a2_scale=a2_scale, layout=layout, alpha=alpha, limit=limit,
    )


def fused_experts(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    inplace: bool = False,
    use_fp8_w8a8: bool = False,
    use_int8_w8a16: bool = False,
    w1_scale: Optional[torch.Tensor] = None,
    w2_scale: Optional[torch.Tensor] = None,
    a1_scale: Optional[torch.Tensor] = None,
    a2_scale: Optional[torch.Tensor] = None,
    w1_bias: Optional[torch.Tensor] = None,
    w2_bias: Optional[torch.Tensor] = None,
    layout: str = "blocked",
    alpha: Optional[float] = None,
    limit: Optional[float] = None,
):
    """What ``FuseMoeTriton`` calls (reference :1258-1290; note the argument order: the scales come before the
    biases here and after them in the two functions above).  Returns ``hidden_states`` itself when ``inplace``."""
    if inplace:
        inplace_fused_experts_impl(
            hidden_states, w1, w2, topk_weights, topk_ids, use_fp8_w8a8, use_int8_w8a16, w1_bias, w2_bias, w1_scale,
            w2_scale, a1_scale, a2_scale, layout=layout, alpha=alpha, limit=limit,
        )
        return hidden_states
    return outplace_fused_experts_impl(
        hidden_states, w1, w2, topk_weights, topk_ids, use_fp8_w8a8, use_int8_w8a16, w1_bias, w2_bias, w1_scale,
        w2_scale, a1_scale, a2_scale, layout=layout, alpha=alpha, limit=limit,
    )

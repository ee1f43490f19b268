"""Grouped block-FP8 GEMMs in the two layouts the expert-parallel caller uses.

LightLLM's EP path hands these to DeepGEMM (lightllm/common/basemodel/triton_kernel/fused_moe/
grouped_fused_moe_ep.py: ``_deepgemm_grouped_fp8_nt_masked`` :584-595, ``deepgemm_grouped_fp8_nt_contiguous``
:361-372, ``masked_group_gemm`` :69-93).  Here both layouts are turned into the index tables of
``mi355_grouped_block_fp8_gemm`` and run on the same kernels as ``grouped_matmul``:

  masked      x [E, T_pad, K] e4m3fn + scales [E, T_pad, K/128]; only the first masked_m[e] rows of expert e count
  contiguous  x [M_sum, K] + scales [M_sum, K/128]; m_indices[row] = expert of the row, -1 = padding row

Weights are e4m3fn [E, N, K] with fp32 128x128-block scales [E, ceil(N/128), K/128]; outputs are bf16.
Rows that belong to no expert (past masked_m, or m_indices < 0) are not written.
"""
import collections
from typing import Tuple

import torch

from .. import _lib
from .grouped_fused_moe import _BLOCK_MS, moe_align2, moe_align_fused
from .moe_silu_and_mul_mix_quant_ep import silu_and_mul_masked_post_quant_fwd

_row_tables = collections.OrderedDict()   # (E, T, device) -> table; the few shapes a server uses, oldest dropped
_ROW_TABLES_KEPT = 8


def _masked_row_table(E: int, T: int, device: torch.device) -> torch.Tensor:
    """int32 [E, T] with entry (e, j) = e*T + j: row j of expert e in the flattened [E*T, K] view."""
    key = (E, T, device)
    t = _row_tables.get(key)
    if t is None:
        t = torch.arange(E * T, dtype=torch.int32, device=device).view(E, T).contiguous()
        _row_tables[key] = t
        while len(_row_tables) > _ROW_TABLES_KEPT:
            _row_tables.popitem(last=False)
    else:
        _row_tables.move_to_end(key)
    return t


def _check_operands(x, xs, w, ws, out, rows):
    assert x.dtype == torch.float8_e4m3fn and w.dtype == torch.float8_e4m3fn
    assert xs.dtype == torch.float32 and ws.dtype == torch.float32 and out.dtype == torch.bfloat16
    assert x.is_contiguous() and xs.is_contiguous() and w.is_contiguous() and ws.is_contiguous() and out.is_contiguous()
    E, N, K = w.shape
    assert x.shape[-1] == K and K % 128 == 0
    assert xs.shape[-1] == K // 128 and ws.shape == (E, (N + 127) // 128, K // 128)
    assert out.shape[-1] == N and out.numel() == rows * N and x.numel() == rows * K
    _lib.require_cuda(x, xs, w, ws, out)
    return E, N, K


def _launch(x, xs, w, ws, out, index, counts, rows, stride, E, N, K, block_m=None):
    lib = _lib.lib()
    if block_m is None:
        block_m = lib.mi355_grouped_block_m(rows, E, N, K)
    assert block_m in _BLOCK_MS
    table = moe_align2(rows, counts, block_m)
    wsp = _lib.workspace(out.device, lib.mi355_grouped_workspace_bytes(table.shape[0])) if block_m == 256 else None
    code = lib.mi355_grouped_block_fp8_gemm(
        x.data_ptr(), xs.data_ptr(), w.data_ptr(), ws.data_ptr(), index.data_ptr(), xs.data_ptr(), counts.data_ptr(),
        table.data_ptr(), table.shape[0], block_m, stride, rows, E, 1, N, K, 0, out.data_ptr(),
        wsp.data_ptr() if wsp is not None else None, wsp.numel() if wsp is not None else 0, _lib.stream_ptr(out.device),
    )
    _lib.check(code, "grouped fp8 gemm")


def _deepgemm_grouped_fp8_nt_masked(input_tuple: Tuple[torch.Tensor, torch.Tensor],
                                    w_tuple: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor,
                                    masked_m: torch.Tensor, expected_m: int):
    """out[e, :masked_m[e]] = blockscaled(x[e, :masked_m[e]] @ w[e].T).  ``expected_m`` (DeepGEMM's tiling hint) is
    used the same way: it picks the row block."""
    x, xs = input_tuple
    w, ws = w_tuple
    assert x.ndim == 3 and out.ndim == 3 and masked_m.dtype == torch.int32 and masked_m.is_contiguous()
    E_x, T, _ = x.shape
    E, N, K = _check_operands(x, xs, w, ws, out, E_x * T)
    assert E_x == E and masked_m.shape == (E,) and out.shape == (E, T, N)
    block_m = None
    if expected_m is not None and expected_m > 0:
        block_m = _lib.lib().mi355_grouped_block_m(int(min(expected_m, T)) * E, E, N, K)
    _launch(x, xs, w, ws, out, _masked_row_table(E, T, x.device), masked_m, E * T, T, E, N, K, block_m)
    return out


def deepgemm_grouped_fp8_nt_contiguous(input_tuple: Tuple[torch.Tensor, torch.Tensor],
                                       w_tuple: Tuple[torch.Tensor, torch.Tensor], out: torch.Tensor,
                                       m_indices: torch.Tensor):
    """out[r] = blockscaled(x[r] @ w[m_indices[r]].T) for every row with m_indices[r] >= 0."""
    x, xs = input_tuple
    w, ws = w_tuple
    assert x.ndim == 2 and out.ndim == 2 and m_indices.dtype == torch.int32 and m_indices.is_contiguous()
    rows = x.shape[0]
    E, N, K = _check_operands(x, xs, w, ws, out, rows)
    assert m_indices.shape == (rows,)
    index = torch.empty((E, rows), dtype=torch.int32, device=x.device)
    weight = torch.empty((E, rows), dtype=torch.float32, device=x.device)
    counts = torch.empty((E,), dtype=torch.int32, device=x.device)
    ones = torch.ones((rows, 1), dtype=torch.float32, device=x.device)
    moe_align_fused(index, weight, counts, m_indices.view(rows, 1), ones)
    _launch(x, xs, w, ws, out, index, counts, rows, rows, E, N, K)
    return out


def masked_group_gemm(recv_x: Tuple[torch.Tensor, torch.Tensor], masked_m: torch.Tensor, dtype: torch.dtype,
                      w1: torch.Tensor, w1_scale: torch.Tensor, w2: torch.Tensor, w2_scale: torch.Tensor,
                      expected_m: int):
    """The expert FFN on the masked (low-latency dispatch) layout: gate/up GEMM, SiLU-mul fused with the group
    quantizer, down GEMM.  Returns bf16 [E, T_pad, hidden]; rows past masked_m[e] are unspecified."""
    assert dtype == torch.bfloat16, "outputs are bf16 on gfx950"
    x = recv_x[0]
    padded_m = x.shape[1]
    E, N, _ = w1.shape
    expected_m = min(expected_m, padded_m)
    gemm_out_a = torch.empty((E, padded_m, N), device=x.device, dtype=dtype)
    qsilu_out = torch.empty((E, padded_m, N // 2), dtype=w1.dtype, device=x.device)
    qsilu_out_scale = torch.empty((E, padded_m, N // 2 // 128), device=x.device, dtype=torch.float32)
    _deepgemm_grouped_fp8_nt_masked(recv_x, (w1, w1_scale), gemm_out_a, masked_m, expected_m)
    silu_and_mul_masked_post_quant_fwd(gemm_out_a, qsilu_out, qsilu_out_scale, 128, masked_m)
    del gemm_out_a
    gemm_out_b = torch.empty((E, padded_m, w2.shape[1]), device=x.device, dtype=dtype)
    _deepgemm_grouped_fp8_nt_masked((qsilu_out, qsilu_out_scale), (w2, w2_scale), gemm_out_b, masked_m, expected_m)
    return gemm_out_b

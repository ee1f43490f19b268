"""The fp8w8a8-b128 quantization method on the gfx950 kernels.

Mirrors FP8w8a8B128QuantizationMethod / FP8w8a8B128TritonQuantizationMethod of the reference
(lightllm/common/quantization/w8a8.py:418-474, 505-533): 128x128 block-quantized e4m3fn weights with
``weight_scale_inv`` scales, dynamic per-token-group activation quantization, bf16 output, no bias.
"""
from typing import Callable, List, Optional, Tuple, Union

import torch

from .fp8act_quant_kernel import per_token_group_quant_fp8
from .fp8w8a8_block_gemm_kernel import w8a8_block_fp8_matmul
from .fp8w8a8_block_quant_kernel import weight_quant
from .quantize_method import QuantizationMethod, WeightPack
from .registry import QUANTMETHODS


class FP8w8a8B128QuantizationMethod(QuantizationMethod):
    """``cache_manager`` may be any object with ``empty(shape, dtype=, device=)`` (LightLLM's g_cache_manager);
    without one, outputs come from torch.empty."""

    def __init__(self, cache_manager=None):
        super().__init__()
        self.cache_manager = cache_manager
        self.block_size = 128
        self.weight_scale_suffix = "weight_scale_inv"
        self.has_weight_scale = True
        self.has_weight_zero_point = False

    def quantize(self, weight: torch.Tensor, output: WeightPack) -> None:
        device = output.weight.device
        qweight, scale = weight_quant(weight.cuda(device).contiguous(), self.block_size)
        output.weight.copy_(qweight)
        output.weight_scale.copy_(scale)

    def _alloc_func(self, use_custom_tensor_mananger: bool) -> Callable:
        if use_custom_tensor_mananger and self.cache_manager is not None:
            return self.cache_manager.empty
        return torch.empty

    def _dynamic_quant_input(
        self,
        input_tensor: torch.Tensor,
        weight_pack: WeightPack,
        out: Optional[torch.Tensor] = None,
        use_custom_tensor_mananger: bool = True,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """The five GEMM operands in the order of `w8a8_block_fp8_matmul`: quantized activations, the [K, N] view
        of the weight (strides (1, K)), activation scales, the [K/128, N/128] view of the weight scales, and the
        output (allocated here unless the caller brings one)."""
        alloc = self._alloc_func(use_custom_tensor_mananger)
        w_kn, ws_kn = weight_pack.weight.t(), weight_pack.weight_scale.t()
        x_q, x_s = per_token_group_quant_fp8(input_tensor, self.block_size, dtype=w_kn.dtype, alloc_func=alloc)
        if out is None:
            rows, cols = input_tensor.shape[0], w_kn.shape[1]
            out = alloc((rows, cols), dtype=input_tensor.dtype, device=input_tensor.device)
        return x_q, w_kn, x_s, ws_kn, out

    def _create_weight(
        self, out_dims: Union[int, List[int]], in_dim: int, dtype: torch.dtype, device_id: int, num_experts: int = 1
    ) -> Tuple[WeightPack, List[WeightPack]]:
        """One e4m3fn [sum(out_dims), in_dim] weight with its [.. // 128, .. // 128] fp32 scales (a leading expert
        axis when num_experts > 1), and one view pair per fused sub-weight, cut along the output rows."""
        b = self.block_size
        parts = list(out_dims) if isinstance(out_dims, (list, tuple)) else [out_dims]
        rows = sum(parts)
        lead = (num_experts,) if num_experts > 1 else ()
        device = torch.device("cuda", device_id)

        def storage(r: int, c: int, dt: torch.dtype) -> torch.Tensor:
            return torch.empty(lead + (r, c), dtype=dt, device=device)

        fused = WeightPack(
            weight=storage(rows, in_dim, torch.float8_e4m3fn),
            weight_scale=storage(rows // b, in_dim // b, torch.float32),
        )
        views = self._split_weight_pack(
            fused,
            weight_out_dims=parts,
            weight_split_dim=-2,
            weight_scale_out_dims=[p // b for p in parts],
            weight_scale_split_dim=-2,
        )
        return fused, views


@QUANTMETHODS.register(["fp8w8a8-b128-mi355", "fp8w8a8-b128-triton", "fp8w8a8-b128"], platform="cuda")
class FP8w8a8B128Mi355QuantizationMethod(FP8w8a8B128QuantizationMethod):
    def apply(
        self,
        input_tensor: torch.Tensor,
        weight_pack: WeightPack,
        out: Optional[torch.Tensor] = None,
        workspace: Optional[torch.Tensor] = None,
        use_custom_tensor_mananger: bool = True,
        bias: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        assert bias is None, f"Bias addition is not supported in {self.method_name} for now"
        qinput_tensor, qweight, input_scale, weight_scale, out = self._dynamic_quant_input(
            input_tensor, weight_pack, out, use_custom_tensor_mananger
        )
        w8a8_block_fp8_matmul(
            qinput_tensor, qweight, input_scale, weight_scale, out, (self.block_size, self.block_size),
            dtype=input_tensor.dtype,
        )
        return out

    @property
    def method_name(self):
        return "fp8w8a8-b128-mi355"

"""Plug-in boundary of the quantized linear layers: WeightPack and the QuantizationMethod base class.

Mirrors lightllm/common/quantization/quantize_method.py:8-149 of the reference (same attribute names,
method names, argument order and load bookkeeping) so that LightLLM's MMWeightTpl / FusedMoeWeight can
hold an object from this package unchanged.
"""
from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch


@dataclass
class WeightPack:
    weight: Optional[torch.Tensor] = None
    weight_scale: Optional[torch.Tensor] = None
    weight_zero_point: Optional[torch.Tensor] = None

    def __post_init__(self):
        # [weight loaded, scale loaded, zero point loaded]; parts a method does not have count as loaded
        self.load_ok = [False, self.weight_scale is None, self.weight_zero_point is None]

    def get_expert(self, expert_idx: int):
        assert self.weight.ndim == 3, f"weight must be a 3D tensor, but got {self.weight.ndim}"
        pick = lambda t: t[expert_idx] if t is not None else None
        return WeightPack(
            weight=self.weight[expert_idx],
            weight_scale=pick(self.weight_scale),
            weight_zero_point=pick(self.weight_zero_point),
        )


class QuantizationMethod(ABC):
    def __init__(self):
        super().__init__()
        self.device_id_ = torch.cuda.current_device() if torch.cuda.is_available() else 0
        self.weight_suffix = "weight"
        self.weight_scale_suffix = None
        self.weight_zero_point_suffix = None
        self.act_scale_suffix = None
        self.has_weight_scale: bool = None
        self.has_weight_zero_point: bool = None
        self.group_size: int = -1  # -1: per-channel; otherwise the group size
        self.pack_factor: int = 1
        self.hf_quantization_config = None

    @abstractmethod
    def quantize(self, weight: torch.Tensor, output: WeightPack) -> None:
        pass

    @abstractmethod
    def apply(
        self,
        input_tensor: torch.Tensor,
        weight_pack: "WeightPack",
        out: Optional[torch.Tensor] = None,
        workspace: Optional[torch.Tensor] = None,
        use_custom_tensor_mananger: bool = True,
        bias: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        pass

    @property
    @abstractmethod
    def method_name(self):
        pass

    def create_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int
    ) -> Tuple[WeightPack, List[WeightPack]]:
        return self._create_weight(out_dims=out_dims, in_dim=in_dim, dtype=dtype, device_id=device_id)

    def create_moe_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int, num_experts: int
    ) -> Tuple[WeightPack, List[WeightPack]]:
        return self._create_weight(
            out_dims=out_dims, in_dim=in_dim, dtype=dtype, device_id=device_id, num_experts=num_experts
        )

    def load_weight(self, weight: torch.Tensor, weight_pack: WeightPack) -> None:
        if self._check_weight_need_quanted(weight):
            self.quantize(weight, weight_pack)
            weight_pack.load_ok = [True, True, True]
            return
        weight_pack.weight[:].copy_(weight)
        weight_pack.load_ok[0] = True

    def load_weight_scale(self, weight_scale: torch.Tensor, weight_pack: WeightPack) -> None:
        if weight_scale is None:
            return
        weight_pack.weight_scale.copy_(weight_scale)
        weight_pack.load_ok[1] = True

    def load_weight_zero_point(self, weight_zero_point: torch.Tensor, weight_pack: WeightPack) -> None:
        if weight_zero_point is None:
            return
        weight_pack.weight_zero_point.copy_(weight_zero_point)
        weight_pack.load_ok[2] = True

    def _check_weight_need_quanted(self, weight: torch.Tensor) -> bool:
        return weight.dtype in [torch.bfloat16, torch.float16, torch.float32, torch.float64]

    def _create_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int, num_experts: int = 1
    ) -> Tuple[WeightPack, List[WeightPack]]:
        pass

    def _split_weight_pack(
        self,
        weight_pack: WeightPack,
        weight_out_dims: List[int],
        weight_split_dim: Optional[int],
        weight_scale_out_dims: List[int] = None,
        weight_scale_split_dim: Optional[int] = None,
        weight_zero_point_out_dims: List[int] = None,
        weight_zero_point_split_dim: Optional[int] = None,
    ) -> List[WeightPack]:
        """Views of a fused weight, one per sub-weight (e.g. gate and up of gate_up_proj)."""
        n = len(weight_out_dims)
        weights = torch.split(weight_pack.weight, weight_out_dims, dim=weight_split_dim)
        scales = (
            [None] * n
            if weight_pack.weight_scale is None
            else torch.split(weight_pack.weight_scale, weight_scale_out_dims, dim=weight_scale_split_dim)
        )
        zeros = (
            [None] * n
            if weight_pack.weight_zero_point is None
            else torch.split(weight_pack.weight_zero_point, weight_zero_point_out_dims, dim=weight_zero_point_split_dim)
        )
        return [WeightPack(weight=w, weight_scale=s, weight_zero_point=z) for w, s, z in zip(weights, scales, zeros)]

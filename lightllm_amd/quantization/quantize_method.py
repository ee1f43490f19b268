"""Plug-in boundary of the quantized linear layers.

LightLLM's layer-weight classes (MMWeightTpl, FusedMoeWeight) talk to a quantization method through two
types, reproduced here with the same names, attributes, method names and argument order
(lightllm/common/quantization/quantize_method.py:8-149) so that they can hold an object from this package
unchanged:

  WeightPack          the up-to-three tensors of one weight ("parts": weight, weight_scale, weight_zero_point)
                      and ``load_ok``, one flag per part that tells the loader whether it has arrived
  QuantizationMethod  creates packs, loads checkpoint tensors into them (quantizing float weights on the way)
                      and applies the linear layer

Internally everything is written over the tuple of parts, so a method with or without scales / zero points
needs no special cases.
"""
from abc import ABC, abstractmethod
from typing import Callable, List, Optional, Sequence, Tuple

import torch

_PARTS = ("weight", "weight_scale", "weight_zero_point")
_FLOAT_DTYPES = (torch.bfloat16, torch.float16, torch.float32, torch.float64)


class WeightPack:
    """weight / weight_scale / weight_zero_point of one (possibly fused, possibly per-expert) weight."""

    def __init__(self, weight: Optional[torch.Tensor] = None, weight_scale: Optional[torch.Tensor] = None,
                 weight_zero_point: Optional[torch.Tensor] = None):
        self.weight = weight
        self.weight_scale = weight_scale
        self.weight_zero_point = weight_zero_point
        # a part the method does not use counts as loaded from the start; the weight itself never does
        self.load_ok = [False] + [getattr(self, part) is None for part in _PARTS[1:]]

    def parts(self) -> Tuple[Optional[torch.Tensor], ...]:
        return tuple(getattr(self, part) for part in _PARTS)

    def _map(self, fn: Callable[[torch.Tensor], torch.Tensor]) -> "WeightPack":
        return WeightPack(*(None if t is None else fn(t) for t in self.parts()))

    def get_expert(self, expert_idx: int) -> "WeightPack":
        assert self.weight.ndim == 3, f"weight must be a 3D tensor, but got {self.weight.ndim}"
        return self._map(lambda t: t[expert_idx])

    def __repr__(self):
        shapes = ", ".join(f"{p}={None if t is None else tuple(t.shape)}" for p, t in zip(_PARTS, self.parts()))
        return f"WeightPack({shapes}, load_ok={self.load_ok})"


class QuantizationMethod(ABC):
    # checkpoint tensor-name suffixes of the parts; subclasses override what they have
    weight_suffix = "weight"
    weight_scale_suffix: Optional[str] = None
    weight_zero_point_suffix: Optional[str] = None
    act_scale_suffix: Optional[str] = None
    has_weight_scale: Optional[bool] = None
    has_weight_zero_point: Optional[bool] = None
    group_size: int = -1   # -1: one scale per output channel; otherwise the quantization group / block size
    pack_factor: int = 1   # weights packed per storage element (sub-byte formats)

    def __init__(self):
        super().__init__()
        self.device_id_ = torch.cuda.current_device() if torch.cuda.is_available() else 0
        self.hf_quantization_config = None   # the checkpoint's own quantization_config, for methods that need it

    # ---- what a method must provide
    @abstractmethod
    def quantize(self, weight: torch.Tensor, output: WeightPack) -> None:
        """Quantize a float weight into the (pre-allocated) pack."""

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
        """input_tensor @ weight.T (+ bias) with this method's arithmetic."""

    @property
    @abstractmethod
    def method_name(self):
        ...

    def _create_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int, num_experts: int = 1
    ) -> Tuple[WeightPack, List[WeightPack]]:
        """Allocate the fused pack and its per-sub-weight views."""

    # ---- allocation
    def create_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int
    ) -> Tuple[WeightPack, List[WeightPack]]:
        return self._create_weight(out_dims=out_dims, in_dim=in_dim, dtype=dtype, device_id=device_id)

    def create_moe_weight(
        self, out_dims: List[int], in_dim: int, dtype: torch.dtype, device_id: int, num_experts: int
    ) -> Tuple[WeightPack, List[WeightPack]]:
        return self._create_weight(out_dims=out_dims, in_dim=in_dim, dtype=dtype, device_id=device_id,
                                   num_experts=num_experts)

    # ---- loading: one checkpoint tensor into one part of a pack
    def _check_weight_need_quanted(self, weight: torch.Tensor) -> bool:
        return weight.dtype in _FLOAT_DTYPES

    @staticmethod
    def _fill(weight_pack: WeightPack, part: int, value: Optional[torch.Tensor]) -> None:
        if value is None:
            return
        getattr(weight_pack, _PARTS[part]).copy_(value)
        weight_pack.load_ok[part] = True

    def load_weight(self, weight: torch.Tensor, weight_pack: WeightPack) -> None:
        if not self._check_weight_need_quanted(weight):
            weight_pack.weight[:].copy_(weight)        # already in the method's storage format
            weight_pack.load_ok[0] = True
            return
        self.quantize(weight, weight_pack)             # produces every part at once
        weight_pack.load_ok = [True] * len(_PARTS)

    def load_weight_scale(self, weight_scale: torch.Tensor, weight_pack: WeightPack) -> None:
        self._fill(weight_pack, 1, weight_scale)

    def load_weight_zero_point(self, weight_zero_point: torch.Tensor, weight_pack: WeightPack) -> None:
        self._fill(weight_pack, 2, weight_zero_point)

    # ---- views of a fused weight, one per sub-weight (e.g. gate and up of gate_up_proj)
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
        how: Sequence[Tuple[Optional[List[int]], Optional[int]]] = (
            (weight_out_dims, weight_split_dim),
            (weight_scale_out_dims, weight_scale_split_dim),
            (weight_zero_point_out_dims, weight_zero_point_split_dim),
        )
        count = len(weight_out_dims)
        columns = [
            [None] * count if tensor is None else list(torch.split(tensor, sizes, dim=dim))
            for tensor, (sizes, dim) in zip(weight_pack.parts(), how)
        ]
        return [WeightPack(*row) for row in zip(*columns)]

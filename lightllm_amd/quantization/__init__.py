from .fp8act_quant_kernel import (  # noqa: F401
    lightllm_per_token_group_quant_fp8,
    per_token_group_quant_fp8,
    tma_align_input_scale,
)
from .fp8w8a8_block_gemm_kernel import w8a8_block_fp8_matmul  # noqa: F401
from .fp8w8a8_block_quant_kernel import mm_weight_quant, weight_quant  # noqa: F401
from .weight_dequant import weight_dequant  # noqa: F401
from .quantize_method import QuantizationMethod, WeightPack  # noqa: F401
from .registry import QUANTMETHODS  # noqa: F401
from .w8a8 import FP8w8a8B128Mi355QuantizationMethod, FP8w8a8B128QuantizationMethod  # noqa: F401
from .quantcfg import EXPERT_DTYPE_TO_QUANT_TYPE, SUPPORTED_EXPERT_DTYPES, Quantcfg  # noqa: F401

from .grouped_fused_moe import (  # noqa: F401
    fused_experts,
    fused_experts_impl,
    grouped_matmul,
    inplace_fused_experts_impl,
    moe_align,
    moe_align1,
    moe_align2,
    moe_align_fused,
    outplace_fused_experts_impl,
)
from .moe_silu_and_mul import silu_and_mul_fwd  # noqa: F401
from .moe_silu_and_mul_mix_quant_ep import (  # noqa: F401
    silu_and_mul_masked_post_quant_fwd,
    silu_and_mul_post_quant_fwd,
)
from .moe_sum_reduce import moe_sum_reduce  # noqa: F401
from .grouped_fused_moe_ep import (  # noqa: F401
    _deepgemm_grouped_fp8_nt_masked,
    deepgemm_grouped_fp8_nt_contiguous,
    masked_group_gemm,
)

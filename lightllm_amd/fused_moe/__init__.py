from .grouped_fused_moe import grouped_matmul, moe_align2, moe_align_fused  # noqa: F401

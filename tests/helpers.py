"""Seeded synthetic inputs and comparison helpers shared by the tests (not part of the product)."""
import numpy as np
import torch

from oracle import torch_ref as tr


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def activations(M: int, K: int, seed: int = 0, outliers: bool = False, zero_row: bool = False) -> torch.Tensor:
    """bf16 [M,K] ~ N(0,1); optionally 1% of entries x50 and row 0 all zero (the quantizer bandwidth config)."""
    g = gen(seed)
    x = torch.randn((M, K), generator=g, dtype=torch.float32)
    if outliers:
        mask = torch.rand((M, K), generator=g) < 0.01
        x = torch.where(mask, x * 50.0, x)
    if zero_row and M > 0:
        x[0] = 0.0
    return x.to(torch.bfloat16)


def weights(N: int, K: int, seed: int = 1) -> torch.Tensor:
    """bf16 [N,K] ~ N(0, 0.02)."""
    return (torch.randn((N, K), generator=gen(seed), dtype=torch.float32) * 0.02).to(torch.bfloat16)


def quantized_weights(N: int, K: int, seed: int = 1, device="cpu"):
    """(q e4m3fn [N,K], s fp32 [ceil(N/128), ceil(K/128)]) via the torch closed form of the reference's
    load-time quantizer, evaluated on `device`."""
    w = weights(N, K, seed).to(device)
    if device == "cpu":
        return tr.block_weight_quant(w)
    return _block_weight_quant_any_device(w)


def _block_weight_quant_any_device(w: torch.Tensor, block: int = 128):
    N, K = w.shape
    nb, kb = -(-N // block), -(-K // block)
    wf = torch.zeros((nb * block, kb * block), dtype=torch.float32, device=w.device)
    wf[:N, :K] = w.float()
    blocks = wf.reshape(nb, block, kb, block).permute(0, 2, 1, 3)
    scale = blocks.abs().amax(dim=(-1, -2)) / 448.0
    q = (blocks / (scale + 1e-6)[:, :, None, None]).to(torch.float8_e4m3fn)
    q = q.permute(0, 2, 1, 3).reshape(nb * block, kb * block)[:N, :K].contiguous()
    return q, scale.contiguous()


def routing(T: int, E: int, topk: int, seed: int = 5, zipf_s: float = 1.1):
    """Seeded Zipf(s) expert popularity over a random permutation, top-k without replacement.
    -> (topk_ids int32 [T,topk], topk_weights fp32 [T,topk])."""
    g = gen(seed)
    perm = torch.randperm(E, generator=g)
    p = torch.zeros(E, dtype=torch.float64)
    p[perm] = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** zipf_s
    p = (p / p.sum()).float()
    ids = torch.multinomial(p.expand(T, E), topk, replacement=False, generator=g).to(torch.int32)
    w = torch.softmax(torch.randn((T, topk), generator=g), dim=-1).float()
    return ids.contiguous(), w.contiguous()


def gemm_metrics(c: torch.Tensor, ref: torch.Tensor):
    return tr.cosine(c, ref), tr.max_rel_err(c, ref)


# acceptance thresholds of the block-FP8 GEMM against the fp32 dequant-then-matmul
GEMM_MAX_REL = 1e-2
GEMM_MIN_COS = 0.9999

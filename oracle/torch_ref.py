"""The reference's torch closed forms, evaluated with torch on the CPU.  TEST INFRASTRUCTURE ONLY.

Second, independent restatement next to ``fp8_oracle.c``: it relies on torch's
own ``float8_e4m3fn`` cast instead of the C file's rounding code, so agreement
between the two pins both.  ``dequant_matmul`` is also the CPU baseline that
``bench.py`` times (the reference's in-file check, evaluated in fp32).
"""
import numpy as np
import torch

FP8_MAX = 448.0


def bits_of(t: torch.Tensor) -> np.ndarray:
    """Raw bit patterns of a bf16 / float8 / fp32 tensor as a numpy unsigned array."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    raise TypeError(t.dtype)


def bf16_from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)


def fp8_from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint8)).view(torch.float8_e4m3fn)


def group_quant(x: torch.Tensor, group: int = 128, eps: float = 1e-10):
    """torch_quant (quantization/fp8act_quant_kernel.py:239-251) plus the kernel's eps floor (:55).

    x: bf16 [M,K] -> (q float8_e4m3fn [M,K], s float32 [M,K/group]).
    """
    M, K = x.shape
    xf = x.to(torch.float32).reshape(-1, group)
    amax = xf.abs().max(-1)[0].clamp_min(torch.tensor(eps, dtype=torch.float32))
    s = amax / FP8_MAX
    q = (xf / s.reshape(-1, 1)).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(M, K), s.reshape(M, K // group)


def block_weight_quant(w: torch.Tensor, block: int = 128):
    """weight_quant_kernel (quantization/fp8w8a8_block_quant_kernel.py:18-27) on one [N,K] matrix."""
    N, K = w.shape
    nb, kb = -(-N // block), -(-K // block)
    wf = torch.zeros((nb * block, kb * block), dtype=torch.float32)
    wf[:N, :K] = w.to(torch.float32)
    blocks = wf.reshape(nb, block, kb, block).permute(0, 2, 1, 3)
    amax = blocks.abs().amax(dim=(-1, -2))
    scale = amax / FP8_MAX
    div = scale + torch.tensor(1e-6, dtype=torch.float32)
    q = (blocks / div[:, :, None, None]).to(torch.float8_e4m3fn)
    q = q.permute(0, 2, 1, 3).reshape(nb * block, kb * block)[:N, :K].contiguous()
    return q, scale


def dequant(q: torch.Tensor, s: torch.Tensor, bn: int, bk: int) -> torch.Tensor:
    """Expand block scales over a [R,K] fp8 matrix: bn rows x bk columns per scale (bn=1 for activations)."""
    R, K = q.shape
    se = s.repeat_interleave(bk, dim=1)[:, :K]
    if bn > 1:
        se = se.repeat_interleave(bn, dim=0)[:R]
    return q.to(torch.float32) * se


def dequant_matmul(Aq, As, Bq_nk, Bs_nk, block=(128, 128), out_dtype=torch.bfloat16) -> torch.Tensor:
    """fp32 dequant-then-matmul (quantization/fp8w8a8_block_gemm_kernel.py:213-217, in fp32)."""
    bn, bk = block
    dA = dequant(Aq, As, 1, bk)
    dB = dequant(Bq_nk, Bs_nk, bn, bk)
    return (dA @ dB.T).to(out_dtype)


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().flatten()
    b = b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-300))


def max_rel_err(c: torch.Tensor, ref: torch.Tensor) -> float:
    """max|c - ref| / max|ref| : the relative-error form the acceptance threshold (1e-2) is stated in."""
    return float((c.double() - ref.double()).abs().max() / ref.double().abs().max().clamp_min(1e-300))

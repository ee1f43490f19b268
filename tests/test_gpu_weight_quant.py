"""GPU parity of the load-time 128x128 block weight quantizer: bytes and scale bits against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,K", [(128, 128), (256, 384), (200, 300), (200, 304), (2112, 1024), (1, 1), (1, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_bit_exact(hip, N, K, dtype):
    from lightllm_amd.quantization import mm_weight_quant

    print(f"weight quant N={N} K={K} {dtype}", flush=True)
    w = H.weights(N, K, seed=N + K).to(dtype)
    q, s = mm_weight_quant(w.cuda())
    torch.cuda.synchronize()
    q_ref, s_ref = oracle.block_weight_quant(w.float().numpy())
    assert np.array_equal(tr.bits_of(s), s_ref.view(np.uint32))
    assert np.array_equal(tr.bits_of(q), q_ref)


def test_three_dims_and_zero_block(hip):
    from lightllm_amd.quantization import weight_quant

    w = H.weights(3 * 256, 256, seed=5).reshape(3, 256, 256).contiguous()
    w[1, :128, :128] = 0  # an all-zero block: scale 0, divisor 1e-6, bytes 0
    q, s = weight_quant(w.cuda())
    torch.cuda.synchronize()
    for e in range(3):
        q_ref, s_ref = oracle.block_weight_quant(w[e].float().numpy())
        assert np.array_equal(tr.bits_of(q[e].contiguous()), q_ref)
        assert np.array_equal(tr.bits_of(s[e].contiguous()), s_ref.view(np.uint32))
    assert float(s[1, 0, 0]) == 0.0

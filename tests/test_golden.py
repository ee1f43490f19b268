"""The committed fixtures (tests/golden) against the CPU oracle, and - on the GPU - against the HIP kernels."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref as tr
from tests import helpers as H

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(HERE, "small_vectors.npz"))


def test_oracle_reproduces_small_vectors(vec):
    for name in ("normal", "outliers", "allbits"):
        q, s = oracle.group_quant_fp8(vec[f"quant_{name}_x"])
        assert np.array_equal(q, vec[f"quant_{name}_q"]) and np.array_equal(s.view(np.uint32), vec[f"quant_{name}_s"])
    wq, ws = oracle.block_weight_quant(oracle.bf16_to_f32(vec["wquant_w"]))
    assert np.array_equal(wq, vec["wquant_q"]) and np.array_equal(ws.view(np.uint32), vec["wquant_s"])
    c = oracle.block_gemm(vec["gemm_xq"], vec["gemm_xs"].view(np.float32), vec["gemm_wq"], vec["gemm_ws"].view(np.float32))
    assert np.array_equal(c, vec["gemm_c"])


def test_torch_closed_form_reproduces_small_vectors(vec):
    for name in ("normal", "outliers"):
        q, s = tr.group_quant(tr.bf16_from_bits(vec[f"quant_{name}_x"]))
        assert np.array_equal(tr.bits_of(q), vec[f"quant_{name}_q"])
        assert np.array_equal(tr.bits_of(s), vec[f"quant_{name}_s"])


def test_oracle_reproduces_digests():
    d = json.load(open(os.path.join(HERE, "digests.json")))
    x = tr.bits_of(H.activations(32, 4096, seed=0))
    q, s = oracle.group_quant_fp8(x)
    assert {"x": _sha(x), "q": _sha(q), "s": _sha(s)} == d["quant_cfg1_32x4096_seed0"]
    x = tr.bits_of(H.activations(512, 7168, seed=0, outliers=True, zero_row=True))
    q, s = oracle.group_quant_fp8(x)
    assert {"x": _sha(x), "q": _sha(q), "s": _sha(s)} == d["quant_outliers_512x7168_seed0"]


@pytest.mark.gpu
def test_hip_kernels_reproduce_fixtures(vec, hip):
    from lightllm_amd.quantization import mm_weight_quant, per_token_group_quant_fp8, w8a8_block_fp8_matmul

    for name in ("normal", "outliers", "allbits"):
        xq, xs = per_token_group_quant_fp8(tr.bf16_from_bits(vec[f"quant_{name}_x"]).cuda(), 128)
        assert np.array_equal(tr.bits_of(xq), vec[f"quant_{name}_q"]), name
        assert np.array_equal(tr.bits_of(xs), vec[f"quant_{name}_s"]), name
    wq, ws = mm_weight_quant(tr.bf16_from_bits(vec["wquant_w"]).cuda())
    assert np.array_equal(tr.bits_of(wq), vec["wquant_q"]) and np.array_equal(tr.bits_of(ws), vec["wquant_s"])
    d = json.load(open(os.path.join(HERE, "digests.json")))
    for key, kw, shape in (("quant_cfg1_32x4096_seed0", {}, (32, 4096)),
                           ("quant_outliers_512x7168_seed0", {"outliers": True, "zero_row": True}, (512, 7168))):
        x = H.activations(*shape, seed=0, **kw)
        xq, xs = per_token_group_quant_fp8(x.cuda(), 128)
        assert _sha(tr.bits_of(xq)) == d[key]["q"] and _sha(tr.bits_of(xs).view(np.float32)) == d[key]["s"]
    # GEMM fixture: within one bf16 ulp of the frozen oracle output (summation order may differ)
    xq = tr.fp8_from_bits(vec["gemm_xq"]).cuda()
    wq = tr.fp8_from_bits(vec["gemm_wq"]).cuda()
    xs = torch.from_numpy(vec["gemm_xs"].view(np.float32)).cuda()
    ws = torch.from_numpy(vec["gemm_ws"].view(np.float32)).cuda()
    C = torch.empty((8, 136), dtype=torch.bfloat16, device="cuda")
    w8a8_block_fp8_matmul(xq, wq.t(), xs, ws.t(), C, [128, 128])
    ref = tr.bf16_from_bits(vec["gemm_c"]).float()
    assert (C.float().cpu() - ref).abs().max() <= ref.abs().max() * 2 ** -7

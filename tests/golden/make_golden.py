"""Writes the golden fixtures of this directory from the CPU oracle (run from the repository root:
`python tests/golden/make_golden.py`).  The reference ships no byte-level vectors for this path (its tests
compare with tolerances), so these vectors are produced by the oracle AFTER it has been pinned by
tests/test_oracle_fp8.py, and they freeze its behaviour: a later change to the oracle that alters any byte fails
tests/test_golden.py.  Small cases hold full inputs and outputs; large ones hold SHA-256 digests.
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from oracle import torch_ref as tr  # noqa: E402
from tests import helpers as H  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    # 1. quantizer, small, full vectors: normal, outliers + zero row, wide dynamic range
    x1 = tr.bits_of(H.activations(4, 256, seed=0))
    x2 = tr.bits_of(H.activations(4, 256, seed=1, outliers=True, zero_row=True))
    rng = np.random.default_rng(2)
    x3 = rng.integers(0, 0x7F80, (4, 256)).astype(np.uint16) | (rng.integers(0, 2, (4, 256)).astype(np.uint16) << 15)
    out = {}
    for name, x in (("normal", x1), ("outliers", x2), ("allbits", x3)):
        q, s = oracle.group_quant_fp8(x)
        out[f"quant_{name}_x"] = x
        out[f"quant_{name}_q"] = q
        out[f"quant_{name}_s"] = s.view(np.uint32)
    # 2. weight quantizer, one ragged matrix
    w = H.weights(130, 200, seed=3).float().numpy()
    wq, ws = oracle.block_weight_quant(w)
    out.update(wquant_w=tr.bits_of(H.weights(130, 200, seed=3)), wquant_q=wq, wquant_s=ws.view(np.uint32))
    # 3. block GEMM, small
    xq, xs = oracle.group_quant_fp8(tr.bits_of(H.activations(8, 256, seed=4)))
    wq2, ws2 = oracle.block_weight_quant(H.weights(136, 256, seed=5).float().numpy())
    c = oracle.block_gemm(xq, xs, wq2, ws2)
    out.update(gemm_xq=xq, gemm_xs=xs.view(np.uint32), gemm_wq=wq2, gemm_ws=ws2.view(np.uint32), gemm_c=c)
    np.savez_compressed(os.path.join(HERE, "small_vectors.npz"), **out)

    # 4. digests of larger cases (inputs are regenerated from the seeds by the test)
    digests = {}
    x = tr.bits_of(H.activations(32, 4096, seed=0))
    q, s = oracle.group_quant_fp8(x)
    digests["quant_cfg1_32x4096_seed0"] = {"x": sha(x), "q": sha(q), "s": sha(s)}
    x = tr.bits_of(H.activations(512, 7168, seed=0, outliers=True, zero_row=True))
    q, s = oracle.group_quant_fp8(x)
    digests["quant_outliers_512x7168_seed0"] = {"x": sha(x), "q": sha(q), "s": sha(s)}
    with open(os.path.join(HERE, "digests.json"), "w") as f:
        json.dump(digests, f, indent=1, sort_keys=True)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()

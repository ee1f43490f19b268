"""CPU oracle for the block-FP8 W8A8 linear path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped package ``lightllm_amd``
never does: its product path runs on the HIP library or fails loudly.

Two independent restatements of the reference arithmetic live here so that each
can pin the other:

* ``fp8_oracle.c`` - scalar C with its own e4m3fn rounding, loaded through ctypes
  (functions below; numpy arrays in, numpy arrays out);
* ``torch_ref.py`` - the reference's torch closed forms evaluated on the CPU
  (torch's own float8 cast).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile fp8_oracle.c with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(
        os.path.join(_HERE, "fp8_oracle.c")
    ):
        subprocess.check_call(["make", "-s", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()  # no-op unless the library is missing or older than its source
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_moe_align2_rows.restype = ctypes.c_int64
        _lib.oracle_moe_align2_rows.argtypes = [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]
        _lib.oracle_fast_quant_mismatches.restype = ctypes.c_int64
        _lib.oracle_fast_quant_mismatches.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


I64 = ctypes.c_int64
I32 = ctypes.c_int32
F32 = ctypes.c_float


def f32_to_e4m3fn(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().oracle_f32_to_e4m3fn_array(_p(x), I64(x.size), _p(out))
    return out


def e4m3fn_to_f32(b) -> np.ndarray:
    b = _c(b, np.uint8)
    out = np.empty(b.shape, np.float32)
    lib().oracle_e4m3fn_to_f32_array(_p(b), I64(b.size), _p(out))
    return out


def f32_to_bf16(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_bf16_array(_p(x), I64(x.size), _p(out))
    return out


def bf16_to_f32(h) -> np.ndarray:
    h = _c(h, np.uint16)
    return (h.astype(np.uint32) << 16).view(np.float32)


def group_quant_fp8(x_bf16_bits, group: int = 128, eps: float = 1e-10, column_major: bool = False):
    """x: uint16 [M,K] bf16 bit patterns -> (q uint8 [M,K], s float32 [M,K/group]).

    With ``column_major`` the scales come back as an [M, K/group] view of a
    [K/group, M] buffer, i.e. strides (1, M).
    """
    x = _c(x_bf16_bits, np.uint16)
    M, K = x.shape
    assert K % group == 0
    G = K // group
    q = np.empty((M, K), np.uint8)
    if column_major:
        buf = np.empty((G, M), np.float32)
        lib().oracle_group_quant_fp8(_p(x), I64(M), I64(K), I32(group), F32(eps), _p(q), _p(buf), I64(1), I64(M))
        return q, buf.T
    s = np.empty((M, G), np.float32)
    lib().oracle_group_quant_fp8(_p(x), I64(M), I64(K), I32(group), F32(eps), _p(q), _p(s), I64(G), I64(1))
    return q, s


def group_quant_fp8_f32(x_f32, group: int = 128, eps: float = 1e-10):
    """x: float32 [M,K] (fp16 and bf16 inputs widen exactly) -> (q uint8 [M,K], s float32 [M,K/group])."""
    x = _c(x_f32, np.float32)
    M, K = x.shape
    assert K % group == 0
    G = K // group
    q = np.empty((M, K), np.uint8)
    s = np.empty((M, G), np.float32)
    lib().oracle_group_quant_fp8_f32(_p(x), I64(M), I64(K), I32(group), F32(eps), _p(q), _p(s), I64(G), I64(1))
    return q, s


def block_weight_quant(w_f32, block: int = 128):
    """w: float32 [N,K] -> (q uint8 [N,K], s float32 [ceil(N/b), ceil(K/b)])."""
    w = _c(w_f32, np.float32)
    N, K = w.shape
    q = np.empty((N, K), np.uint8)
    s = np.empty(((N + block - 1) // block, (K + block - 1) // block), np.float32)
    lib().oracle_block_weight_quant(_p(w), I64(N), I64(K), I32(block), _p(q), _p(s))
    return q, s


def block_gemm(Aq, As, Bq_nk, Bs_nk, bn: int = 128, bk: int = 128, want_f32: bool = False):
    """Aq [M,K] u8, As [M,K/bk] f32, Bq [N,K] u8, Bs [ceil(N/bn),K/bk] f32 -> bf16 bits [M,N]."""
    Aq, As, Bq, Bs = _c(Aq, np.uint8), _c(As, np.float32), _c(Bq_nk, np.uint8), _c(Bs_nk, np.float32)
    M, K = Aq.shape
    N = Bq.shape[0]
    assert Bq.shape[1] == K and As.shape == (M, (K + bk - 1) // bk)
    assert Bs.shape == ((N + bn - 1) // bn, (K + bk - 1) // bk)
    cbf = np.empty((M, N), np.uint16)
    c32 = np.empty((M, N), np.float32)
    lib().oracle_block_gemm(_p(Aq), _p(As), _p(Bq), _p(Bs), I64(M), I64(N), I64(K), I32(bn), I32(bk), _p(c32), _p(cbf))
    return (cbf, c32) if want_f32 else cbf


def dequant_matmul_sampled(Aq, As, Bq_nk, Bs_nk, rows, cols, bn: int = 128, bk: int = 128) -> np.ndarray:
    """float64 dequant-then-matmul at C[rows][:, cols]."""
    Aq, As, Bq, Bs = _c(Aq, np.uint8), _c(As, np.float32), _c(Bq_nk, np.uint8), _c(Bs_nk, np.float32)
    rows, cols = _c(rows, np.int64), _c(cols, np.int64)
    M, K = Aq.shape
    N = Bq.shape[0]
    out = np.empty((rows.size, cols.size), np.float64)
    lib().oracle_dequant_matmul_sampled(
        _p(Aq), _p(As), _p(Bq), _p(Bs), I64(M), I64(N), I64(K), I32(bn), I32(bk),
        _p(rows), I64(rows.size), _p(cols), I64(cols.size), _p(out),
    )
    return out


def moe_align_fused(topk_ids, topk_weights, num_experts: int):
    """-> (expert_to_token_index int32 [E,P] (-1 where unset), expert_to_weight f32 [E,P], expert_token_num int32 [E])."""
    ids = _c(topk_ids, np.int32).reshape(-1)
    w = _c(topk_weights, np.float32).reshape(-1)
    P = ids.size
    idx = np.full((num_experts, P), -1, np.int32)
    ew = np.zeros((num_experts, P), np.float32)
    cnt = np.empty((num_experts,), np.int32)
    lib().oracle_moe_align_fused(_p(ids), _p(w), I64(P), I32(num_experts), _p(idx), _p(ew), _p(cnt))
    return idx, ew, cnt


def moe_align(topk_ids, num_experts: int) -> np.ndarray:
    ids = _c(topk_ids, np.int32).ravel()
    out = np.empty((num_experts, ids.size), np.int32)
    lib().oracle_moe_align(_p(ids), I64(ids.size), I32(num_experts), _p(out))
    return out


def moe_align1(experts_info, topk_weights, experts_weight_info):
    """In place on copies of the two tables -> (experts_info, experts_weight_info, expert_token_num)."""
    info = np.array(experts_info, dtype=np.int32, order="C", copy=True)
    wout = np.array(experts_weight_info, dtype=np.float32, order="C", copy=True)
    w = _c(topk_weights, np.float32).ravel()
    E, P = info.shape
    assert w.size == P and wout.shape == info.shape
    cnt = np.empty((E,), np.int32)
    lib().oracle_moe_align1(_p(info), _p(w), I64(P), I32(E), _p(wout), _p(cnt))
    return info, wout, cnt


def moe_align2(num_pairs: int, expert_token_num, block_m: int) -> np.ndarray:
    """-> int32 [max_blocks, 4]; columns 1-3 of padding rows are left at -1 here."""
    cnt = _c(expert_token_num, np.int32)
    E = cnt.size
    rows = lib().oracle_moe_align2_rows(I64(num_pairs), I32(E), I32(block_m))
    table = np.full((rows, 4), -1, np.int32)
    lib().oracle_moe_align2(_p(cnt), I32(E), I32(block_m), I64(rows), _p(table))
    return table


def grouped_block_gemm(Xq, Xs, W, Ws, expert_to_token_index, expert_to_weights, expert_token_num,
                       topk_num: int, mul_routed_weight: bool, bn: int = 128, bk: int = 128, out=None, bias=None):
    """-> bf16 bits [num_pairs, N]; rows no pair maps to keep the value they had in ``out`` (zeros if None).
    ``bias`` fp32 [E, N] is added to the accumulator before the routed weight."""
    Xq, Xs, W, Ws = _c(Xq, np.uint8), _c(Xs, np.float32), _c(W, np.uint8), _c(Ws, np.float32)
    idx, ew, cnt = _c(expert_to_token_index, np.int32), _c(expert_to_weights, np.float32), _c(expert_token_num, np.int32)
    E, N, K = W.shape
    P = idx.shape[1]
    if out is None:
        out = np.zeros((P, N), np.uint16)
    bias = None if bias is None else _c(bias, np.float32)
    assert bias is None or bias.shape == (E, N)
    lib().oracle_grouped_block_gemm(
        _p(Xq), _p(Xs), _p(W), _p(Ws), _p(idx), _p(ew), _p(cnt), I64(P), I32(E), I32(topk_num),
        I64(N), I64(K), I32(bn), I32(bk), I32(1 if mul_routed_weight else 0),
        _p(bias) if bias is not None else None, _p(out),
    )
    return out


def fast_quant_mismatches(amax_lo: int = 0, amax_hi: int = 0x7F80, step: int = 1) -> int:
    """Pairs (bf16 amax, bf16 x) for which the HIP quantizer's division shortcut would differ from IEEE."""
    return int(lib().oracle_fast_quant_mismatches(amax_lo, amax_hi, step))


def silu_and_mul(x_bf16_bits) -> np.ndarray:
    x = _c(x_bf16_bits, np.uint16)
    M, H2 = x.shape
    out = np.empty((M, H2 // 2), np.uint16)
    lib().oracle_silu_and_mul(_p(x), I64(M), I64(H2 // 2), _p(out))
    return out


def silu_and_mul_ex(x_bf16_bits, layout: str = "blocked", limit=None, alpha=None) -> np.ndarray:
    x = _c(x_bf16_bits, np.uint16)
    M, H2 = x.shape
    out = np.empty((M, H2 // 2), np.uint16)
    lib().oracle_silu_and_mul_ex(_p(x), I64(M), I64(H2 // 2), I32(1 if layout == "interleaved" else 0),
                                 I32(0 if limit is None else 1), F32(0.0 if limit is None else limit),
                                 F32(0.0 if alpha is None else alpha), _p(out))
    return out


def moe_sum_reduce(x_bf16_bits) -> np.ndarray:
    x = _c(x_bf16_bits, np.uint16)
    T, topk, H = x.shape
    out = np.empty((T, H), np.uint16)
    lib().oracle_moe_sum_reduce(_p(x), I64(T), I32(topk), I64(H), _p(out))
    return out


def block_weight_dequant(q_bytes, scales, block: int = 128) -> np.ndarray:
    q, sc = _c(q_bytes, np.uint8), _c(scales, np.float32)
    N, K = q.shape
    assert sc.shape == ((N + block - 1) // block, (K + block - 1) // block)
    out = np.empty((N, K), np.uint16)
    lib().oracle_block_weight_dequant(_p(q), _p(sc), I64(N), I64(K), I32(block), _p(out))
    return out


def silu_and_mul_group_quant(x_bf16_bits, group: int = 128):
    """silu_and_mul followed by the group quantizer: what the fused kernel must reproduce
    (fused_moe/moe_silu_and_mul_mix_quant_ep.py:51-74 repeats the quantizer's arithmetic on the bf16 product)."""
    return group_quant_fp8(silu_and_mul(x_bf16_bits), group)


def fused_experts(x_bf16_bits, w1_q, w1_s, w2_q, w2_s, topk_ids, topk_weights, layout="blocked", limit=None,
                  alpha=None, w1_bias=None, w2_bias=None) -> np.ndarray:
    """The routed-expert FFN as the reference sequences it (fused_moe/grouped_fused_moe.py:1048-1113):
    routing tables, quantize, gate/up grouped GEMM, silu_and_mul, quantize, down grouped GEMM times the routed
    weight, sum over slots.  x bf16 bits [T,H]; w1 e4m3 bytes [E,2I,H]; w2 [E,H,I] -> bf16 bits [T,H]."""
    x = _c(x_bf16_bits, np.uint16)
    ids = _c(topk_ids, np.int32)
    T, topk = ids.shape
    E = w1_q.shape[0]
    idx, ew, cnt = moe_align_fused(ids, topk_weights, E)
    xq, xs = group_quant_fp8(x)
    h1 = grouped_block_gemm(xq, xs, w1_q, w1_s, idx, ew, cnt, topk, False, bias=w1_bias)
    aq, as_ = group_quant_fp8(silu_and_mul_ex(h1, layout, limit, alpha))
    h3 = grouped_block_gemm(aq, as_, w2_q, w2_s, idx, ew, cnt, 1, True, bias=w2_bias)
    return moe_sum_reduce(h3.reshape(T, topk, -1))

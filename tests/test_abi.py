"""CPU checks of the drop-in boundary: the library loads and exports every symbol the header declares, the
ctypes table covers the header, the Python functions keep the reference's signatures, and argument checks
fire before any launch."""
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "mi355_fp8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from lightllm_amd import _lib

    lib = _lib.lib()
    names = _header_symbols()
    assert len(names) >= 11
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_error_strings():
    from lightllm_amd import _lib

    lib = _lib.lib()
    assert lib.mi355_error_string(0) == b"ok"
    for code in range(-6, 0):
        assert lib.mi355_error_string(code) not in (b"ok", b"unknown error code")
    assert lib.mi355_error_string(-99) == b"unknown error code"


def test_pure_host_entry_points():
    from lightllm_amd import _lib

    lib = _lib.lib()
    # rows of the schedule table: min(pairs, ceil((pairs + E*(bm-1))/bm))   (reference test_moe_align2)
    assert lib.mi355_moe_align2_rows(100, 4, 16) == 10
    assert lib.mi355_moe_align2_rows(8, 10, 16) == 8
    assert lib.mi355_grouped_block_m(32768, 256, 4096, 7168) == 256
    assert lib.mi355_grouped_block_m(32768, 256, 4096, 7168 + 128) == 256   # any K/128 takes the 256-row blocks
    assert lib.mi355_grouped_block_m(64, 256, 4096, 7168) == 16
    # 12..64 rows per expert: the two-queue launch of 256-row blocks where it has more tiles than compute units
    # (256 assumed without a device), the row-sized tiles otherwise
    assert lib.mi355_grouped_block_m(8192, 256, 4096, 7168) == 256
    assert lib.mi355_grouped_block_m(2048, 256, 4096, 7168) == 16
    assert lib.mi355_grouped_block_m(16 * 24, 16, 4096, 7168) == 32
    assert lib.mi355_grouped_block_m(16 * 50, 16, 4096, 8192) == 64
    assert lib.mi355_grouped_block_m(64 * 50, 64, 1024, 7168) == 64
    assert lib.mi355_grouped_block_m(64 * 50, 64, 2816, 2048) == 128
    # 8 experts: 64-row blocks from 9 rows per expert; few tiles or a small launch with a short K: 128-row blocks
    assert lib.mi355_grouped_block_m(8 * 24, 8, 4096, 7168) == 64
    assert lib.mi355_grouped_block_m(8 * 50, 8, 4096, 14336) == 128
    assert lib.mi355_grouped_block_m(128 * 64, 128, 2048, 768) == 128
    assert lib.mi355_grouped_block_m(128 * 300, 128, 2048, 768) == 256
    # an expert's N under 4096: the two-queue launch from 25 rows per expert
    assert lib.mi355_grouped_block_m(128 * 16, 128, 3072, 4096) == 16
    assert lib.mi355_grouped_block_m(128 * 32, 128, 3072, 4096) == 256
    assert lib.mi355_block_fp8_gemm_workspace_bytes(4096, 4096, 4096, 0) == 65536  # large M: tile counters only
    assert lib.mi355_block_fp8_gemm_workspace_bytes(32, 4096, 14336, 0) > 65536   # the stream shares K
    assert lib.mi355_block_fp8_gemm_workspace_bytes(8, 4096, 14336, 0) == 0        # one share per unit, whole K


def test_preconditions_are_checked_before_launch():
    """Null pointers and bad shapes are rejected on the host; nothing reaches the (absent) GPU."""
    from lightllm_amd import _lib

    lib = _lib.lib()
    assert lib.mi355_group_quant_fp8(None, 0, None, None, 4, 100, 128, 1e-10, 1, 1, None) == -2   # K % 128
    assert lib.mi355_group_quant_fp8(None, 0, None, None, 4, 256, 0, 1e-10, 4, 1, None) == -1     # group <= 0
    assert lib.mi355_group_quant_fp8(None, 0, None, None, 4, 256, 96, 1e-10, 4, 1, None) == -2    # K % group
    assert lib.mi355_group_quant_fp8(None, 0, None, None, 4, 256, 128, 1e-10, 2, 1, None) == -1   # null
    assert lib.mi355_group_quant_fp8(None, 0, None, None, 0, 256, 128, 1e-10, 2, 1, None) == 0    # empty
    # other block sizes: only the plain kernel (AUTO or GENERIC) takes them
    assert lib.mi355_block_fp8_gemm(None, None, None, None, None, 4, 4, 128, 128, 1, 128, 4, 1, 1, 1, 1, 64, 128,
                                    None, 0, 2, None) == -6
    assert lib.mi355_block_fp8_gemm(None, None, None, None, None, 4, 4, 128, 128, 1, 128, 4, 1, 1, 1, 1, 64, 128,
                                    None, 0, 0, None) == -1
    assert lib.mi355_block_fp8_gemm(None, None, None, None, None, 4, 4, 128, 128, 1, 128, 4, 1, 1, 1, 1, 0, 128,
                                    None, 0, 0, None) == -1
    assert lib.mi355_block_fp8_gemm(None, None, None, None, None, 4, 4, 128, 128, 1, 128, 4, 1, 1, 1, 1, 128, 128,
                                    None, 0, 0, None) == -1
    assert lib.mi355_block_fp8_gemm(None, None, None, None, None, 0, 4, 128, 128, 1, 128, 4, 1, 1, 1, 1, 128, 128,
                                    None, 0, 0, None) == 0
    assert lib.mi355_block_weight_quant_fp8(None, 7, None, None, 4, 4, 128, None) == -1
    assert lib.mi355_moe_align2(None, 0, 16, 4, None, None) == -1


REFERENCE_SIGNATURES = {
    # (module, function): signature string of the reference's function of the same name
    ("lightllm_amd.quantization.fp8act_quant_kernel", "per_token_group_quant_fp8"):
        "(x, group_size, eps=1e-10, dtype=torch.float8_e4m3fn, column_major_scales=False, scale_tma_aligned=False, alloc_func=torch.empty)",
    ("lightllm_amd.quantization.fp8act_quant_kernel", "lightllm_per_token_group_quant_fp8"):
        "(x, group_size, x_q, x_s, eps=1e-10, dtype=torch.float8_e4m3fn)",
    ("lightllm_amd.quantization.fp8w8a8_block_gemm_kernel", "w8a8_block_fp8_matmul"):
        "(A, B, Ascale, Bscale, C, block_size, dtype=torch.bfloat16, run_config=None)",
    ("lightllm_amd.quantization.fp8w8a8_block_quant_kernel", "weight_quant"): "(x, block_size=128)",
    ("lightllm_amd.quantization.fp8w8a8_block_quant_kernel", "mm_weight_quant"): "(x, block_size=128)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "moe_align_fused"):
        "(expert_to_token_index, expert_to_weight, expert_token_num, topk_ids, topk_weights)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "moe_align2"): "(token_num_mul_topk_num, exports_token_num, block_m)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "grouped_matmul"):
        "(token_num_mul_topk_num, token_inputs, token_input_scale, expert_to_token_num, expert_to_token_index, "
        "expert_to_weights, expert_weights, expert_to_weights_scale, topk_num, out, mul_routed_weight, use_fp8_w8a8, "
        "alloc_tensor_func=torch.empty, reused_mblock_infos=None, run_config=None, bias=None)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "fused_experts_impl"):
        "(hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, use_fp8_w8a8=False, use_int8_w8a16=False, "
        "w1_bias=None, w2_bias=None, w1_scale=None, w2_scale=None, a1_scale=None, a2_scale=None, "
        "alloc_tensor_func=torch.empty, run_config=None, layout=blocked, limit=None, alpha=None)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "inplace_fused_experts_impl"):
        "(hidden_states, w1, w2, topk_weights, topk_ids, use_fp8_w8a8=False, use_int8_w8a16=False, w1_bias=None, "
        "w2_bias=None, w1_scale=None, w2_scale=None, a1_scale=None, a2_scale=None, layout=blocked, alpha=None, limit=None)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "outplace_fused_experts_impl"):
        "(hidden_states, w1, w2, topk_weights, topk_ids, use_fp8_w8a8=False, use_int8_w8a16=False, w1_bias=None, "
        "w2_bias=None, w1_scale=None, w2_scale=None, a1_scale=None, a2_scale=None, layout=blocked, alpha=None, limit=None)",
    ("lightllm_amd.fused_moe.grouped_fused_moe", "fused_experts"):
        "(hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, use_fp8_w8a8=False, use_int8_w8a16=False, "
        "w1_scale=None, w2_scale=None, a1_scale=None, a2_scale=None, w1_bias=None, w2_bias=None, layout=blocked, "
        "alpha=None, limit=None)",
}


def _sig_string(fn):
    parts = []
    for p in inspect.signature(fn).parameters.values():
        if p.default is inspect._empty:
            parts.append(p.name)
        else:
            d = p.default
            if d is torch.empty:
                d = "torch.empty"
            elif isinstance(d, torch.dtype):
                d = str(d)
            parts.append(f"{p.name}={d}")
    return "(" + ", ".join(parts) + ")"


@pytest.mark.parametrize("key", sorted(REFERENCE_SIGNATURES))
def test_python_signatures_match_the_reference(key):
    import importlib

    mod, name = key
    fn = getattr(importlib.import_module(mod), name)
    assert _sig_string(fn) == REFERENCE_SIGNATURES[key]


def test_quantization_method_surface():
    """The plug-in object exposes what LightLLM's MMWeightTpl calls (quantize_method.py:25-149, w8a8.py:418-533)."""
    from lightllm_amd.quantization import QUANTMETHODS, QuantizationMethod, WeightPack

    cls = type(QUANTMETHODS.get("fp8w8a8-b128"))
    assert issubclass(cls, QuantizationMethod)
    assert type(QUANTMETHODS.get("fp8w8a8-b128-triton", platform="cuda")) is cls
    assert QUANTMETHODS.get("fp8w8a8-b128") is not QUANTMETHODS.get("fp8w8a8-b128")   # a fresh object per lookup
    with pytest.raises(ValueError):
        QUANTMETHODS.get("no-such-method")
    with pytest.raises(ValueError):
        QUANTMETHODS.get("fp8w8a8-b128", platform="musa")
    apply_sig = list(inspect.signature(cls.apply).parameters)
    assert apply_sig == ["self", "input_tensor", "weight_pack", "out", "workspace", "use_custom_tensor_mananger", "bias"]
    for meth in ("quantize", "create_weight", "create_moe_weight", "load_weight", "load_weight_scale",
                 "load_weight_zero_point", "_create_weight", "_split_weight_pack", "_check_weight_need_quanted"):
        assert callable(getattr(cls, meth))
    m = cls()
    assert m.block_size == 128 and m.weight_scale_suffix == "weight_scale_inv" and m.has_weight_scale
    assert m.method_name.startswith("fp8w8a8-b128")
    pack = WeightPack(weight=torch.zeros((2, 4, 4)), weight_scale=torch.ones((2, 1, 1)))
    assert pack.load_ok == [False, False, True]
    sub = pack.get_expert(1)
    assert sub.weight.shape == (4, 4) and sub.weight_scale.shape == (1, 1) and sub.weight_zero_point is None
    # fused weights are split as views along dim -2, scales in units of 128 rows
    big = WeightPack(weight=torch.zeros((384, 256)), weight_scale=torch.zeros((3, 2)))
    parts = m._split_weight_pack(big, [256, 128], -2, [2, 1], -2)
    assert [p.weight.shape[0] for p in parts] == [256, 128] and [p.weight_scale.shape[0] for p in parts] == [2, 1]
    assert parts[1].weight.data_ptr() == big.weight[256:].data_ptr()


def test_operators_refuse_cpu_tensors():
    """No CPU fallback: the operators raise instead of computing on the host."""
    from lightllm_amd._lib import Mi355Error
    from lightllm_amd.quantization import per_token_group_quant_fp8

    with pytest.raises(Mi355Error):
        per_token_group_quant_fp8(torch.zeros((2, 128), dtype=torch.bfloat16), 128)


def test_shape_table_choices_on_256_compute_units():
    """The shape -> kernel table for the model linears it was measured on, planned for 256 compute units with
    room for every workspace.  A change of a rule that moves one of these shapes shows here."""
    from lightllm_amd import _lib

    lib = _lib.lib()
    T256, T128, SKINNY, GENERIC, T256x128, STREAMK, XSHARE, ROWS, CU, ROWSM = 1, 2, 3, 4, 5, 8, 9, 10, 11, 12
    expect = {
        (4096, 36864, 7168): T256, (4096, 2112, 7168): T256, (2048, 24576, 1536): T256, (256, 36864, 7168): T256,
        (512, 36864, 7168): T256,                       # launched as a full round plus a second launch for the rest
        (1, 28672, 4096): SKINNY, (8, 4096, 14336): CU, (16, 14336, 4096): CU, (1, 7168, 8192): SKINNY, (64, 4096, 14336): SKINNY, (8, 36864, 7168): SKINNY,
        (64, 128256, 4096): XSHARE, (64, 8192, 8192): SKINNY, (64, 16384, 7168): SKINNY,   # 512 / 256 workgroups
        (64, 14336, 4096): ROWS, (48, 10240, 8192): ROWS, (64, 6144, 4096): SKINNY,
        (16, 7168, 18432): CU, (32, 18432, 7168): ROWS, (32, 28672, 4096): SKINNY, (8, 7168, 18432): CU,
        (16, 36864, 4096): ROWS, (24, 36864, 7168): ROWS, (64, 28672, 4096): ROWS, (100, 7168, 18432): ROWS, (128, 24576, 1536): ROWS,
        (128, 2112, 7168): ROWS, (200, 4096, 14336): ROWS, (384, 4096, 14336): ROWS,
        (192, 36864, 7168): ROWS, (176, 28672, 4096): ROWS, (224, 28672, 4096): T128,   # narrower workgroups up to 208 rows
        (300, 28672, 4096): T256, (512, 4096, 4096): ROWSM, (2048, 4096, 4096): ROWSM, (1024, 1024, 4096): ROWSM,
        (3072, 4096, 4096): T256, (1024, 6144, 4096): T128, (1024, 4096, 8192): STREAMK,   # more than 8 row blocks, a wider N, a longer K
        (300, 36864, 7168): T256,                       # likewise: a full round and the rest
        (512, 7168, 18432): STREAMK, (2048, 4096, 14336): STREAMK, (1024, 7168, 18432): STREAMK,
        (2048, 2112, 7168): ROWSM, (512, 4096, 14336): STREAMK,     # the panel split
        (240, 7168, 18432): STREAMK, (352, 7168, 18432): STREAMK, (300, 7168, 18432): ROWS,
        (768, 2112, 7168): ROWSM, (768, 2112, 8192): T256x128, (600, 5120, 6144): T256x128, (512, 5120, 5120): ROWSM, (1024, 2112, 7168): ROWSM, (512, 4096, 7168): STREAMK,
        (384, 16384, 4096): T128, (512, 16384, 7168): STREAMK, (300, 10240, 8192): ROWS, (384, 10240, 4096): T128,
        (512, 1536, 7168): T128, (4096, 7168, 256): T128, (1024, 512, 7168): T128, (256, 4096, 4096): T128,
        (16, 256, 100): GENERIC,
    }
    got = {shape: lib.mi355_block_fp8_gemm_plan(*shape, 1 << 32, 256) for shape in expect}
    assert got == expect, {k: (got[k], expect[k]) for k in expect if got[k] != expect[k]}


_T256, _T128, _SKINNY, _GENERIC, _T256x128, _STREAMK, _XSHARE, _ROWS, _CU, _ROWSM = 1, 2, 3, 4, 5, 8, 9, 10, 11, 12


def _sweep_shapes(seed: int, count: int):
    import random

    rnd = random.Random(seed)
    model = [(28672, 4096), (4096, 14336), (36864, 7168), (7168, 18432), (2112, 7168), (24576, 1536), (6144, 4096),
             (5120, 13824), (128256, 4096), (10240, 8192), (7168, 2048), (4096, 7168), (1536, 7168), (512, 7168)]
    for _ in range(count):
        if rnd.random() < 0.6:
            n, k = rnd.choice(model)
        else:
            n, k = rnd.randrange(1, 400) * 64, rnd.randrange(1, 150) * 128
        m = rnd.choice([rnd.randrange(1, 65), rnd.randrange(65, 130), rnd.randrange(129, 385), rnd.randrange(385, 8193)])
        yield m, n, k


def test_auto_never_fails_for_want_of_a_workspace():
    """Whatever the table picks, an AUTO call without a workspace - or with the fixed scratch of the entry point
    that allocates nothing - ends in a kernel whose plan needs none (or no more than that): the ROWS128 band
    129 <= M <= 384 under a long K used to fall through to a stream-K plan that then reported MI355_EWORKSPACE."""
    from lightllm_amd import _lib

    lib = _lib.lib()
    scratch = _lib.WS_COUNTER_BYTES + (8 << 20)
    # the shapes of the report, then a seeded sweep; cus = 0 plans for the current device, whose count
    # mi355_block_fp8_gemm_workspace_bytes uses as well
    shapes = [(200, 7168, 18432), (256, 4096, 14336), (300, 4096, 14336), (384, 4096, 14336), (320, 5120, 13824),
              (128, 7168, 18432), (8, 4096, 14336), (64, 28672, 4096), (512, 7168, 18432)]
    shapes += list(_sweep_shapes(11, 4000))
    optional = (_T256, _T128, _T256x128, _XSHARE, _GENERIC, _CU, _ROWSM)   # run unsplit / one workgroup per tile without one
    for ws_bytes in (0, scratch):
        for m, n, k in shapes:
            v = lib.mi355_block_fp8_gemm_plan(m, n, k, ws_bytes, 0)
            assert v in (_T256, _T128, _SKINNY, _GENERIC, _T256x128, _STREAMK, _XSHARE, _ROWS, _CU, _ROWSM), (m, n, k, v)
            if v not in optional:
                need = lib.mi355_block_fp8_gemm_workspace_bytes(m, n, k, v)
                assert need <= ws_bytes, (m, n, k, v, need, ws_bytes)
    # with room for everything the plan is the table's own choice
    for m, n, k in shapes[:200]:
        assert lib.mi355_block_fp8_gemm_plan(m, n, k, 1 << 34, 0) == lib.mi355_block_fp8_gemm_variant(m, n, k)


@pytest.mark.parametrize("cus", [8, 64, 128, 304])
def test_shape_table_off_256_compute_units(cus):
    """The table's thresholds are all relative to the compute-unit count but were measured at 256.  On other counts
    (a partitioned device, another bin) its rules must still hold together: every shape gets a kernel that exists,
    the weight-streaming kernels keep to their row limits, and a compute-bound shape with whole rounds of
    256 x 256 tiles gets those tiles."""
    from lightllm_amd import _lib

    lib = _lib.lib()
    for m, n, k in _sweep_shapes(cus, 3000):
        for ws_bytes in (0, 1 << 34):
            v = lib.mi355_block_fp8_gemm_plan(m, n, k, ws_bytes, cus)
            assert v in (_T256, _T128, _SKINNY, _T256x128, _STREAMK, _XSHARE, _ROWS, _CU, _ROWSM), (m, n, k, v)
            if v == _ROWSM:
                assert m > 384 and k <= 7168, (m, n, k, v)
            if v == _CU:
                assert m <= 16, (m, n, k, v)
            if v in (_SKINNY, _XSHARE):
                assert m <= 64, (m, n, k, v)
            if v == _ROWS:
                assert 16 <= m <= 384, (m, n, k, v)
            if v in (_T256, _STREAMK, _T256x128, _ROWSM):
                assert m > 64, (m, n, k, v)
            if m <= 64:
                assert v in (_SKINNY, _XSHARE, _ROWS, _T128, _CU), (m, n, k, v)
    # whole rounds of 256 x 256 tiles, K long enough to be compute-bound: the ping-pong tiles on every count
    rounds = 4
    n = 256 * max(cus // 8, 1)
    assert lib.mi355_block_fp8_gemm_plan(256 * 8 * rounds, n, 7168, 1 << 34, cus) == _T256
    # decode rows stream the weights on every count
    assert lib.mi355_block_fp8_gemm_plan(1, 28672, 4096, 1 << 34, cus) == _SKINNY
    assert lib.mi355_block_fp8_gemm_plan(8, 4096, 14336, 0, cus) in (_SKINNY, _T128, _CU)

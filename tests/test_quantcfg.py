"""Per-layer quant-type resolution (host logic only, no GPU): the precedence rules of the reference's Quantcfg
(lightllm/common/quantization/__init__.py:21-130) restricted to the block-FP8 method."""
import pytest

from lightllm_amd.quantization import QUANTMETHODS, Quantcfg
from lightllm_amd.quantization.quantcfg import BLOCK_FP8
from lightllm_amd.quantization.w8a8 import FP8w8a8B128Mi355QuantizationMethod

NET = {"n_layer": 4}


def test_plain_start_argument():
    cfg = Quantcfg(NET, quant_type="fp8w8a8-b128")
    assert not cfg.quantized_weight and not cfg.static_activation and cfg.hf_quantization_config is None
    for layer in range(4):
        assert cfg.get_quant_type(layer, "gate_up_proj") == "fp8w8a8-b128"
    m = cfg.get_quant_method(2, "down_proj")
    assert isinstance(m, FP8w8a8B128Mi355QuantizationMethod) and m.hf_quantization_config is None
    assert m.method_name == QUANTMETHODS.get(BLOCK_FP8).method_name


def test_hf_block_fp8_checkpoint_selects_the_block_method():
    hf = {"quant_method": "fp8", "weight_block_size": [128, 128], "fmt": "e4m3"}
    cfg = Quantcfg({"n_layer": 2, "quantization_config": hf, "activation_scheme": "dynamic"}, quant_type="none")
    assert cfg.quantized_weight and not cfg.static_activation
    assert cfg.get_quant_type(0, "q_proj") == BLOCK_FP8
    assert cfg.get_quant_method(1, "kv_b_proj").hf_quantization_config is hf
    static = Quantcfg({"n_layer": 2, "quantization_config": hf, "activation_scheme": "static"})
    assert static.static_activation
    # fp8 without 128x128 blocks (per-tensor checkpoints) keeps the requested type
    other = Quantcfg({"n_layer": 1, "quantization_config": {"quant_method": "fp8"}}, quant_type="none")
    assert other.get_quant_type(0, "x") == "none"


def test_custom_yaml_mix_bits(tmp_path):
    path = tmp_path / "q.yaml"
    path.write_text(
        "quant_type: fp8w8a8-b128\n"
        "mix_bits:\n"
        "  - name: down_proj\n    quant_type: none\n    layer_nums: [0, 3]\n"
        "  - name: fused_moe\n    quant_type: fp8w8a8-b128-mi355\n"
    )
    cfg = Quantcfg(NET, quant_type="none", custom_cfg_path=str(path))
    assert cfg.get_quant_type(1, "gate_up_proj") == "fp8w8a8-b128"       # global type comes from the file
    assert cfg.get_quant_type(0, "down_proj") == "none" and cfg.get_quant_type(3, "down_proj") == "none"
    assert cfg.get_quant_type(1, "down_proj") == "fp8w8a8-b128"
    assert all(cfg.get_quant_type(i, "fused_moe") == BLOCK_FP8 for i in range(4))  # no layer_nums = every layer
    with pytest.raises(ValueError):
        cfg.get_quant_method(0, "down_proj")                              # "none" is not a method of this package


def test_expert_dtype_precedence(tmp_path):
    path = tmp_path / "q.yaml"
    path.write_text("quant_type: none\nmix_bits:\n  - name: fused_moe\n    quant_type: custom-moe\n    layer_nums: [1]\n")
    # model config fills only the layers the file left open
    cfg = Quantcfg({"n_layer": 3, "expert_dtype": "fp8"}, custom_cfg_path=str(path))
    assert [cfg.get_quant_type(i, "fused_moe") for i in range(3)] == [BLOCK_FP8, "custom-moe", BLOCK_FP8]
    assert cfg.get_quant_type(0, "q_proj") == "none"
    # the start argument overrides every layer, the file included
    forced = Quantcfg({"n_layer": 3}, custom_cfg_path=str(path), expert_dtype="fp8")
    assert [forced.get_quant_type(i, "fused_moe") for i in range(3)] == [BLOCK_FP8] * 3
    with pytest.raises(ValueError):
        Quantcfg({"n_layer": 1}, expert_dtype="fp4")
    with pytest.raises(ValueError):
        Quantcfg({"n_layer": 1, "expert_dtype": "int3"})


def test_unknown_layer_falls_back_to_global_type():
    cfg = Quantcfg({"n_layer": 2}, quant_type="fp8w8a8-b128-mi355")
    assert cfg.get_quant_type(17, "anything") == "fp8w8a8-b128-mi355"

"""Checkpoint -> QuantConfig parsing on the Hugging Face configs the reference's own test holds
(tests/golden/hf_configs/*.json are copies of max/tests/tests/pipelines/testdata/: data fixtures)
with the expectations of that test (max/tests/tests/pipelines/test_parse_quant_config.py:109-170,
175-440, 494-535, 630-777)."""
import copy
import json
import os
from types import SimpleNamespace

import pytest
import torch

from modular_amd.quant_config import QuantFormat, ScaleGranularity, ScaleOrigin
from modular_amd.weights_quant import parse_quant_config

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hf_configs")
FP8 = torch.float8_e4m3fn


def load(name):
    d = json.load(open(os.path.join(HERE, name)))
    cfg = SimpleNamespace(**{k: v for k, v in d.items() if k != "text_config"})
    if "text_config" in d:
        cfg.text_config = SimpleNamespace(**d["text_config"])
        cfg.text_config.quantization_config = d.get("quantization_config")
    return cfg


def meta(shape, dtype):
    return torch.empty(shape, dtype=dtype, device="meta")


def fbgemm_state(with_lm_head=True):
    sd = {"layers.0.mlp.down_proj.weight_scale": meta((1, 1), FP8)}
    if with_lm_head:
        sd["lm_head.weight"] = meta((1, 1), torch.bfloat16)
    return sd


@pytest.mark.parametrize("name", ["llama_3_1_405b_instruct_fp8.json", "llama_3_1_405b_fp8.json"])
def test_fbgemm(name):
    hf = load(name)
    qc = parse_quant_config(hf, fbgemm_state(), FP8)
    assert qc.format == QuantFormat.FBGEMM_FP8
    assert qc.input_scale.granularity == ScaleGranularity.COLWISE and qc.input_scale.origin == ScaleOrigin.DYNAMIC
    assert qc.input_scale.dtype == FP8 and qc.input_scale.activation_scale_ub == hf.quantization_config["activation_scale_ub"]
    assert qc.weight_scale.granularity == ScaleGranularity.ROWWISE and qc.weight_scale.dtype == FP8
    assert qc.embedding_output_dtype == torch.bfloat16
    # layer 0's MLP and attention are in modules_to_not_convert
    assert qc.mlp_quantized_layers == set(range(1, hf.num_hidden_layers))
    assert qc.attn_quantized_layers == set(range(1, hf.num_hidden_layers))


def test_wrong_dtype_and_missing_config():
    hf = load("llama_3_1_405b_instruct_fp8.json")
    assert parse_quant_config(hf, {}, torch.bfloat16) is None
    hf2 = copy.deepcopy(hf)
    del hf2.quantization_config
    with pytest.raises(ValueError, match="expected a `quantization_config` field"):
        parse_quant_config(hf2, {}, FP8)
    hf3 = copy.deepcopy(hf)
    hf3.quantization_config["quant_method"] = "unsupported_method"
    with pytest.raises(ValueError, match="Unrecognized quantization config"):
        parse_quant_config(hf3, fbgemm_state(), FP8)


def test_fbgemm_scale_errors():
    hf = load("llama_3_1_405b_instruct_fp8.json")
    with pytest.raises(ValueError, match="could not find weight scale dtype"):
        parse_quant_config(hf, {"lm_head.weight": meta((1, 1), torch.bfloat16)}, FP8)
    sd = fbgemm_state()
    sd["layers.1.mlp.down_proj.weight_scale"] = meta((1, 1), torch.float32)
    with pytest.raises(ValueError, match="only row-wise weight quantization with uniform weight scale"):
        parse_quant_config(hf, sd, FP8)
    sd = {"layers.0.mlp.down_proj.weight_scale": meta((1, 2), FP8)}
    with pytest.raises(ValueError, match="only row-wise weight quantization"):
        parse_quant_config(hf, sd, FP8)


def test_partial_quantisation_errors():
    hf = load("llama_3_1_405b_instruct_fp8.json")
    hf.quantization_config["modules_to_not_convert"] = ["model.layers.1.mlp.gate_proj"]
    with pytest.raises(ValueError, match="uniform quantization for MLPs"):
        parse_quant_config(hf, fbgemm_state(), FP8)
    hf.quantization_config["modules_to_not_convert"] = ["model.layers.1.self_attn.q_proj"]
    with pytest.raises(ValueError, match="uniform quantization for attention"):
        parse_quant_config(hf, fbgemm_state(), FP8)
    hf.quantization_config["modules_to_not_convert"] = ["lm_head"]
    with pytest.raises(ValueError, match="cannot determine original type from checkpoint"):
        parse_quant_config(hf, fbgemm_state(with_lm_head=False), FP8)


def gemma_state():
    return {
        "language_model.layers.0.mlp.down_proj.input_scale": meta((1, 1), torch.float32),
        "language_model.layers.0.mlp.down_proj.weight_scale": meta((1, 1), torch.float32),
        "language_model.embed_tokens.weight": meta((1, 1), torch.bfloat16),
        "language_model.lm_head.weight": meta((1, 1), FP8),
    }


def test_gemma3_compressed_tensors():
    hf = load("gemma-3-4b-it-FP8-dynamic.json")
    qc = parse_quant_config(hf.text_config, gemma_state(), FP8, state_dict_name_prefix="language_model.",
                            ignored_modules_prefix="language_model.")
    assert qc.format == QuantFormat.COMPRESSED_TENSORS_FP8
    assert qc.input_scale.granularity == ScaleGranularity.COLWISE and qc.input_scale.origin == ScaleOrigin.DYNAMIC
    assert qc.input_scale.dtype == torch.float32
    assert qc.weight_scale.granularity == ScaleGranularity.ROWWISE and qc.weight_scale.dtype == torch.float32
    assert qc.embedding_output_dtype == torch.bfloat16          # embed_tokens takes priority over lm_head
    layers = set(range(hf.text_config.num_hidden_layers))
    assert qc.mlp_quantized_layers == layers and qc.attn_quantized_layers == layers
    # without embed_tokens the lm_head dtype is used
    sd = gemma_state()
    del sd["language_model.embed_tokens.weight"]
    assert parse_quant_config(hf.text_config, sd, FP8, "language_model.", "language_model.").embedding_output_dtype == FP8


def test_compressed_tensors_errors():
    hf = load("gemma-3-4b-it-FP8-dynamic.json").text_config
    for field, key, val, msg in [("input_activations", "strategy", "group", "unsupported FP8 input activation strategy"),
                                 ("weights", "strategy", "group", "unsupported FP8 weight strategy"),
                                 ("weights", "dynamic", True, "dynamic weight scaling is not supported")]:
        bad = copy.deepcopy(hf)
        bad.quantization_config["config_groups"]["group_0"][field][key] = val
        with pytest.raises(ValueError, match=msg):
            parse_quant_config(bad, gemma_state(), FP8, "language_model.", "language_model.")


def fp8_hf(**quant):
    return SimpleNamespace(num_hidden_layers=4, quantization_config={"quant_method": "fp8", **quant})


def test_blockscaled_and_tensorwise_fp8():
    sd = {"layers.0.mlp.down_proj.weight_scale_inv": meta((2, 2), torch.float32), "layers.0.mlp.down_proj.bias": meta((4,), torch.float16)}
    qc = parse_quant_config(fp8_hf(activation_scheme="dynamic", weight_block_size=[128, 128]), sd, FP8)
    assert qc.format == QuantFormat.BLOCKSCALED_FP8 and qc.bias_dtype == torch.float16
    assert qc.input_scale.block_size == (1, 128) and qc.weight_scale.block_size == (128, 128)
    assert qc.input_scale.dtype == torch.float32 and qc.mlp_quantized_layers == {0, 1, 2, 3} == qc.attn_quantized_layers
    assert qc.scales_granularity_mnk == (1, 128, 128)
    with pytest.raises(ValueError, match="weight_block_size must be"):
        parse_quant_config(fp8_hf(activation_scheme="dynamic", weight_block_size=[64, 64]), sd, FP8)
    with pytest.raises(ValueError, match="activation_scheme must be dynamic"):
        parse_quant_config(fp8_hf(activation_scheme="static", weight_block_size=[128, 128]), sd, FP8)
    for scheme, origin in (("dynamic", ScaleOrigin.DYNAMIC), ("static", ScaleOrigin.STATIC)):
        qc = parse_quant_config(fp8_hf(activation_scheme=scheme), {"layers.0.mlp.down_proj.weight_scale": meta((), torch.float32)}, FP8)
        assert qc.input_scale.granularity == ScaleGranularity.TENSOR == qc.weight_scale.granularity
        assert qc.input_scale.origin == origin and qc.is_static == (scheme == "static")
    with pytest.raises(ValueError, match="Unsupported activation_scheme"):
        parse_quant_config(fp8_hf(activation_scheme="other"), sd, FP8)


def test_bias_dtype_rules():
    hf = load("llama_3_1_405b_instruct_fp8.json")
    sd = fbgemm_state()
    assert parse_quant_config(hf, sd, FP8).bias_dtype is None
    sd["layers.0.self_attn.q_proj.bias"] = meta((4,), torch.float32)
    assert parse_quant_config(hf, sd, FP8).bias_dtype == torch.float32
    sd["layers.0.self_attn.k_proj.bias"] = meta((4,), torch.bfloat16)
    with pytest.raises(ValueError, match="Inconsistent bias dtypes"):
        parse_quant_config(hf, sd, FP8)

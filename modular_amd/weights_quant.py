"""Checkpoint -> QuantConfig for the FP8 formats: which scaling a Hugging Face checkpoint uses,
read from its `quantization_config` and the dtypes / shapes of its scale tensors.  Mirrors
`parse_quant_config` for dtype float8_e4m3fn (max/python/max/pipelines/weights/quant.py:1135-1218,
dispatch :699-755) and its FP8 parsers: compressed-tensors (:288-397), fbgemm_fp8 (:451-505),
tensor-wise fp8 (:508-585) and block-scaled fp8 (:588-650).  The FP4 / MX formats are other
operators and are rejected here.

`huggingface_config` is any object with the config's attributes (`quantization_config` mapping,
`num_hidden_layers`, optionally `text_config`); `state_dict` maps weight names to anything with
`.dtype` and `.shape` (tensors, or meta tensors)."""
from __future__ import annotations

from typing import Any, Mapping

import torch

from .quant_config import (InputScaleSpec, QuantConfig, QuantFormat, ScaleGranularity, ScaleOrigin,
                           WeightScaleSpec)

_FP8 = torch.float8_e4m3fn
_KNOWN_METHODS = ("compressed-tensors", "fbgemm_fp8", "fp8", "gptq", "modelopt", "mxfp4", "mxfp6", "mxfp8", "quark")


def _get_num_hidden_layers(huggingface_config: Any) -> int:
    """Multi-modal configs keep the language model's depth in text_config (quant.py:85-94)."""
    if hasattr(huggingface_config, "text_config"):
        return huggingface_config.text_config.num_hidden_layers
    return huggingface_config.num_hidden_layers


def _quantized_layers_and_embedding_dtype(huggingface_config: Any, ignored_modules: set[str],
                                          state_dict: Mapping[str, Any], state_dict_name_prefix: str = "",
                                          ignored_modules_prefix: str = "model."):
    """Which layers have their MLP / attention projections in float8, and the dtype the embedding
    produces (quant.py:97-166)."""
    mlp_layers: set[int] = set()
    attn_layers: set[int] = set()
    for i in range(_get_num_hidden_layers(huggingface_config)):
        mlp = [f"{ignored_modules_prefix}layers.{i}.mlp.{proj}" in ignored_modules
               for proj in ("gate_proj", "up_proj", "down_proj")]
        if not any(mlp):
            mlp_layers.add(i)
        elif not all(mlp):
            raise ValueError("float8 quantization currently assumes uniform quantization for MLPs")
        attn = [f"{ignored_modules_prefix}layers.{i}.self_attn.{proj}" in ignored_modules
                for proj in ("q_proj", "k_proj", "v_proj", "o_proj")]
        if not any(attn):
            attn_layers.add(i)
        elif not all(attn):
            raise ValueError(
                "float8 quantization currently assumes uniform quantization for attention QKV and output projections")
    if f"{state_dict_name_prefix}embed_tokens.weight" in state_dict:
        embedding_dtype = state_dict[f"{state_dict_name_prefix}embed_tokens.weight"].dtype
    elif f"{state_dict_name_prefix}lm_head.weight" in state_dict:
        embedding_dtype = state_dict[f"{state_dict_name_prefix}lm_head.weight"].dtype
    elif f"{state_dict_name_prefix}lm_head" in ignored_modules:
        raise ValueError("cannot determine original type from checkpoint")
    else:
        embedding_dtype = _FP8
    return mlp_layers, attn_layers, embedding_dtype


def _weight_scale_dtype(state_dict: Mapping[str, Any]) -> torch.dtype:
    """fbgemm: every weight scale is row-wise [N, 1] and of one dtype (quant.py:400-428)."""
    found = None
    for name, weight in state_dict.items():
        if "weight_scale" not in name:
            continue
        if len(weight.shape) != 2 or weight.shape[1] != 1 or (found and weight.dtype != found):
            raise ValueError(
                "only row-wise weight quantization with uniform weight scale dtype is supported for FBGEMM FP8")
        found = weight.dtype
    if not found:
        raise ValueError("could not find weight scale dtype for FBGEMM FP8 quantized weights")
    return found


def _any_weight_scale_dtype(state_dict: Mapping[str, Any], what: str) -> torch.dtype:
    found = None
    for name, weight in state_dict.items():
        if "weight_scale" in name:
            found = weight.dtype
    if not found:
        raise ValueError(f"could not find weight scale dtype for {what}")
    return found


def _bias_dtype(state_dict: Mapping[str, Any]) -> torch.dtype | None:
    """dtype shared by every `.bias` weight, None without biases (quant.py:431-448)."""
    found = None
    for name, weight in state_dict.items():
        if name.endswith(".bias"):
            if found is None:
                found = weight.dtype
            elif weight.dtype != found:
                raise ValueError(f"Inconsistent bias dtypes found: {found} vs {weight.dtype} in {name}")
    return found


_STRATEGY = {"tensor": ScaleGranularity.TENSOR, "channel": ScaleGranularity.ROWWISE, "token": ScaleGranularity.COLWISE}


def _parse_compressed_tensors(huggingface_config, state_dict, dtype, state_dict_name_prefix, ignored_modules_prefix):
    cfg = huggingface_config.quantization_config
    group = cfg["config_groups"]["group_0"]          # only group_0 matters for now
    acts, weights = group["input_activations"], group["weights"]
    origin = ScaleOrigin.DYNAMIC if acts["dynamic"] else ScaleOrigin.STATIC
    if acts["strategy"] not in _STRATEGY:
        raise ValueError(f"unsupported FP8 input activation strategy: {acts['strategy']}")
    input_scale_name = f"{state_dict_name_prefix}layers.0.mlp.down_proj.input_scale"
    in_dtype = state_dict[input_scale_name].dtype if input_scale_name in state_dict else dtype
    input_spec = InputScaleSpec(_STRATEGY[acts["strategy"]], origin, in_dtype, activation_scale_ub=None)
    if weights["strategy"] not in _STRATEGY:
        raise ValueError(f"unsupported FP8 weight strategy: {weights['strategy']}")
    if weights["dynamic"]:
        raise ValueError("dynamic weight scaling is not supported for compressed-tensors FP8 method")
    weight_scale = state_dict[f"{state_dict_name_prefix}layers.0.mlp.down_proj.weight_scale"]
    weight_spec = WeightScaleSpec(_STRATEGY[weights["strategy"]], weight_scale.dtype)
    mlp, attn, emb = _quantized_layers_and_embedding_dtype(huggingface_config, set(cfg.get("ignore", [])), state_dict,
                                                           state_dict_name_prefix, ignored_modules_prefix)
    return QuantConfig(input_scale=input_spec, weight_scale=weight_spec, mlp_quantized_layers=mlp,
                       attn_quantized_layers=attn, embedding_output_dtype=emb, bias_dtype=_bias_dtype(state_dict),
                       format=QuantFormat.COMPRESSED_TENSORS_FP8)


def _parse_fbgemm(huggingface_config, state_dict, dtype):
    cfg = huggingface_config.quantization_config
    # input: dynamic, per token; weight: static, per output channel
    input_spec = InputScaleSpec(ScaleGranularity.COLWISE, ScaleOrigin.DYNAMIC, dtype,
                                activation_scale_ub=cfg.get("activation_scale_ub"))
    weight_spec = WeightScaleSpec(ScaleGranularity.ROWWISE, _weight_scale_dtype(state_dict))
    mlp, attn, emb = _quantized_layers_and_embedding_dtype(huggingface_config,
                                                           set(cfg.get("modules_to_not_convert", [])), state_dict)
    return QuantConfig(input_scale=input_spec, weight_scale=weight_spec, mlp_quantized_layers=mlp,
                       attn_quantized_layers=attn, embedding_output_dtype=emb, bias_dtype=_bias_dtype(state_dict),
                       format=QuantFormat.FBGEMM_FP8)


def _parse_tensorwise(huggingface_config, state_dict, dtype):
    cfg = huggingface_config.quantization_config
    scheme = cfg.get("activation_scheme")
    if scheme == "dynamic":
        origin = ScaleOrigin.DYNAMIC
    elif scheme == "static":
        origin = ScaleOrigin.STATIC
    else:
        raise ValueError(f"Unsupported activation_scheme for tensorwise FP8: '{scheme}'. Expected 'dynamic' or 'static'.")
    sdt = _any_weight_scale_dtype(state_dict, "tensorwise FP8 quantized weights")
    mlp, attn, emb = _quantized_layers_and_embedding_dtype(huggingface_config,
                                                           set(cfg.get("modules_to_not_convert", [])), state_dict)
    return QuantConfig(input_scale=InputScaleSpec(ScaleGranularity.TENSOR, origin, sdt),
                       weight_scale=WeightScaleSpec(ScaleGranularity.TENSOR, sdt), mlp_quantized_layers=mlp,
                       attn_quantized_layers=attn, embedding_output_dtype=emb, bias_dtype=_bias_dtype(state_dict),
                       format=QuantFormat.FBGEMM_FP8)   # (the reference labels this flavour FBGEMM_FP8 too, quant.py:584)


def _parse_blockscaled(huggingface_config, state_dict, dtype):
    cfg = huggingface_config.quantization_config
    if "activation_scheme" not in cfg:
        raise ValueError("activation_scheme must be specified")
    if cfg["activation_scheme"] != "dynamic":
        raise ValueError("activation_scheme must be dynamic")
    if "weight_block_size" not in cfg:
        raise ValueError("weight_block_size must be specified")
    if list(cfg["weight_block_size"]) != [128, 128]:
        raise ValueError("weight_block_size must be [128, 128]")
    sdt = _any_weight_scale_dtype(state_dict, "FP8 quantized weights")
    all_layers = set(range(_get_num_hidden_layers(huggingface_config)))   # every linear is FP8 in this format
    return QuantConfig(
        input_scale=InputScaleSpec(ScaleGranularity.BLOCK, ScaleOrigin.DYNAMIC, sdt, block_size=(1, 128)),
        weight_scale=WeightScaleSpec(ScaleGranularity.BLOCK, sdt, block_size=(128, 128)),
        mlp_quantized_layers=all_layers, attn_quantized_layers=set(all_layers),
        embedding_output_dtype=torch.bfloat16, bias_dtype=_bias_dtype(state_dict), format=QuantFormat.BLOCKSCALED_FP8)


def parse_quant_config(huggingface_config: Any, state_dict: Mapping[str, Any], dtype: torch.dtype,
                       state_dict_name_prefix: str = "", ignored_modules_prefix: str = "model.") -> QuantConfig | None:
    """QuantConfig of a float8 checkpoint; None when `dtype` is not float8_e4m3fn."""
    cfg = getattr(huggingface_config, "quantization_config", None)
    if cfg:
        method = cfg.get("quant_method", "")
        if method and method not in _KNOWN_METHODS:
            raise ValueError("Unrecognized quantization config: the `quant_method` "
                             f"field ({method!r}) is provided but not recognized.")
    if dtype != _FP8:
        return None
    if not cfg:
        raise ValueError("expected a `quantization_config` field in Hugging Face config when the dtype is float8")
    method = cfg.get("quant_method")
    if method == "compressed-tensors":
        return _parse_compressed_tensors(huggingface_config, state_dict, dtype, state_dict_name_prefix,
                                         ignored_modules_prefix)
    if method == "fbgemm_fp8":
        return _parse_fbgemm(huggingface_config, state_dict, dtype)
    if method == "fp8":
        if cfg.get("weight_block_size"):
            return _parse_blockscaled(huggingface_config, state_dict, dtype)
        return _parse_tensorwise(huggingface_config, state_dict, dtype)   # tensor-wise scaling is the fallback
    raise ValueError("FP8 dtype specified, but an unsupported or incompatible 'quantization_config' "
                     f"was found. Quant method: '{method}'. "
                     "Supported methods are 'compressed-tensors', 'fbgemm_fp8', and 'fp8'.")

"""Model registry: config.json's architecture name -> (configuration reader, model class, checkpoint adapter).

`load_model(dir)` is how the command line (generate, trace) and the benchmark get a model: it reads config.json, picks the entry,
streams model.safetensors to the device (loader.py) and builds the modules."""
from __future__ import annotations

import json
import os

import torch

from .config import ExLlamaV2Config, LayeredConfig

ARCHITECTURES = {}


def register(name: str, read_config, build):
    """read_config(dict) -> config object; build(config, tensors, device, dtype, ext) -> loaded model"""
    ARCHITECTURES[name] = (read_config, build)


def _build_layered(cfg, tensors, device, dtype, ext):
    from .layered import LayeredModel
    return LayeredModel(cfg, device=device, dtype=dtype or torch.bfloat16, ext=ext).load(tensors)


def _read_llama(d: dict) -> ExLlamaV2Config:
    heads = int(d["num_attention_heads"])
    return ExLlamaV2Config(hidden_size=int(d["hidden_size"]), intermediate_size=int(d["intermediate_size"]),
                           num_hidden_layers=int(d["num_hidden_layers"]), num_attention_heads=heads,
                           num_key_value_heads=int(d.get("num_key_value_heads", heads)),
                           head_dim=int(d.get("head_dim") or int(d["hidden_size"]) // heads), vocab_size=int(d["vocab_size"]),
                           max_seq_len=int(d.get("max_position_embeddings", 4096)), norm_eps=float(d.get("rms_norm_eps", 1e-5)),
                           rotary_embedding_base=float(d.get("rope_theta", 10000.0)),
                           num_experts=int(d.get("num_local_experts", 0)), num_experts_per_token=int(d.get("num_experts_per_tok", 2)),
                           arch="mixtral" if d.get("num_local_experts") else "llama")


def _build_quantized(cfg, tensors, device, dtype, ext):
    """EXL2 / GPTQ checkpoints of the Llama family: `<key>.q_weight` ... tensors grouped per linear, `<key>.weight` plain"""
    from .model import ExLlamaV2
    if dtype not in (None, torch.float16):
        raise RuntimeError("quantized Llama-family models run in float16")
    ck = {}
    for name, t in tensors.items():
        key, _, leaf = name.rpartition(".")
        if leaf == "weight":
            ck[key] = t
        else:
            ck.setdefault(key, {})[leaf] = t
    for key, v in ck.items():
        if isinstance(v, dict) and "q_invperm" in v and "q_perm" not in v:
            v["q_perm"] = torch.argsort(v["q_invperm"]).to(torch.int32)
    return ExLlamaV2(cfg, device=device, ext=ext).load(ck)


register("Benolix", LayeredConfig.from_dict, _build_layered)
register("Tibalorn", LayeredConfig.from_dict_prenorm, _build_layered)
register("Negilorn", LayeredConfig.from_dict_prerms_shift, _build_layered)
register("Kilurax", LayeredConfig.from_dict_sandwich, _build_layered)
register("LlamaForCausalLM", _read_llama, _build_quantized)
register("MixtralForCausalLM", _read_llama, _build_quantized)


def read_config(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        d = json.load(f)
    name = d.get("architecture") or (d.get("architectures") or [None])[0]
    if name not in ARCHITECTURES:
        raise RuntimeError(f"config.json names architecture {name!r}; known: {sorted(ARCHITECTURES)}")
    return name, ARCHITECTURES[name][0](d)


def needs_whole_library(model_dir: str) -> bool:
    """False for architectures served by the dense-model subset of the library alone (build.py: DENSE_SOURCES)"""
    name, _cfg = read_config(model_dir)
    return ARCHITECTURES[name][1] is not _build_layered


def load_model(model_dir: str, device="cuda:0", dtype=None, ext=None):
    from .ext import ext_c
    from .loader import load_tensors
    ext = ext or ext_c
    name, cfg = read_config(model_dir)
    tensors = load_tensors(os.path.join(model_dir, "model.safetensors"), device, ext)
    return ARCHITECTURES[name][1](cfg, tensors, device, dtype, ext)

"""Weights into a model: safetensors files (reference: tinyvllm/utils/loader.py:11-30), bf16 or
quantised offline by ``quantize_checkpoint``, or a seeded random initialisation for the benchmark /
parity configurations."""
from __future__ import annotations

import os
from glob import glob

import torch
from torch import nn


def default_weight_loader(param: nn.Parameter, loaded_weight: torch.Tensor):
    param.data.copy_(loaded_weight)


def load_model(model: nn.Module, path: str):
    """Copy every tensor of ``path/*.safetensors`` into the model; q/k/v and gate/up projections are
    routed into the packed parameters through ``packed_modules_mapping`` and per-parameter loaders."""
    from safetensors import safe_open
    packed = getattr(model, "packed_modules_mapping", {})
    for file in sorted(glob(os.path.join(path, "*.safetensors"))):
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                load_tensor(model, packed, name, f.get_tensor(name))
    finish_load(model)


def load_tensor(model: nn.Module, packed: dict, name: str, tensor: torch.Tensor):
    kind = name.rsplit(".", 1)[-1]
    if kind in ("qweight", "qscale"):          # a checkpoint written by quantize_checkpoint
        module_name, shard_id = name.rsplit(".", 1)[0], None
        for key, (target, sid) in packed.items():
            if key in module_name:
                module_name, shard_id = module_name.replace(key, target), sid
                break
        model.get_submodule(module_name).load_quantized_shard(kind, tensor, shard_id)
        return
    stem = name.rsplit(".", 2)[-2] if name.count(".") >= 1 else name
    if stem in {target for target, _ in packed.values()}:
        # already packed (``qkv_proj``, ``gate_up_proj``: a state dict taken from this model): whole copy
        default_weight_loader(model.get_parameter(name), tensor)
        return
    for key, (target, shard_id) in packed.items():
        if key in name:
            param = model.get_parameter(name.replace(key, target))
            param.weight_loader(param, tensor, shard_id)
            return
    param = model.get_parameter(name)
    getattr(param, "weight_loader", default_weight_loader)(param, tensor)


def finish_load(model: nn.Module):
    for m in model.modules():
        if getattr(m, "pending_quantized", False):
            m.finish_quantized_load()


QUANTIZED_SUFFIXES = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


def quantize_checkpoint(src: str, dst: str):
    """Offline weight-only int8: every ``*_proj.weight`` of ``src/*.safetensors`` becomes ``*.qweight`` (int8,
    same ``[out, in]`` layout) plus ``*.qscale`` (fp32 ``[out]``, ``max|row| / 127``) in ``dst``; every other
    tensor is copied.  Rows are independent, so the unpacked q/k/v and gate/up tensors quantise to exactly
    the rows that quantising the packed weight gives.  Streams one file at a time."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    from ..layers.linear import quantize_per_channel
    os.makedirs(dst, exist_ok=True)
    for file in sorted(glob(os.path.join(src, "*.safetensors"))):
        out = {}
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                t = f.get_tensor(name)
                stem = name[:-len(".weight")] if name.endswith(".weight") else None
                if stem is not None and stem.rsplit(".", 1)[-1] in QUANTIZED_SUFFIXES and t.dim() == 2:
                    wq, scale = quantize_per_channel(t)
                    out[stem + ".qweight"], out[stem + ".qscale"] = wq, scale
                else:
                    out[name] = t.contiguous()
        save_file(out, os.path.join(dst, os.path.basename(file)))
    for extra in ("config.json",):
        p = os.path.join(src, extra)
        if os.path.exists(p):
            import shutil
            shutil.copy(p, os.path.join(dst, extra))


def load_state_dict(model: nn.Module, state: dict):
    """Same routing as ``load_model`` for an in-memory ``{hf_name: tensor}`` dict."""
    packed = getattr(model, "packed_modules_mapping", {})
    for name, tensor in state.items():
        load_tensor(model, packed, name, tensor)
    finish_load(model)


def random_init_(model: nn.Module, seed: int = 0, std: float = 0.02, device_fill: bool = False):
    """Random weights in ``named_parameters()`` order: fp32 N(0, std) rounded to the parameter dtype;
    RMSNorm weights stay 1; a tied LM head shares the embedding.

    ``device_fill=False`` draws on the CPU from ``torch.Generator().manual_seed(seed)`` so that a CPU
    restatement can hold identical weights (parity configuration); ``device_fill=True`` draws on the
    GPU (8B / 32B shapes, where only the distribution matters).
    """
    gen = None if device_fill else torch.Generator().manual_seed(seed)
    if device_fill:
        torch.manual_seed(seed)
    cfg = getattr(model, "config", None)
    tied = cfg is not None and getattr(cfg, "tie_word_embeddings", False)
    for name, p in model.named_parameters():
        if tied and name == "lm_head.weight":
            continue                                   # shares the embedding's storage
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            p.data.fill_(1.0)
            continue
        if device_fill:
            p.data.normal_(0.0, std)
        else:
            w = torch.empty(p.shape, dtype=torch.float32).normal_(0.0, std, generator=gen)
            p.data.copy_(w.to(p.dtype))
    if tied:
        model.lm_head.weight.data = model.model.embed_tokens.weight.data
    return model

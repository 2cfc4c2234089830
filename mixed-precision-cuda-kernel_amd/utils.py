"""Model surgery and the on-disk format of packed models.

Counterpart of the reference's utils.py:66-149 without its HF-transformers / accelerate
scaffolding: `make_quant` swaps fake-quant training linears for packed ones, `pack_model` fills
them, `save_quantized` writes `pytorch_model-{w_bits}bit-{group_size}g.bin` (a plain state dict)
next to `config.json`, and `from_quantized` builds this package's decoder from such a directory.
The file name, the state-dict key names and the buffer dtypes/shapes are the reference's, so a
directory written by the reference's `save_quantized` for a LLaMA model loads here unchanged
(its pickle is read with `weights_only=True`).
"""
from __future__ import annotations

import dataclasses
import json
import os

import torch
import torch.nn as nn

from llama.cherry_linear import QuantLinear as QuantLinearForTraining
from llama.qlinear import QuantLinear


def get_device(obj):
    if isinstance(obj, torch.Tensor):
        return obj.device
    return next(obj.parameters()).device


def make_quant(module: nn.Module, name: str = "") -> dict:
    """Replace every fake-quant training linear below `module` by an empty packed QuantLinear of
    the same geometry, in place; returns {qualified name: the training module it replaced}.
    utils.py:66-92."""
    replaced = {}
    if isinstance(module, QuantLinearForTraining):
        return replaced
    for attr, child in list(module.named_children()):
        full = f"{name}.{attr}" if name else attr
        if isinstance(child, QuantLinearForTraining):
            packed = QuantLinear(child.w_bits, child.group_size, child.quantizer, child.cherry_fraction,
                                 child.in_features, child.out_features, child.bias)
            setattr(module, attr, packed.to(get_device(child)))
            replaced[full] = child
        else:
            replaced.update(make_quant(child, full))
    return replaced


def pack_model(model: nn.Module) -> None:
    """make_quant, then pack every new module from the training module it replaced.  utils.py:95-101."""
    replaced = make_quant(model)
    for name, module in model.named_modules():
        if isinstance(module, QuantLinear) and name in replaced:
            module.pack(replaced[name])


def _checkpoint_name(w_bits, group_size) -> str:
    return f"pytorch_model-{w_bits}bit-{group_size}g.bin"


def _config_dict(model) -> dict:
    cfg = getattr(model, "config", None) or getattr(model, "cfg", None)
    if cfg is None:
        return {}
    if dataclasses.is_dataclass(cfg):
        return dataclasses.asdict(cfg)
    if hasattr(cfg, "to_dict"):
        return cfg.to_dict()
    return dict(vars(cfg))


def save_quantized(model: nn.Module, save_dir: str) -> str:
    """Write the packed model: state dict (CPU tensors) + config.json.  utils.py:104-122.
    A model with `reference_state_dict()` (this package's decoder) is written under the
    reference's LLaMA key names.  Returns the checkpoint path."""
    w_bits = group_size = None
    for module in model.modules():
        if isinstance(module, QuantLinear):
            w_bits, group_size = module.w_bits, module.group_size
            break
    if w_bits is None:
        raise ValueError("save_quantized: the model holds no packed QuantLinear")
    sd = model.reference_state_dict() if hasattr(model, "reference_state_dict") else model.state_dict()
    sd = {k: v.detach().cpu().contiguous() for k, v in sd.items()}
    os.makedirs(save_dir, exist_ok=True)
    path = os.path.join(save_dir, _checkpoint_name(w_bits, group_size))
    torch.save(sd, path)
    cfg = getattr(model, "config", None)
    if cfg is not None and hasattr(cfg, "save_pretrained"):
        cfg.save_pretrained(save_dir)
    else:
        d = _config_dict(model)
        d.setdefault("w_bits", w_bits)
        d.setdefault("group_size", group_size)
        d.setdefault("model_type", "llama")
        with open(os.path.join(save_dir, "config.json"), "w") as f:
            json.dump(d, f, indent=2, sort_keys=True)
    gen = getattr(model, "generation_config", None)
    if gen is not None and hasattr(gen, "save_pretrained"):
        gen.save_pretrained(save_dir)
    return path


def from_quantized(model_name_or_path: str, model_type: str = "llama", torch_dtype=None, device_map=None,
                   prepack: bool = True, release_reference: bool = False):
    """Build this package's decoder from a directory written by `save_quantized` (here or by the
    reference, utils.py:125-149) and load the packed weights.  `device_map` may be None / "cuda" /
    a device; the whole model lives on that one device.  `prepack` (default) also repacks, once,
    the layers whose shape the library recommends it for into the weight streams the batch-1
    kernels read fastest (CherryLlamaDecoder.prepack); the checkpoint-layout buffers stay unless
    `release_reference` frees them (one copy of the weights on the device: a decode deployment)."""
    if model_type != "llama":
        raise NotImplementedError(f"model_type {model_type!r}")
    if torch_dtype not in (None, torch.float16):
        raise NotImplementedError("packed models are fp16")
    import cherryq_decoder as cd
    with open(os.path.join(model_name_or_path, "config.json")) as f:
        raw = json.load(f)
    if raw.get("cherryq") is False:
        raise ValueError("config.json says cherryq=false: not a CherryQ checkpoint")
    fields = {f.name for f in dataclasses.fields(cd.DecoderConfig)}
    kwargs = {k: raw[k] for k in fields if k in raw and raw[k] is not None}
    if "num_key_value_heads" not in kwargs and "num_attention_heads" in kwargs:
        kwargs["num_key_value_heads"] = kwargs["num_attention_heads"]
    cfg = cd.DecoderConfig(**kwargs)
    if cfg.group_size == -1:
        raise NotImplementedError("group_size -1 (one group per row) differs per layer; not supported by the decoder")
    device = "cuda" if device_map in (None, "auto") else device_map
    if isinstance(device, dict):
        device = next(iter(device.values()))
    model = cd.CherryLlamaDecoder(cfg, seed=0, device=device)
    path = os.path.normpath(os.path.join(model_name_or_path, _checkpoint_name(cfg.w_bits, cfg.group_size)))
    sd = torch.load(path, map_location="cpu", weights_only=True)
    model.load_reference_state_dict(sd)
    if prepack and model.device_.type == "cuda":
        model.prepack(release_reference=release_reference)
    return model

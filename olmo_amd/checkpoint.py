"""Checkpoint formats either side of the forward path: AutoGPTQ int4 directories, unsharded OLMo
checkpoints, and the OLMo <-> HF ``Olmo2ForCausalLM`` tensor layouts.

Host-side, one-time code (file formats and name mapping); the tensors end up in the modules of
``olmo_amd.model`` / ``olmo_amd.qlinear``, whose ``post_init`` builds the kernel layouts.

* ``BaseQuantizeConfig``, ``save_quantized``, ``from_quantized`` follow
  ``AGQ/auto_gptq/modeling/_base.py:43-120,534-603,784-918`` (AGQ =
  ``inference/compression/dependencies/AutoGPTQ``): ``quantize_config.json``, ``config.json`` and
  ``gptq_model-{bits}bit-{group_size}g.{safetensors,bin}`` whose tensor names are the HF module
  tree's (``model.transformer.blocks.{i}.att_proj.qweight`` ...).
* ``make_state_dict_compatible`` / ``load_unsharded_checkpoint`` follow ``olmo/model.py:1730-1764,1786-1878``
  (``config.yaml`` + ``model.pt``).
* ``olmo_to_hf_olmo2_state_dict`` / ``hf_olmo2_to_olmo_state_dict`` follow
  ``scripts/convert_olmo2_to_hf.py:110-163`` (split orders: q | k | v and up | gate).

Files are read with loaders that execute nothing from the file (safetensors,
``torch.load(weights_only=True)``, ``yaml.safe_load``, json).
"""

from __future__ import annotations

import json
import os
import re
from dataclasses import dataclass, field, fields
from fnmatch import fnmatch
from typing import Any, Dict, Iterator, Optional, Tuple

import torch

from .config import ModelConfig

__all__ = [
    "BaseQuantizeConfig", "save_quantized", "from_quantized", "make_state_dict_compatible",
    "load_unsharded_checkpoint", "olmo_to_hf_olmo2_state_dict", "hf_olmo2_to_olmo_state_dict",
]


# ---------------------------------------------------------------------------------------------
# AutoGPTQ directories
# ---------------------------------------------------------------------------------------------
@dataclass
class BaseQuantizeConfig:
    """``BaseQuantizeConfig`` of ``AGQ/auto_gptq/modeling/_base.py:43-120``: same fields, defaults,
    validation messages and ``quantize_config.json`` layout."""

    bits: int = field(default=4, metadata={"choices": [2, 3, 4, 8]})
    group_size: int = field(default=-1)
    damp_percent: float = field(default=0.01)
    desc_act: bool = field(default=True)
    static_groups: bool = field(default=False)
    sym: bool = field(default=True)
    true_sequential: bool = field(default=True)
    model_name_or_path: Optional[str] = field(default=None)
    model_file_base_name: Optional[str] = field(default=None)

    def __post_init__(self):
        choices = fields(self)[0].metadata["choices"]
        if self.bits not in choices:
            raise ValueError(f"only support quantize to {choices} bits.")
        if self.group_size != -1 and self.group_size <= 0:
            raise ValueError("unless equal to -1, group_size must greater then 0.")
        if not (0 < self.damp_percent < 1):
            raise ValueError("damp_percent must between 0 and 1.")

    def save_pretrained(self, save_dir: str, **kwargs):
        with open(os.path.join(save_dir, "quantize_config.json"), "w", encoding="utf-8") as f:
            json.dump(self.to_dict(), f, indent=2)

    @classmethod
    def from_pretrained(cls, save_dir: str, **kwargs) -> "BaseQuantizeConfig":
        if not os.path.isdir(save_dir):
            raise FileNotFoundError(f"{save_dir}: only local directories are supported (no hub access)")
        with open(os.path.join(save_dir, "quantize_config.json"), "r", encoding="utf-8") as f:
            d = json.load(f)
        known = {f.name for f in fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in known})

    def to_dict(self) -> Dict[str, Any]:
        return {f.name: getattr(self, f.name) for f in fields(self)}


def _model_base_name(qc: BaseQuantizeConfig) -> str:
    return qc.model_file_base_name or f"gptq_model-{qc.bits}bit-{qc.group_size}g"  # _base.py:545-548


def _config_to_json(hf_config) -> Dict[str, Any]:
    d = {f.name: getattr(hf_config, f.name) for f in fields(ModelConfig) if f.name != "extra"}
    d.update(model_type=getattr(hf_config, "model_type", "hf_olmo"), architectures=list(hf_config.architectures),
             use_cache=bool(hf_config.use_cache))
    return d


def save_quantized(hf_model, quantize_config: BaseQuantizeConfig, save_dir: str, use_safetensors: bool = False,
                   safetensors_metadata: Optional[Dict[str, str]] = None) -> str:
    """Write ``config.json``, ``quantize_config.json`` and the model file the way ``save_quantized``
    does (``_base.py:534-603``).  Returns the model file's path."""
    from .qlinear import QuantLinear

    os.makedirs(save_dir, exist_ok=True)
    for name, m in hf_model.named_modules():
        if isinstance(m, QuantLinear) and m.qweight.numel() == 0:
            raise EnvironmentError(f"{name}: the checkpoint buffers were freed after post_init; nothing to save")
    base = _model_base_name(quantize_config)
    sd = {k: v.detach().to("cpu").clone().contiguous() for k, v in hf_model.state_dict().items()}
    if use_safetensors:
        from safetensors.torch import save_file

        if safetensors_metadata is None:
            safetensors_metadata = {}
        elif not isinstance(safetensors_metadata, dict):
            raise TypeError("safetensors_metadata must be a dictionary.")
        meta = {str(k): str(v) for k, v in safetensors_metadata.items()}
        meta.update(format="pt", gptq_bits=str(quantize_config.bits), gptq_group_size=str(quantize_config.group_size),
                    gptq_desc_act=str(quantize_config.desc_act), gptq_damp_percent=str(quantize_config.damp_percent))
        path = os.path.join(save_dir, base + ".safetensors")
        save_file(sd, path, meta)
    else:
        path = os.path.join(save_dir, base + ".bin")
        torch.save(sd, path)
    with open(os.path.join(save_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(_config_to_json(hf_model.config), f, indent=2)
    quantize_config.save_pretrained(save_dir)
    quantize_config.model_name_or_path = save_dir
    quantize_config.model_file_base_name = base
    return path


def _iter_tensors(path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """Tensors of a ``.safetensors`` / ``.bin`` / ``.pt`` file, one at a time where the format allows."""
    if path.endswith(".safetensors"):
        from safetensors import safe_open

        with safe_open(path, framework="pt", device="cpu") as f:
            for k in f.keys():
                yield k, f.get_tensor(k)
    else:
        sd = torch.load(path, map_location="cpu", weights_only=True, mmap=True)
        if not isinstance(sd, dict):
            raise TypeError(f"{path}: expected a state dict")
        for k, v in sd.items():
            yield k, v


def from_quantized(model_name_or_path: str, device="cuda:0", use_safetensors: Optional[bool] = None,
                   quantize_config: Optional[BaseQuantizeConfig] = None, model_basename: Optional[str] = None,
                   dtype: torch.dtype = torch.bfloat16, max_cache_len: Optional[int] = None,
                   free_checkpoint_buffers: bool = False):
    """``from_quantized`` (``_base.py:784-918``) for a local directory: read the configs, build the HF-style
    model with ``QuantLinear`` in place of the block Linears, load every tensor by name straight to the GPU,
    build the kernel layouts.  Returns ``(hf_model, quantize_config)``."""
    from .hf import OLMoConfig, OLMoForCausalLM
    from .model import OLMo
    from .qlinear import OLMoGPTQForCausalLM, QuantLinear

    if not os.path.isdir(model_name_or_path):
        raise FileNotFoundError(f"{model_name_or_path}: only local directories are supported (no hub access)")
    with open(os.path.join(model_name_or_path, "config.json"), "r", encoding="utf-8") as f:
        cj = json.load(f)
    if cj.get("model_type", "hf_olmo") not in ("hf_olmo", "olmo"):
        raise TypeError(f"{cj.get('model_type')} isn't supported yet.")  # _base.py:845-846
    if quantize_config is None:
        quantize_config = BaseQuantizeConfig.from_pretrained(model_name_or_path)
    base = model_basename or _model_base_name(quantize_config)
    exts = [".safetensors"] if use_safetensors else ([".bin", ".pt"] if use_safetensors is False else [".safetensors", ".bin", ".pt"])
    path = next((os.path.join(model_name_or_path, base + e) for e in exts
                 if os.path.isfile(os.path.join(model_name_or_path, base + e))), None)
    if path is None:
        raise FileNotFoundError(f"Could not find model in {model_name_or_path}")  # _base.py:861

    mc = ModelConfig.from_dict(cj)
    hf_cfg = OLMoConfig.from_model_config(mc, use_cache=bool(cj.get("use_cache", False)))
    model = OLMo(mc, device=device, dtype=dtype, max_cache_len=max_cache_len, block_weight_device="meta")
    hf = OLMoForCausalLM(hf_cfg, model=model)
    layers = [n for n in _linear_names(hf) if n.startswith(OLMoGPTQForCausalLM.layers_block_name + ".")]
    from .qlinear import make_quant

    make_quant(hf, layers, quantize_config.bits, quantize_config.group_size, desc_act=False, device=device)

    own = dict(hf.named_parameters())
    own.update(dict(hf.named_buffers()))
    seen = set()
    with torch.no_grad():
        for k, v in _iter_tensors(path):
            tgt = own.get(k)
            if tgt is None:
                continue  # tensors this path has no use for (e.g. rotary inv_freq buffers)
            if tuple(v.shape) != tuple(tgt.shape):
                raise ValueError(f"{k}: shape {tuple(v.shape)} != {tuple(tgt.shape)}")
            tgt.copy_(v.to(device=tgt.device, dtype=tgt.dtype))
            seen.add(k)
    missing = [k for k in own if k not in seen and not k.endswith((".g_idx", ".bias"))]
    if missing:
        raise KeyError(f"missing tensors in {path}: {missing[:5]}{'...' if len(missing) > 5 else ''}")
    for m in hf.modules():
        if isinstance(m, QuantLinear):
            m._tiled = None
            m.post_init(free_checkpoint_buffers=free_checkpoint_buffers)
    model.post_init()
    quantize_config.model_name_or_path = model_name_or_path
    quantize_config.model_file_base_name = base
    return hf, quantize_config


def _linear_names(module: torch.nn.Module):
    from .qlinear import find_layers

    return find_layers(module)


# ---------------------------------------------------------------------------------------------
# unsharded OLMo checkpoints
# ---------------------------------------------------------------------------------------------
def make_state_dict_compatible(state_dict: Dict[str, torch.Tensor], config: ModelConfig) -> Dict[str, torch.Tensor]:
    """The key fix-ups of ``OLMo._make_state_dict_compatible`` (``olmo/model.py:1786-1878``), for a model
    whose blocks are a flat list: FSDP prefixes dropped, a shared ``norm`` split into ``attn_norm`` and
    ``ff_norm``, block groups flattened to ``transformer.blocks.{i}``.  Modifies and returns ``state_dict``."""
    for key in list(state_dict.keys()):
        new = key.replace("_fsdp_wrapped_module.", "")
        if new != key:
            state_dict[new] = state_dict.pop(key)
    if config.block_type == "sequential":
        for key in list(state_dict.keys()):
            for leaf in ("weight", "bias"):
                if fnmatch(key, f"transformer.*.norm.{leaf}"):
                    t = state_dict.pop(key)
                    state_dict[key.replace(f"norm.{leaf}", f"attn_norm.{leaf}")] = t
                    state_dict[key.replace(f"norm.{leaf}", f"ff_norm.{leaf}")] = t.clone()
    if "transformer.block_groups.0.0.attn_out.weight" in state_dict:
        gsz = len([k for k in state_dict if fnmatch(k, "transformer.block_groups.0.*.attn_out.weight")])
        for key in list(state_dict.keys()):
            m = re.match(r"transformer.block_groups\.(\d+)\.(\d+)\..*", key)
            if m is not None:
                gi, bi = int(m.group(1)), int(m.group(2))
                state_dict[key.replace(f"block_groups.{gi}.{bi}.", f"blocks.{gi * gsz + bi}.")] = state_dict.pop(key)
    return state_dict


def load_unsharded_checkpoint(checkpoint_dir: str, device="cuda:0", dtype: torch.dtype = torch.bfloat16,
                              max_cache_len: Optional[int] = None):
    """``OLMo.from_checkpoint`` for the unsharded layout (``olmo/model.py:1730-1764``): ``config.yaml``
    (its ``model`` section) plus ``model.pt`` (or ``model.safetensors``).  Sharded checkpoints belong to the
    training side and are not read here."""
    import yaml

    from .model import OLMo

    with open(os.path.join(checkpoint_dir, "config.yaml"), "r", encoding="utf-8") as f:
        y = yaml.safe_load(f)
    mc = ModelConfig.from_dict(y["model"] if "model" in y else y)
    path = next((os.path.join(checkpoint_dir, n) for n in ("model.safetensors", "model.pt")
                 if os.path.isfile(os.path.join(checkpoint_dir, n))), None)
    if path is None:
        raise FileNotFoundError(f"{checkpoint_dir}: no model.pt / model.safetensors (sharded checkpoints are not supported)")
    sd = make_state_dict_compatible(dict(_iter_tensors(path)), mc)
    model = OLMo(mc, device=device, dtype=dtype, max_cache_len=max_cache_len)
    model.load_reference_state_dict(sd)
    return model.post_init().eval()


# ---------------------------------------------------------------------------------------------
# OLMo <-> HF Olmo2ForCausalLM tensor layouts
# ---------------------------------------------------------------------------------------------
_HF_BLOCK = {  # HF name under model.layers.{i}.  <-  OLMo name under transformer.blocks.{i}.
    "self_attn.o_proj.weight": "attn_out.weight",
    "self_attn.q_norm.weight": "q_norm.weight",
    "self_attn.k_norm.weight": "k_norm.weight",
    "mlp.down_proj.weight": "ff_out.weight",
    "post_attention_layernorm.weight": "attn_norm.weight",
    "post_feedforward_layernorm.weight": "ff_norm.weight",
}


def _kv_width(config: ModelConfig) -> int:
    return config.head_dim * config.effective_n_kv_heads


def olmo_to_hf_olmo2_state_dict(sd: Dict[str, torch.Tensor], config: ModelConfig) -> Dict[str, torch.Tensor]:
    """``scripts/convert_olmo2_to_hf.py:110-163``: ``att_proj`` rows split into q | k | v, ``ff_proj`` rows
    chunked into up | gate, the rest renamed; the lm head falls back to the embedding when tied."""
    out: Dict[str, torch.Tensor] = {}
    d, dkv = config.d_model, _kv_width(config)
    for i in range(config.n_layers):
        src, dst = f"transformer.blocks.{i}.", f"model.layers.{i}."
        q, k, v = torch.split(sd[src + "att_proj.weight"], [d, dkv, dkv], dim=0)
        up, gate = torch.chunk(sd[src + "ff_proj.weight"], 2, dim=0)
        out[dst + "self_attn.q_proj.weight"], out[dst + "self_attn.k_proj.weight"] = q, k
        out[dst + "self_attn.v_proj.weight"] = v
        out[dst + "mlp.up_proj.weight"], out[dst + "mlp.gate_proj.weight"] = up, gate
        for hf_name, olmo_name in _HF_BLOCK.items():
            out[dst + hf_name] = sd[src + olmo_name]
    out["model.embed_tokens.weight"] = sd["transformer.wte.weight"]
    out["model.norm.weight"] = sd["transformer.ln_f.weight"]
    out["lm_head.weight"] = sd.get("transformer.ff_out.weight", sd["transformer.wte.weight"])
    return out


def hf_olmo2_to_olmo_state_dict(sd: Dict[str, torch.Tensor], config: ModelConfig) -> Dict[str, torch.Tensor]:
    """Inverse of :func:`olmo_to_hf_olmo2_state_dict`: fuse q | k | v into ``att_proj`` and up | gate into
    ``ff_proj`` so HF ``Olmo2ForCausalLM`` weights run through this path."""
    out: Dict[str, torch.Tensor] = {}
    for i in range(config.n_layers):
        src, dst = f"model.layers.{i}.", f"transformer.blocks.{i}."
        out[dst + "att_proj.weight"] = torch.cat([sd[src + f"self_attn.{p}_proj.weight"] for p in ("q", "k", "v")], dim=0)
        out[dst + "ff_proj.weight"] = torch.cat([sd[src + "mlp.up_proj.weight"], sd[src + "mlp.gate_proj.weight"]], dim=0)
        for hf_name, olmo_name in _HF_BLOCK.items():
            out[dst + olmo_name] = sd[src + hf_name]
    out["transformer.wte.weight"] = sd["model.embed_tokens.weight"]
    out["transformer.ln_f.weight"] = sd["model.norm.weight"]
    out["transformer.ff_out.weight"] = sd.get("lm_head.weight", sd["model.embed_tokens.weight"])
    return out

"""Random-initialised models of the reference's shapes, built directly on the GPU.

Dense weights ~ N(0, init_std) as ``olmo/initialization.py:8-22`` prescribes; int4 block Linears
are random AutoGPTQ buffers (uniform nibbles in ``qweight`` / ``qzeros``, fp16 scales
``|N(0, 0.01)|``, sequential groups of 128) swapped in with ``make_quant`` exactly as
``AutoGPTQForCausalLM.from_quantized`` does (``AGQ/auto_gptq/modeling/_base.py:863-880``).
Filling buffers with random numbers is done with torch's generators (data, not compute).
"""

from __future__ import annotations

from typing import Optional

import torch

from .config import ModelConfig
from .model import OLMo
from .qlinear import OLMoGPTQForCausalLM, QuantLinear, make_quant

__all__ = ["build_random_model", "fill_random_int4"]


@torch.no_grad()
def fill_random_int4(m: QuantLinear, gen: torch.Generator) -> None:
    dev = m.qweight.device
    for name in ("qweight", "qzeros"):
        t = getattr(m, name)
        r = torch.randint(-(2 ** 31), 2 ** 31 - 1, t.shape, dtype=torch.int64, device=dev, generator=gen)
        t.copy_(r.to(torch.int32))
    s = torch.empty(m.scales.shape, dtype=torch.float32, device=dev).normal_(0.0, 0.01, generator=gen).abs_()
    m.scales.copy_(s.to(torch.float16))


def build_random_model(cfg: ModelConfig, dtype: torch.dtype = torch.bfloat16, quantized: bool = False, seed: int = 0,
                       device="cuda", max_cache_len: Optional[int] = None,
                       free_checkpoint_buffers: bool = False) -> OLMo:
    model = OLMo(cfg, device=device, dtype=dtype, max_cache_len=max_cache_len,
                 block_weight_device="meta" if quantized else None)
    model.reset_parameters(seed)
    if quantized:
        names = [f"transformer.blocks.{i}.{n}" for i in range(cfg.n_layers)
                 for (n,) in OLMoGPTQForCausalLM.inside_layer_modules]
        make_quant(model, names, 4, 128, device=device)
        gen = torch.Generator(device=device).manual_seed(seed + 1)
        for mod in model.modules():
            if isinstance(mod, QuantLinear):
                fill_random_int4(mod, gen)
                mod.post_init(free_checkpoint_buffers=free_checkpoint_buffers)
    model.post_init()
    return model

"""Group-wise int4 ``QuantLinear`` with the reference's module surface, computed by the HIP
kernels of this package.

Mirrors AutoGPTQ's ``QuantLinear`` as vendored in the reference
(``inference/compression/dependencies/AutoGPTQ/auto_gptq/nn_modules/qlinear/qlinear_cuda_old.py:22-97,192-290``):
same constructor, attributes (``QUANT_TYPE, infeatures, outfeatures, bits, group_size, maxq``),
buffer names / shapes / dtypes (``qweight, qzeros, scales, g_idx, bias``) so checkpoints load by
name, ``post_init()``, ``pack()`` and ``forward()``; plus ``make_quant`` (``.../modeling/_utils.py:52-111``)
and the OLMo wiring constants of ``inference/compression/olmo_gptq_class.py:4-17``.

Differences, on purpose:
  * ``forward`` returns the input's dtype (bfloat16 on this path) instead of always float16
    (``qlinear_cuda_old.py:287-290``), so that residual adds stay in one dtype;
  * ``post_init`` derives a re-tiled copy of the weight for the matrix-core kernels, the way the
    reference's exllama back-end rewrites ``qweight`` in its own ``post_init``
    (``qlinear_exllama.py:85-98``);
  * only ``bits=4``, ``group_size=128`` run through the linear kernels (the dequantise table kernel
    also handles other group sizes); act-order checkpoints (non-sequential ``g_idx``) get their rows
    sorted by group in ``post_init`` and their activation columns gathered in ``forward``, as the
    reference's exllama back-end does (``qlinear_exllama.py:85-98``, ``q4_matrix.cu:105-169``).
"""

from __future__ import annotations

import math
from typing import Iterable, Optional

import torch
import torch.nn as nn

from . import ops

__all__ = ["QuantLinear", "make_quant", "OLMoGPTQForCausalLM", "find_layers"]


class QuantLinear(nn.Module):
    QUANT_TYPE = "hip-mi355x"

    def __init__(self, bits, group_size, infeatures, outfeatures, bias, use_cuda_fp16=True,
                 kernel_switch_threshold=128, trainable=False, device=None):
        super().__init__()
        if bits not in [2, 3, 4, 8]:
            raise NotImplementedError("Only 2,3,4,8 bits are supported.")  # same message as the reference
        if bits != 4:
            raise NotImplementedError("the MI355X kernels implement bits=4 only")
        if trainable:
            raise NotImplementedError("trainable=True is not implemented (inference only)")
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.bits = bits
        self.group_size = group_size if group_size != -1 else infeatures
        self.maxq = 2 ** self.bits - 1
        G = math.ceil(infeatures / self.group_size)
        self.register_buffer("qweight", torch.zeros((infeatures // 32 * bits, outfeatures), dtype=torch.int32, device=device))
        self.register_buffer("qzeros", torch.zeros((G, outfeatures // 32 * bits), dtype=torch.int32, device=device))
        self.register_buffer("scales", torch.zeros((G, outfeatures), dtype=torch.float16, device=device))
        self.register_buffer("g_idx", (torch.arange(infeatures, dtype=torch.int32, device=device) // self.group_size))
        if bias:
            self.register_buffer("bias", torch.zeros((outfeatures), dtype=torch.float16, device=device))
        else:
            self.bias = None
        self.use_cuda_fp16 = use_cuda_fp16
        self.kernel_switch_threshold = kernel_switch_threshold
        self.trainable = trainable
        self._tiled: Optional[ops.W4Tiled] = None
        self._perm: Optional[torch.Tensor] = None  # act-order: row order of the tiled copy (int32 [K])
        self._has_bias = False  # decided in post_init: whether forward() adds the bias buffer

    # -- one-time preparation ------------------------------------------------------------------
    def post_init(self, free_checkpoint_buffers: bool = False):
        """Validate the buffers and build the tiled copy on the GPU (no-op when already built)."""
        if self._tiled is not None:
            return self
        if not self.qweight.is_cuda:
            raise RuntimeError("QuantLinear.post_init needs the buffers on the GPU; there is no CPU path")
        K = self.infeatures
        seq = torch.arange(K, dtype=torch.int32, device=self.g_idx.device) // self.group_size
        qweight = self.qweight
        self._perm = None
        if not torch.equal(self.g_idx.to(torch.int32), seq):
            # act-order: sort the rows of W by group once (stable, so rows keep their order inside a group);
            # forward() gathers the activation columns to match -- what the reference's exllama back-end does
            # (q4_matrix.cu:105-169 make_sequential, column_remap.cu:9-63)
            perm = torch.argsort(self.g_idx.to(torch.int64), stable=True)
            if not torch.equal(self.g_idx.to(torch.int32)[perm], seq):
                raise NotImplementedError("g_idx whose groups do not hold exactly group_size rows each is not supported")
            sh = torch.arange(0, 32, 4, dtype=torch.int32, device=qweight.device).view(1, 8, 1)
            q = ((qweight.unsqueeze(1) >> sh) & 15).reshape(K, self.outfeatures)[perm]  # nibbles, rows sorted
            qweight = (q.view(K // 8, 8, self.outfeatures) << sh).sum(1, dtype=torch.int32)  # nibble 7 lands in the sign bit
            self._perm = perm.to(torch.int32).contiguous()
        # a bias that is all zero (what make_quant creates and OLMo checkpoints hold) costs nothing
        self._has_bias = self.bias is not None and bool(self.bias.any())
        self._tiled = ops.w4_repack(qweight, self.qzeros, self.scales, self.group_size)
        if free_checkpoint_buffers:
            empty = torch.empty(0, dtype=torch.int32, device=self.qweight.device)
            self.qweight, self.qzeros = empty, empty.clone()
            self.scales = torch.empty(0, dtype=torch.float16, device=self.scales.device)
        return self

    def _load_from_state_dict(self, *args, **kwargs):
        self._tiled = None  # new buffers: the tiled copy must be rebuilt
        return super()._load_from_state_dict(*args, **kwargs)

    @property
    def tiled(self) -> ops.W4Tiled:
        if self._tiled is None:
            self.post_init()
        return self._tiled

    def dequantize(self) -> torch.Tensor:
        """fp16 ``[K, N]`` table (the reference's torch dequantize, bit for bit)."""
        if self._tiled is not None:
            t = ops.w4t_dequant_fp16(self._tiled)
            if self._perm is None:
                return t
            out = torch.empty_like(t)
            out[self._perm.long()] = t  # row i of the sorted table is row perm[i] of W
            return out
        return ops.w4_dequant_fp16(self.qweight, self.qzeros, self.scales, self.group_size, self.g_idx)

    # -- quantise a dense layer with given parameters ----------------------------------------------
    def pack(self, linear, scales, zeros, g_idx=None):
        """``QuantLinear.pack`` (``qlinear_cuda_old.py:98-190``): ``q = round((W + s*z)/s)``, stored
        zero is ``z-1``.  ``scales`` / ``zeros``: ``[N, G]``.  Host-side, one-time."""
        W = linear.weight.data.detach().to("cpu", torch.float32)
        s = scales.detach().to("cpu", torch.float32).t().contiguous()
        z = zeros.detach().to("cpu", torch.float32).t().contiguous()
        dev = self.qweight.device
        s16 = s.half()
        gi = torch.arange(self.infeatures) // self.group_size
        intw = torch.round((W.t() + (z * s)[gi]) / s16[gi].float()).to(torch.int64).clamp_(0, self.maxq)
        sh = torch.arange(0, 32, 4, dtype=torch.int64)
        qw = (intw.view(-1, 8, intw.shape[1]) << sh.view(1, 8, 1)).sum(1)
        zq = (z - 1).to(torch.int64).clamp_(0, self.maxq)
        qz = (zq.view(zq.shape[0], -1, 8) << sh.view(1, 1, 8)).sum(2)

        def to_i32(t):
            return torch.where(t >= 2 ** 31, t - 2 ** 32, t).to(torch.int32)

        self.qweight = to_i32(qw).to(dev)
        self.qzeros = to_i32(qz).to(dev)
        self.scales = s16.to(dev)
        if getattr(linear, "bias", None) is not None and self.bias is not None:
            self.bias = linear.bias.detach().clone().half().to(dev)
        self._tiled = None

    # -- forward ---------------------------------------------------------------------------------
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # bf16 rows (the model's own activations) stay bf16; anything else goes through the reference's own arithmetic:
        # cast to fp16, fp16 weights, result cast back (qlinear_cuda_old.py:287-290)
        in_dtype = x.dtype
        if in_dtype not in (torch.bfloat16, torch.float16):
            x = x.to(torch.float16)
        t = self.tiled
        x = x.contiguous()
        if self._perm is not None:
            x = ops.gather_columns(x, self._perm)
        y = ops.w4_linear(x, t)
        if self._has_bias:  # qlinear_cuda_old.py:288-290
            y = ops.add_bias(y, self.bias)
        return y if y.dtype == in_dtype else y.to(in_dtype)

    def extra_repr(self):
        return f"in={self.infeatures}, out={self.outfeatures}, bits={self.bits}, group_size={self.group_size}"


def find_layers(module: nn.Module, layers=(nn.Linear,), name: str = ""):
    """``find_layers`` of ``AGQ/auto_gptq/modeling/_utils.py:40-49``."""
    if isinstance(module, tuple(layers)):
        return {name: module}
    res = {}
    for n, child in module.named_children():
        res.update(find_layers(child, layers, name + "." + n if name else n))
    return res


def make_quant(module: nn.Module, names: Iterable[str], bits: int, group_size: int, name: str = "",
               use_triton: bool = False, disable_exllama: bool = False, use_cuda_fp16: bool = True,
               desc_act: bool = False, trainable: bool = False, device=None):
    """Replace every ``nn.Linear`` whose qualified name is in ``names`` by a ``QuantLinear`` with a
    zero bias buffer -- same contract as the reference's ``make_quant``
    (``AGQ/auto_gptq/modeling/_utils.py:52-111``).  ``device`` (not in the reference) places the buffers of
    layers that replace meta-device Linears."""
    if use_triton:
        raise NotImplementedError("no Triton back-end here")
    names = set(names)
    if isinstance(module, QuantLinear):
        return
    for attr, child in list(module.named_children()):
        name1 = name + "." + attr if name else attr
        if name1 in names and isinstance(child, nn.Linear):
            dev = child.weight.device
            dev = device if dev.type == "meta" else dev  # meta: the caller says where the buffers go
            new = QuantLinear(bits, group_size, child.in_features, child.out_features, True,
                              use_cuda_fp16=use_cuda_fp16, trainable=trainable, device=dev)
            setattr(module, attr, new)
        else:
            make_quant(child, names, bits, group_size, name1, use_triton=use_triton, disable_exllama=disable_exllama,
                       use_cuda_fp16=use_cuda_fp16, desc_act=desc_act, trainable=trainable, device=device)


class OLMoGPTQForCausalLM:
    """``OLMoGPTQForCausalLM`` (``inference/compression/olmo_gptq_class.py:4-17``) on top of the parts of
    ``BaseGPTQForCausalLM`` the inference path uses (``AGQ/auto_gptq/modeling/_base.py:85-100,450-460,
    534-603,784-918``): the wiring constants, the Linear -> ``QuantLinear`` swap, ``from_quantized`` /
    ``save_quantized`` for local AutoGPTQ directories, and ``forward`` / ``generate`` passed through to the
    wrapped HF-style model.  Calibration (``quantize``) is outside this path."""

    layer_type = "OLMoBlock"
    layers_block_name = "model.transformer.blocks"
    outside_layer_modules = ["model.transformer.wte", "model.transformer.ln_f"]
    inside_layer_modules = [["att_proj"], ["attn_out"], ["ff_proj"], ["ff_out"]]
    lm_head_name = "model.transformer.ff_out"

    def __init__(self, model: nn.Module, quantized: bool, quantize_config):
        self.model = model
        self._quantized = quantized
        self.quantize_config = quantize_config
        self.config = model.config

    @property
    def quantized(self) -> bool:
        return self._quantized

    @property
    def device(self) -> torch.device:
        return next(self.model.parameters()).device

    def to(self, device):
        self.model.to(device)
        return self

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)

    __call__ = forward

    def generate(self, **kwargs):
        with torch.inference_mode():
            return self.model.generate(**kwargs)

    def prepare_inputs_for_generation(self, *args, **kwargs):
        return self.model.prepare_inputs_for_generation(*args, **kwargs)

    def quantize(self, *args, **kwargs):
        raise NotImplementedError("GPTQ calibration is not part of the inference path; load a quantized directory")

    def save_quantized(self, save_dir: str, use_safetensors: bool = False, safetensors_metadata=None):
        if not self.quantized:
            raise EnvironmentError("can only save quantized model, please execute .quantize first.")  # _base.py:540-541
        from .checkpoint import save_quantized

        return save_quantized(self.model, self.quantize_config, save_dir, use_safetensors, safetensors_metadata)

    def save_pretrained(self, save_dir: str, use_safetensors: bool = False, safetensors_metadata=None, **kwargs):
        return self.save_quantized(save_dir, use_safetensors, safetensors_metadata)  # _base.py:605-614

    @classmethod
    def from_quantized(cls, model_name_or_path: str, device="cuda:0", use_safetensors: Optional[bool] = None,
                       quantize_config=None, model_basename: Optional[str] = None, use_triton: bool = False,
                       trainable: bool = False, **kwargs) -> "OLMoGPTQForCausalLM":
        if use_triton:
            raise NotImplementedError("no Triton back-end here")
        if trainable:
            raise NotImplementedError("trainable=True is not implemented (inference only)")
        from .checkpoint import from_quantized

        hf, qc = from_quantized(model_name_or_path, device=device, use_safetensors=use_safetensors,
                                quantize_config=quantize_config, model_basename=model_basename, **kwargs)
        return cls(hf, True, qc)

    @classmethod
    def quantize_modules(cls, hf_model: nn.Module, bits: int = 4, group_size: int = 128) -> nn.Module:
        """Swap the four block Linears of every layer for ``QuantLinear`` (lm head and embedding stay dense)."""
        layers = find_layers(hf_model)
        ignore = [cls.lm_head_name] + cls.outside_layer_modules
        names = [n for n in layers
                 if not any(n.startswith(i) for i in ignore) and n.startswith(cls.layers_block_name + ".")]
        make_quant(hf_model, names, bits, group_size)
        return hf_model

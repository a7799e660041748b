"""Model hyper-parameters for the inference forward pass.

Field names and defaults follow the reference's ``ModelConfig``
(``olmo/config.py:235-497``) so that a reference config (YAML section ``model:`` or
the HF ``config.json``) can be passed through ``ModelConfig.from_dict`` unchanged.
Only the switches that the inference path implements are accepted with non-default
values; everything else raises ``OLMoConfigurationError`` (same exception name as
``olmo/exceptions.py``) instead of silently computing something different.
"""

from __future__ import annotations

from dataclasses import dataclass, field, fields
from typing import Any, Dict, Optional

__all__ = ["ModelConfig", "OLMoConfigurationError", "PRESETS"]


class OLMoConfigurationError(Exception):
    """Raised for a configuration the inference path cannot run (``olmo/exceptions.py``)."""


@dataclass
class ModelConfig:
    # -- the reference's vocabulary (olmo/config.py:242-470) -------------------------------
    d_model: int = 768
    n_heads: int = 12
    n_kv_heads: Optional[int] = None
    clip_qkv: Optional[float] = None
    n_layers: int = 12
    mlp_ratio: int = 4
    mlp_hidden_size: Optional[int] = None
    activation_type: str = "swiglu"
    block_type: str = "sequential"
    block_group_size: int = 1
    alibi: bool = False
    alibi_bias_max: float = 8.0
    rope: bool = False
    rope_full_precision: bool = True
    rope_theta: float = 10_000
    flash_attention: bool = False
    attention_dropout: float = 0.1
    multi_query_attention: Optional[bool] = None
    attention_layer_norm: bool = False
    residual_dropout: float = 0.1
    embedding_dropout: float = 0.1
    embedding_layer_norm: bool = False
    layer_norm_type: str = "default"
    layer_norm_with_affine: bool = True
    layer_norm_eps: float = 1e-05
    attention_layer_norm_with_affine: bool = True
    max_sequence_length: int = 1024
    include_bias: bool = True
    bias_for_layer_norm: Optional[bool] = None
    scale_logits: bool = False
    vocab_size: int = 50257
    embedding_size: Optional[int] = 50304
    weight_tying: bool = True
    eos_token_id: int = 50256
    pad_token_id: int = 50256
    init_device: Optional[str] = None
    init_fn: str = "normal"
    init_std: float = 0.02
    init_cutoff_factor: Optional[float] = None
    precision: Optional[str] = None
    scale_emb_init: bool = False
    emb_init_std: Optional[float] = None
    norm_after: bool = False
    # anything else found in a reference config is kept here, untouched
    extra: Dict[str, Any] = field(default_factory=dict)

    # -- derived quantities ----------------------------------------------------------------
    @property
    def effective_n_kv_heads(self) -> int:
        """``olmo/config.py:477-496``."""
        if self.n_kv_heads is None:
            return 1 if self.multi_query_attention is True else self.n_heads
        if self.multi_query_attention is None:
            return self.n_kv_heads
        should_be = 1 if self.multi_query_attention else self.n_heads
        if self.n_kv_heads == should_be:
            return should_be
        raise OLMoConfigurationError("You can't set `multi_query_attention` and `n_kv_heads` at the same time.")

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_heads

    @property
    def hidden_size(self) -> int:
        """Width of ``ff_proj``'s output (``olmo/model.py:421-423``)."""
        return self.mlp_hidden_size if self.mlp_hidden_size is not None else self.mlp_ratio * self.d_model

    @property
    def act_out_size(self) -> int:
        """Width of ``ff_out``'s input: SwiGLU halves it (``olmo/model.py:370-372,457-462``)."""
        return self.hidden_size // 2 if self.activation_type == "swiglu" else self.hidden_size

    @property
    def logits_size(self) -> int:
        return self.embedding_size or self.vocab_size

    # -- construction ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        known = {f.name for f in fields(cls)} - {"extra"}
        kw = {k: v for k, v in d.items() if k in known}
        extra = {k: v for k, v in d.items() if k not in known}
        for k in ("activation_type", "block_type", "layer_norm_type", "init_fn"):
            if k in kw and kw[k] is not None:
                kw[k] = str(getattr(kw[k], "value", kw[k]))
        return cls(**kw, extra=extra)

    def validate_for_inference(self) -> None:
        """Reject what the HIP path does not implement (mirrors ``olmo/model.py:1076-1100``)."""

        def bad(msg: str):
            raise OLMoConfigurationError(msg)

        if self.alibi and self.rope:
            bad("ALiBi and RoPE are mutually exclusive")
        if self.alibi or not self.rope:
            bad("the MI355X inference path implements rotary positions only (rope=true, alibi=false)")
        if self.block_type != "sequential":
            bad(f"block_type={self.block_type!r} is not implemented; only 'sequential'")
        if self.activation_type != "swiglu":
            bad(f"activation_type={self.activation_type!r} is not implemented; only 'swiglu'")
        if self.include_bias:
            bad("include_bias=true is not implemented")
        if self.embedding_layer_norm or self.scale_logits:
            bad("embedding_layer_norm / scale_logits are not implemented")
        if self.clip_qkv is not None and not self.clip_qkv > 0:
            bad("clip_qkv must be positive")  # olmo/model.py:444-445
        if self.layer_norm_type == "rms":
            if not self.layer_norm_with_affine:
                bad("rms layer norm without affine is not implemented")
        elif self.layer_norm_type == "default":
            if self.layer_norm_with_affine:
                bad("affine 'default' LayerNorm is not implemented; only the non-parametric one")
        else:
            bad(f"layer_norm_type={self.layer_norm_type!r} is not implemented")
        if self.attention_layer_norm and self.layer_norm_type != "rms":
            bad("attention_layer_norm needs layer_norm_type='rms'")
        if self.d_model % self.n_heads:
            bad("d_model must be divisible by n_heads")
        if self.n_heads % self.effective_n_kv_heads:
            bad("n_heads must be divisible by n_kv_heads")
        if self.head_dim not in (32, 64, 128):
            bad(f"head_dim={self.head_dim} is not implemented (32, 64 or 128)")
        if self.hidden_size % 2:
            bad("mlp_hidden_size must be even for SwiGLU")


def _olmo2(d, L, H, hidden, vocab=100352, maxlen=4096) -> ModelConfig:
    # configs/official-1124/OLMo2-7B-stage1.yaml:5-36 (7B), OLMo2-13B-stage1.yaml:5-36,
    # configs/official-0425/OLMo2-1B-stage1.yaml:10-41
    return ModelConfig(
        d_model=d, n_heads=H, n_layers=L, mlp_hidden_size=hidden, weight_tying=False, alibi=False, rope=True,
        rope_theta=500000, flash_attention=False, attention_dropout=0.0, attention_layer_norm=True,
        include_bias=False, layer_norm_type="rms", layer_norm_with_affine=True, layer_norm_eps=1e-6,
        bias_for_layer_norm=False, attention_layer_norm_with_affine=True, norm_after=True,
        max_sequence_length=maxlen, vocab_size=100278, embedding_size=vocab, eos_token_id=100257,
        pad_token_id=100277, residual_dropout=0.0, embedding_dropout=0.0, init_fn="normal", init_std=0.02,
        init_cutoff_factor=3.0,
    )


PRESETS = {
    # 20M-style fp32 model with non-parametric LayerNorm (shapes of configs/tiny/OLMo-20M.yaml,
    # norm as in configs/official-0724/OLMo-1B.yaml:23-26), 16 layers
    "olmo-20m": ModelConfig(
        d_model=256, n_heads=8, n_layers=16, mlp_ratio=8, weight_tying=False, alibi=False, rope=True,
        attention_dropout=0.0, attention_layer_norm=False, include_bias=False, layer_norm_type="default",
        layer_norm_with_affine=False, layer_norm_eps=1e-5, max_sequence_length=4096, vocab_size=50280,
        embedding_size=50304, eos_token_id=0, pad_token_id=1, residual_dropout=0.0, embedding_dropout=0.0,
        norm_after=False,
    ),
    "olmo2-1b": _olmo2(2048, 16, 16, 16384),
    "olmo2-7b": _olmo2(4096, 32, 32, 22016),
    "olmo2-13b": _olmo2(5120, 40, 40, 27648),
}

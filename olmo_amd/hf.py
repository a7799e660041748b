"""HF-style wrapper: ``OLMoConfig`` and ``OLMoForCausalLM`` with the surface of
``hf_olmo/configuration_olmo.py:14-59`` and ``hf_olmo/modeling_olmo.py:41-160``.

``forward`` passes through to ``OLMo.forward`` and returns a ``CausalLMOutputWithPast``-shaped
object; ``prepare_inputs_for_generation`` keeps only the last token when a cache is given
(``modeling_olmo.py:150-160``).  ``generate`` is this package's own loop (the HF
``GenerationMixin`` is third-party code and is not reimplemented): prefill, then one captured
decode step per token, greedy or sampled; ``num_beams > 1`` runs OLMo's own beam search.  The module tree is ``self.model.transformer...`` so the names AutoGPTQ
addresses (``model.transformer.blocks.{i}.att_proj`` ...,
``inference/compression/olmo_gptq_class.py:6``) resolve.
"""

from __future__ import annotations

from dataclasses import asdict, fields
from typing import Any, Dict, List, NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from .config import ModelConfig
from .generate import greedy_generate
from .model import OLMo

__all__ = ["OLMoConfig", "OLMoForCausalLM", "CausalLMOutputWithPast"]


class CausalLMOutputWithPast(NamedTuple):
    """Field names of ``transformers.modeling_outputs.CausalLMOutputWithPast``."""

    loss: Optional[torch.Tensor]
    logits: torch.Tensor
    past_key_values: Optional[List[Tuple[torch.Tensor, torch.Tensor]]]
    hidden_states: Optional[Tuple[torch.Tensor, ...]]


class OLMoConfig:
    """Every ``ModelConfig`` field mirrored as an attribute, plus ``use_cache`` (default False as in
    ``configuration_olmo.py:18-22``) and the HF aliases (``:28-38``)."""

    model_type = "hf_olmo"

    def __init__(self, use_cache: bool = False, **kwargs):
        base = {f.name: getattr(ModelConfig(), f.name) for f in fields(ModelConfig) if f.name != "extra"}
        base.update(kwargs)
        for k, v in base.items():
            setattr(self, k, v)
        self.use_cache = use_cache
        self.architectures = base.get("architectures") or ["OLMoForCausalLM"]
        self.use_return_dict = True

    @classmethod
    def from_model_config(cls, mc: ModelConfig, use_cache: bool = False) -> "OLMoConfig":
        d = asdict(mc)
        d.pop("extra", None)
        return cls(use_cache=use_cache, **d)

    def to_model_config(self) -> ModelConfig:
        """``create_model_config_from_pretrained_config`` (``hf_olmo/modeling_olmo.py:19-38``)."""
        return ModelConfig.from_dict({f.name: getattr(self, f.name) for f in fields(ModelConfig) if f.name != "extra"})

    @property
    def num_attention_heads(self):
        return self.n_heads

    @property
    def num_hidden_layers(self):
        return self.n_layers

    @property
    def hidden_size(self):
        return self.d_model


class OLMoForCausalLM(nn.Module):
    _no_split_modules = ["OLMoBlock"]
    base_model_prefix = "model"

    def __init__(self, config: OLMoConfig, model: Optional[OLMo] = None, device="cuda",
                 dtype: torch.dtype = torch.bfloat16, **model_kwargs):
        super().__init__()
        self.config = config
        self.model = model if model is not None else OLMo(config.to_model_config(), device=device, dtype=dtype,
                                                          **model_kwargs)

    def forward(
        self,
        input_ids: torch.LongTensor = None,
        inputs_embeds: Optional[torch.FloatTensor] = None,
        attention_mask: Optional[torch.Tensor] = None,
        attention_bias: Optional[torch.Tensor] = None,
        past_key_values: Optional[List[torch.FloatTensor]] = None,
        labels: Optional[torch.LongTensor] = None,
        use_cache: Optional[bool] = None,
        output_attentions: Optional[bool] = None,
        output_hidden_states: Optional[bool] = None,
        return_dict: Optional[bool] = None,
        cache_position: Any = None,
    ):
        if use_cache is None:
            use_cache = self.config.use_cache
        if output_attentions:
            raise ValueError("output_attentions is not yet supported in OLMo")  # modeling_olmo.py:103-104
        return_dict = return_dict if return_dict is not None else self.config.use_return_dict
        if past_key_values is not None and hasattr(past_key_values, "get_seq_length"):
            # a transformers Cache object: this path keeps its own cache, only an empty one is accepted
            if past_key_values.get_seq_length() != 0:
                raise NotImplementedError("transformers Cache objects are not supported; pass the returned "
                                          "past_key_values list back instead")
            past_key_values = None
        outputs = self.model.forward(
            input_ids=input_ids,
            input_embeddings=inputs_embeds,
            attention_mask=attention_mask,
            attention_bias=attention_bias,
            past_key_values=past_key_values,
            use_cache=use_cache,
            output_hidden_states=output_hidden_states,
        )
        logits = outputs.logits
        loss = None
        if labels is not None:
            # shifted cross entropy (modeling_olmo.py:123-135): evaluation bookkeeping, plain torch
            shift_logits = logits[..., :-1, :].contiguous().view(-1, logits.shape[-1]).float()
            shift_labels = labels[..., 1:].contiguous().view(-1).to(shift_logits.device)
            loss = torch.nn.functional.cross_entropy(shift_logits, shift_labels)
        if not return_dict:
            output = (logits,) + tuple(outputs[1:])
            return (loss,) + output if loss is not None else output
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=outputs.attn_key_values,
                                      hidden_states=outputs.hidden_states)

    @classmethod
    def can_generate(cls) -> bool:
        return True

    def prepare_inputs_for_generation(self, input_ids: torch.LongTensor, past_key_values=None, **kwargs):
        if past_key_values:
            input_ids = input_ids[:, -1:]
        model_inputs: Dict[str, Any] = {"input_ids": input_ids, "past_key_values": past_key_values}
        model_inputs.update(kwargs)
        model_inputs["use_cache"] = kwargs.pop("use_cache", self.config.use_cache)
        return model_inputs

    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor, attention_mask: Optional[torch.Tensor] = None,
                 max_new_tokens: int = 20, do_sample: bool = False, num_beams: int = 1,
                 eos_token_id: Optional[int] = None, pad_token_id: Optional[int] = None, use_graph: bool = True,
                 temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0,
                 **unused) -> torch.Tensor:
        """Greedy, sampled or beam-searched continuation: returns ``[B, prompt + new tokens]`` token ids like HF
        ``generate`` (``num_beams > 1``: the best beam, fewer than ``max_new_tokens`` columns when every beam ended early).
        With ``do_sample`` the logits go through temperature, top-k and top-p in HF's order and one token is
        drawn per step on the device (``top_k=0`` / ``top_p=1.0`` switch a filter off); ``seed`` fixes the draw."""
        if num_beams != 1:
            # OLMo's own search (olmo/beam_search.py via OLMo.generate), not transformers' BeamSearchScorer:
            # summed log-probabilities, no length penalty; the best beam of each sequence, padded with the
            # end token once it has ended
            sampler = None
            if do_sample:  # per-node candidates drawn instead of taken from the top (olmo/beam_search.py samplers)
                from .beam_search import MultinomialSampler, TopKSampler, TopPSampler

                if top_p < 1.0:
                    sampler = TopPSampler(p=top_p, temperature=temperature, seed=seed)
                elif top_k:
                    sampler = TopKSampler(k=top_k, temperature=temperature, seed=seed)
                else:
                    sampler = MultinomialSampler(temperature=temperature, seed=seed)
            out = self.model.generate(input_ids, attention_mask=attention_mask, max_steps=max_new_tokens,
                                      beam_size=num_beams, sampler=sampler)
            return torch.cat((input_ids.to(out.token_ids.device), out.token_ids[:, 0]), dim=1)
        sampling = dict(temperature=temperature, top_k=top_k or 0, top_p=top_p, seed=seed) if do_sample else None
        new = greedy_generate(self.model, input_ids, attention_mask, max_new_tokens, use_graph=use_graph,
                              eos_token_id=eos_token_id, pad_token_id=pad_token_id, sampling=sampling)
        return torch.cat((input_ids.to(new.device), new), dim=1)

    def get_input_embeddings(self):
        return self.model.transformer["wte"]

    def set_input_embeddings(self, value: nn.Module) -> None:  # modeling_olmo.py:175-176
        self.model.transformer["wte"] = value
        self.model._prepared = False  # tiled copies of the head are rebuilt on the next forward

    def get_output_embeddings(self):  # modeling_olmo.py:178-182: the embedding itself when the weights are tied
        if self.config.weight_tying:
            return self.model.transformer["wte"]
        return self.model.transformer["ff_out"]

    def set_output_embeddings(self, value: nn.Module) -> None:  # modeling_olmo.py:184-188
        self.model.transformer["wte" if self.config.weight_tying else "ff_out"] = value
        self.model._prepared = False

    def tie_weights(self) -> None:
        """A no-op as in the reference (modeling_olmo.py:190-202): with ``weight_tying`` the model has no ``ff_out``
        and multiplies by the embedding matrix itself."""

    def resize_token_embeddings(self, new_num_tokens: Optional[int] = None, pad_to_multiple_of: Optional[int] = None):
        raise NotImplementedError("resizing the embeddings (modeling_olmo.py:204-246) belongs to fine-tuning set-up")

"""HF wrapper: ``OLMoConfig`` and ``OLMoForCausalLM`` with the surface of
``hf_olmo/configuration_olmo.py:14-63`` and ``hf_olmo/modeling_olmo.py:41-261``.

As in the reference the classes are a ``transformers.PretrainedConfig`` and a ``PreTrainedModel`` +
``GenerationMixin`` registered with ``AutoConfig`` / ``AutoModelForCausalLM`` (``configuration_olmo.py:63``,
``modeling_olmo.py:261``), so transformers' own ``generate`` (greedy, sampling, its beam search, logits
processors, stopping criteria) drives ``forward`` + ``prepare_inputs_for_generation``.  ``forward`` passes through
to ``OLMo.forward`` (``modeling_olmo.py:84-147``).  transformers hands ``forward`` a ``Cache`` object; the keys and
values stay in this package's contiguous per-layer buffers and go back to transformers as an :class:`OLMoCache`,
a ``transformers.Cache`` whose layers are views of those buffers and whose ``reorder_cache`` / ``crop`` /
``batch_*`` act on them.  A list of ``(k, v)`` is returned, as the reference does, when the caller passed a list or
nothing.

``generate`` runs this package's captured loop (prefill, then one HIP-graph replay per token; OLMo's own beam
search for ``num_beams > 1``) when every argument is one that loop understands, and transformers' loop otherwise
or on request (``loop="transformers"``).  The module tree is ``self.model.transformer...`` so the names AutoGPTQ
addresses (``model.transformer.blocks.{i}.att_proj`` ..., ``inference/compression/olmo_gptq_class.py:6``) resolve.
Without an importable ``transformers`` the same classes are plain objects / ``nn.Module`` with the captured loop only.
"""

from __future__ import annotations

from dataclasses import asdict, fields
from typing import Any, Dict, List, NamedTuple, Optional, Tuple

import torch
import torch.nn as nn

from .config import ModelConfig
from .generate import greedy_generate
from .model import KVCache, LayerKV, OLMo

try:  # the HF surface proper needs transformers; everything else of the package does not
    from transformers import AutoConfig, AutoModelForCausalLM, GenerationMixin, PretrainedConfig, PreTrainedModel
    from transformers.cache_utils import Cache, CacheLayerMixin
    from transformers.modeling_outputs import CausalLMOutputWithPast

    HAVE_TRANSFORMERS = True
except ImportError:  # pragma: no cover - the image ships transformers
    HAVE_TRANSFORMERS = False

__all__ = ["OLMoConfig", "OLMoForCausalLM", "OLMoCache", "CausalLMOutputWithPast", "HAVE_TRANSFORMERS"]

# arguments of forward(); transformers' loop adds bookkeeping of its own to the model inputs, which is dropped
_FORWARD_KEYS = ("inputs_embeds", "attention_mask", "attention_bias", "labels", "use_cache", "output_attentions",
                 "output_hidden_states", "return_dict", "cache_position")


def _model_config_defaults() -> Dict[str, Any]:
    d = asdict(ModelConfig())
    d.pop("extra", None)
    return d


if HAVE_TRANSFORMERS:

    class OLMoConfig(PretrainedConfig):
        """``hf_olmo/configuration_olmo.py:14-59``: every ``ModelConfig`` field as an attribute, ``use_cache``
        (default False) and the HF aliases."""

        model_type = "hf_olmo"
        keys_to_ignore_at_inference = ["past_key_values"]

        def __init__(self, use_cache: bool = False, **kwargs):
            all_kwargs = _model_config_defaults()
            all_kwargs.update(kwargs)
            all_kwargs.update({"use_cache": use_cache})
            all_kwargs.update({"architectures": all_kwargs.get("architectures", ["OLMoForCausalLM"]) or ["OLMoForCausalLM"]})
            super().__init__(**all_kwargs)
            self.use_cache = use_cache  # transformers >= 5 strips generation arguments from the config's kwargs

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

        @property
        def effective_n_kv_heads(self) -> int:  # configuration_olmo.py:40-58
            return self.to_model_config().effective_n_kv_heads

    class _CacheLayerView(CacheLayerMixin):
        """One layer of an :class:`OLMoCache`: ``keys`` / ``values`` are views ``[:, :, :length]`` of the
        layer's buffers, set by the owning cache; the buffers are written by the attention kernels, never here."""

        is_sliding = False

        def __init__(self, owner: "OLMoCache"):
            super().__init__()
            self._owner = owner
            self.is_initialized = True

        def lazy_initialization(self, key_states, value_states) -> None:
            pass

        def update(self, key_states, value_states, *args, **kwargs):
            raise NotImplementedError("OLMoCache is filled by OLMo.forward, not through Cache.update")

        def get_seq_length(self) -> int:
            return self._owner.kv.length

        def get_mask_sizes(self, query_length: int) -> Tuple[int, int]:
            return self.get_seq_length() + query_length, 0

        def get_max_length(self) -> int:
            return -1  # grows like a dynamic cache as far as the caller is concerned (up to the buffers' capacity)

    class OLMoCache(Cache):
        """A ``transformers.Cache`` over a :class:`olmo_amd.model.KVCache` (contiguous per-layer buffers, keys
        stored rotated).  What transformers' generation loops do to a cache acts on the buffers: ``reorder_cache``
        (its beam search) permutes the rows in place, ``crop`` moves the length back, ``batch_repeat_interleave`` /
        ``batch_select_indices`` build buffers of the new batch size."""

        def __init__(self, kv: KVCache):
            self.kv = kv
            super().__init__(layers=[_CacheLayerView(self) for _ in kv.k])
            self.refresh()

        def refresh(self) -> "OLMoCache":
            L = self.kv.length
            for layer, k, v in zip(self.layers, self.kv.k, self.kv.v):
                layer.keys, layer.values = k[:, :, :L], v[:, :, :L]
            return self

        def legacy(self) -> List[LayerKV]:
            """The list of ``(k, v)`` views ``OLMo.forward`` takes back as ``past_key_values``."""
            return self.kv.views()

        def get_seq_length(self, layer_idx: int = 0) -> int:
            return self.kv.length

        def reset(self):
            self.kv.set_length(0)
            self.refresh()

        def reorder_cache(self, beam_idx: torch.LongTensor):
            L = self.kv.length
            if L == 0:
                return
            idx = beam_idx.to(self.kv.k[0].device)
            for t in (*self.kv.k, *self.kv.v):
                t[:, :, :L] = t[:, :, :L].index_select(0, idx)

        def crop(self, tokens_to_remove: int) -> None:
            L = self.kv.length
            new = L - abs(tokens_to_remove) if tokens_to_remove < 0 else min(tokens_to_remove, L)  # > 0: final length (legacy)
            if tokens_to_remove != 0:
                self.kv.set_length(max(new, 0))
                self.refresh()

        def _rebatch(self, pick) -> None:
            old, L = self.kv, self.kv.length
            k0 = pick(old.k[0][:, :, :L])
            new = KVCache(len(old.k), k0.shape[0], k0.shape[1], old.capacity, k0.shape[3], k0.dtype, k0.device)
            for i in range(len(old.k)):
                new.k[i][:, :, :L] = pick(old.k[i][:, :, :L])
                new.v[i][:, :, :L] = pick(old.v[i][:, :, :L])
            new.set_length(L)
            self.kv = new
            self.refresh()

        def batch_repeat_interleave(self, repeats: int):
            self._rebatch(lambda t: t.repeat_interleave(repeats, dim=0))

        def batch_select_indices(self, indices: torch.Tensor):
            self._rebatch(lambda t: t[indices.to(t.device), ...])

    _ModelBase: Tuple[type, ...] = (PreTrainedModel, GenerationMixin)

else:  # pragma: no cover

    class CausalLMOutputWithPast(NamedTuple):
        """Field names of ``transformers.modeling_outputs.CausalLMOutputWithPast``."""

        loss: Optional[torch.Tensor]
        logits: torch.Tensor
        past_key_values: Optional[List[Tuple[torch.Tensor, torch.Tensor]]]
        hidden_states: Optional[Tuple[torch.Tensor, ...]]

    class OLMoConfig:
        model_type = "hf_olmo"

        def __init__(self, use_cache: bool = False, **kwargs):
            base = _model_config_defaults()
            base.update(kwargs)
            for k, v in base.items():
                setattr(self, k, v)
            self.use_cache = use_cache
            self.architectures = base.get("architectures") or ["OLMoForCausalLM"]
            self.return_dict = True

        @classmethod
        def from_model_config(cls, mc: ModelConfig, use_cache: bool = False) -> "OLMoConfig":
            d = asdict(mc)
            d.pop("extra", None)
            return cls(use_cache=use_cache, **d)

        def to_model_config(self) -> ModelConfig:
            return ModelConfig.from_dict({f.name: getattr(self, f.name) for f in fields(ModelConfig) if f.name != "extra"})

        num_attention_heads = property(lambda self: self.n_heads)
        num_hidden_layers = property(lambda self: self.n_layers)
        hidden_size = property(lambda self: self.d_model)

    class OLMoCache:  # never constructed without transformers
        pass

    _ModelBase = (nn.Module,)


def _is_cache_object(p) -> bool:
    return p is not None and hasattr(p, "get_seq_length")


class OLMoForCausalLM(*_ModelBase):
    """``hf_olmo/modeling_olmo.py:41-246``."""

    config_class = OLMoConfig
    base_model_prefix = "model"
    _no_split_modules = ["OLMoBlock"]
    _supports_sdpa = True
    supports_gradient_checkpointing = False  # inference only

    def __init__(self, config: OLMoConfig, model: Optional[OLMo] = None, init_params: bool = False, device="cuda",
                 dtype: Optional[torch.dtype] = None, **model_kwargs):
        if HAVE_TRANSFORMERS:
            super().__init__(config)
        else:
            super().__init__()
            self.config = config
        if model is None:
            if dtype is None:  # what the directory being loaded says (``from_pretrained``), else bfloat16
                dtype = getattr(config, "dtype", None)
                dtype = dtype if dtype in (torch.bfloat16, torch.float16, torch.float32) else torch.bfloat16
            model = OLMo(config.to_model_config(), device=device, dtype=dtype, **model_kwargs)
            if init_params:
                model.reset_parameters()
        self.model = model
        if HAVE_TRANSFORMERS:
            self.post_init()  # transformers' own bookkeeping (tied-weight keys, parallel plans); initialises nothing here

    # ------------------------------------------------------------------------------------------
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
        return_dict = return_dict if return_dict is not None else self.config.return_dict

        # a transformers Cache: ours carries the buffers; an empty one means "no past"; a populated foreign one
        # holds plain (k, v) per layer in the reference's form (keys not rotated) and is taken over as such
        cache_in = past_key_values if _is_cache_object(past_key_values) else None
        if cache_in is not None:
            if isinstance(cache_in, OLMoCache):
                past_key_values = cache_in.legacy() if cache_in.kv.length > 0 else None
            elif cache_in.get_seq_length() == 0:
                past_key_values = None
            else:
                past_key_values = [(layer.keys, layer.values) for layer in cache_in.layers]
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
        kvs = outputs.attn_key_values
        if kvs is not None and cache_in is not None:  # a Cache came in, a Cache goes out
            kv = kvs[0].cache
            if isinstance(cache_in, OLMoCache) and cache_in.kv is kv:
                kvs = cache_in.refresh()
            else:
                kvs = OLMoCache(kv)
        if not return_dict:
            output = (logits, kvs, outputs.hidden_states)
            return (loss,) + output if loss is not None else output
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=kvs, hidden_states=outputs.hidden_states)

    @classmethod
    def can_generate(cls) -> bool:
        return True

    def prepare_inputs_for_generation(self, input_ids: torch.LongTensor, past_key_values=None, **kwargs):
        """``modeling_olmo.py:150-160``: with a cache only the last token is processed.  transformers >= 5 says how
        many trailing tokens are new (``next_sequence_length``); its other bookkeeping arguments are not ``forward``'s
        and are dropped."""
        n_new = kwargs.pop("next_sequence_length", None)
        if _is_cache_object(past_key_values):
            has_past = past_key_values.get_seq_length() > 0
        else:
            has_past = bool(past_key_values)
        if n_new is not None:
            input_ids = input_ids[:, -n_new:]
        elif has_past:
            input_ids = input_ids[:, -1:]
        model_inputs: Dict[str, Any] = {"input_ids": input_ids, "past_key_values": past_key_values}
        model_inputs.update({k: v for k, v in kwargs.items() if k in _FORWARD_KEYS})
        model_inputs["use_cache"] = kwargs.pop("use_cache", self.config.use_cache)
        return model_inputs

    # ------------------------------------------------------------------------------------------
    _CAPTURED_ARGS = frozenset(("attention_mask", "max_new_tokens", "do_sample", "num_beams", "eos_token_id",
                                "pad_token_id", "use_graph", "temperature", "top_k", "top_p", "seed"))

    def _route(self, input_ids, args, kwargs) -> Tuple[str, Dict[str, Any]]:
        """Which loop a ``generate`` call without ``loop=`` takes, and with which arguments.  HF's ``generate`` is the
        reference wrapper's (``hf_olmo/modeling_olmo.py`` inherits it), so whatever the captured loop would do
        differently goes to transformers: anything but plain greedy decoding of a given number of new tokens
        (sampling draws from another random stream, ``num_beams > 1`` is HF's length-normalised search there and
        OLMo's own here), several end tokens, arguments the captured loop does not know.  For the calls it keeps, the
        captured loop takes the end and padding tokens from ``generation_config`` where the call does not name
        them, as HF does, and ends once every sequence has ended."""
        if not HAVE_TRANSFORMERS:
            return "captured", kwargs
        gc = getattr(self, "generation_config", None)
        if input_ids is None or args or not set(kwargs) <= self._CAPTURED_ARGS or "max_new_tokens" not in kwargs:
            return "transformers", kwargs

        def setting(name, default):
            if name in kwargs:
                return kwargs[name]
            return default if gc is None or getattr(gc, name, None) is None else getattr(gc, name)

        if setting("do_sample", False) or setting("num_beams", 1) != 1:
            return "transformers", kwargs
        eos = setting("eos_token_id", None)
        if isinstance(eos, (list, tuple)):
            if len(eos) > 1:
                return "transformers", kwargs
            eos = eos[0] if eos else None
        filled = dict(kwargs, eos_token_id=eos, pad_token_id=setting("pad_token_id", None))
        return "captured", filled

    @torch.no_grad()
    def generate(self, input_ids: Optional[torch.LongTensor] = None, *args, loop: Optional[str] = None, **kwargs):
        """Continuation ``[B, prompt + new tokens]`` like HF ``generate``.

        ``loop="transformers"``: ``GenerationMixin.generate`` with all of its arguments, calling ``forward`` once per
        token.  ``loop="captured"``: this package's loop -- prefill, then one captured decode step per token, greedy or
        sampled on the device (temperature, top-k, top-p in HF's order; ``top_k=0`` / ``top_p=1.0`` switch a filter
        off; ``seed`` fixes the draw); ``num_beams > 1`` runs OLMo's own beam search (``olmo/beam_search.py``: summed
        log-probabilities, no length penalty, the best beam, fewer than ``max_new_tokens`` columns when every beam
        ended early) -- named explicitly, it does exactly what its arguments say and reads nothing from
        ``generation_config``.  Default (see :meth:`_route`): the captured loop for plain greedy decoding, where it
        returns the tokens HF's loop would (end and padding tokens from ``generation_config``), transformers'
        loop for everything else."""
        if loop is None:
            loop, kwargs = self._route(input_ids, args, kwargs)
            if loop == "captured" and HAVE_TRANSFORMERS:
                kwargs["_hf_stop"] = True
        if loop == "transformers":
            if not HAVE_TRANSFORMERS:
                raise RuntimeError("transformers is not importable")
            kwargs.pop("use_graph", None)
            kwargs.pop("seed", None)
            kwargs.setdefault("use_cache", True)
            return super().generate(input_ids, *args, **kwargs)
        if loop != "captured":
            raise ValueError(f"loop must be 'captured' or 'transformers', not {loop!r}")
        unknown = set(kwargs) - self._CAPTURED_ARGS - {"_hf_stop"}
        if args or unknown:
            raise TypeError(f"the captured loop does not take {sorted(unknown) or 'positional arguments'}")
        return self._generate_captured(input_ids, **kwargs)

    def _generate_captured(self, input_ids: torch.LongTensor, attention_mask: Optional[torch.Tensor] = None,
                           max_new_tokens: int = 20, do_sample: bool = False, num_beams: int = 1,
                           eos_token_id: Optional[int] = None, pad_token_id: Optional[int] = None, use_graph: bool = True,
                           temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0,
                           _hf_stop: bool = False) -> torch.Tensor:
        if num_beams != 1:
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
                                      beam_size=num_beams, sampler=sampler, use_graph=use_graph)
            return torch.cat((input_ids.to(out.token_ids.device), out.token_ids[:, 0]), dim=1)
        sampling = dict(temperature=temperature, top_k=top_k or 0, top_p=top_p, seed=seed) if do_sample else None
        new = greedy_generate(self.model, input_ids, attention_mask, max_new_tokens, use_graph=use_graph,
                              eos_token_id=eos_token_id, pad_token_id=pad_token_id, sampling=sampling,
                              stop_when_all_ended=_hf_stop)
        return torch.cat((input_ids.to(new.device), new), dim=1)

    # ------------------------------------------------------------------------------------------
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

    def tie_weights(self, *args, **kwargs) -> None:
        """A no-op as in the reference (modeling_olmo.py:190-202): with ``weight_tying`` the model has no ``ff_out``
        and multiplies by the embedding matrix itself."""

    def _init_weights(self, module) -> None:
        """Weights come from a checkpoint or from ``OLMo.reset_parameters``; transformers' own initialisation pass
        must leave them alone."""

    def resize_token_embeddings(self, new_num_tokens: Optional[int] = None, pad_to_multiple_of: Optional[int] = None):
        raise NotImplementedError("resizing the embeddings (modeling_olmo.py:204-246) belongs to fine-tuning set-up")


if HAVE_TRANSFORMERS:
    # modeling_olmo.py:258-261, configuration_olmo.py:60-63 (exist_ok: the reference's own package may be importable too)
    AutoConfig.register("hf_olmo", OLMoConfig, exist_ok=True)
    AutoModelForCausalLM.register(OLMoConfig, OLMoForCausalLM, exist_ok=True)

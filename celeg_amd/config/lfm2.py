"""Typed configuration of the LFM2 dense decoder and its translation into parts.

The reference has no class for this architecture: it recognises the layers from
tensor names (src/model/inference/rules.cpp:12-90 for the short convolution,
src/model/inference/rules_attention.cpp:138-345 for attention) and reads the
scalar keys through its metadata normaliser
(src/model/inference/metadata.cpp:350-703).  Here every size comes from
``config.json``; nothing about a particular checkpoint stands in code.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Optional, Tuple

from .spec import LayerSpec, ModelSpec, PartSpec, RunStep


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key."""


_LAYER_KINDS = ("conv", "full_attention")


def _require(cfg: Mapping[str, Any], key: str, kind):
    if key not in cfg or cfg[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    return _typed(cfg, key, kind)


def _typed(cfg: Mapping[str, Any], key: str, kind):
    value = cfg[key]
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            if isinstance(value, float) and value.is_integer():
                return int(value)
            raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
        return int(value)
    if kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"config.json: '{key}' must be a number, got {value!r}")
        return float(value)
    if kind is bool:
        if not isinstance(value, bool):
            raise ConfigError(f"config.json: '{key}' must be true or false, got {value!r}")
        return value
    raise TypeError(kind)


def _alias(cfg: Mapping[str, Any], keys: Tuple[str, ...], kind, default):
    """First present alias wins; two aliases that disagree are an error, as in the
    reference (src/model/inference/metadata.cpp:350-703 raises ConflictingMetadata)."""
    found = [(k, _typed(cfg, k, kind)) for k in keys if k in cfg and cfg[k] is not None]
    if not found:
        return default
    for k, v in found[1:]:
        if v != found[0][1]:
            raise ConfigError(f"config.json: '{found[0][0]}'={found[0][1]!r} and "
                              f"'{k}'={v!r} disagree")
    return found[0][1]


def feed_forward_width(intermediate_size: int, auto_adjust: bool, multiple_of: int,
                       multiplier: Optional[float]) -> int:
    """The SwiGLU width.  With ``block_auto_adjust_ff_dim`` the width is two thirds
    of ``intermediate_size``, times the multiplier, rounded up to a multiple of
    ``block_multiple_of``; otherwise it is ``intermediate_size`` itself.  (The
    reference takes it from the rows of w1, src/model/inference/global_facts.cpp:127-152.)"""
    if not auto_adjust:
        return intermediate_size
    width = int(2 * intermediate_size / 3)
    if multiplier is not None:
        width = int(multiplier * width)
    return multiple_of * ((width + multiple_of - 1) // multiple_of)


@dataclass(frozen=True)
class Lfm2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    layer_types: Tuple[str, ...]
    conv_L_cache: int
    conv_bias: bool
    rope_theta: float
    norm_eps: float
    max_position_embeddings: int
    block_auto_adjust_ff_dim: bool
    block_multiple_of: int
    block_ffn_dim_multiplier: Optional[float]
    tie_word_embeddings: bool
    bos_token_id: int = 0
    eos_token_ids: Tuple[int, ...] = (0,)
    pad_token_id: int = 1
    architecture: str = "Lfm2ForCausalLM"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any],
                  tensor_shapes: Optional[Mapping[str, Tuple[int, ...]]] = None) -> "Lfm2Config":
        """Keys and defaults follow src/model/inference/metadata.cpp: hidden_size
        (353), intermediate_size (355-357), num_hidden_layers (358-360),
        num_attention_heads (364-366), num_key_value_heads (367-369), head_dim
        (370), vocab_size (399), max_position_embeddings (404-406), norm_eps
        (407-409, default 1e-6 at 643), conv_L_cache (425-426), rope_theta
        (427-429: also as ``rope_parameters.rope_theta``; required 663-666),
        block_auto_adjust_ff_dim (512-514), tying (630-632), token ids (638-642).

        ``tensor_shapes`` (name -> shape of the checkpoint's tensors), when given, fills
        what config.json leaves out the way the reference does: the kind of every layer
        from the tensors it has (``conv.in_proj.weight`` or ``self_attn.q_proj.weight``,
        src/model/inference/rules.cpp:18-26, rules_attention.cpp:138-160) and the
        feed-forward width from the rows of w1 (global_facts.cpp:127-152); a
        ``layer_types`` that contradicts the tensors is an error.  The original LFM2 keys
        ``full_attn_idxs`` (the attention layers; every other layer is a convolution) and
        ``block_ff_dim`` (= intermediate_size) are read too."""
        cfg = dict(cfg)
        nested = cfg.get("rope_parameters")
        if isinstance(nested, Mapping) and nested.get("rope_theta") is not None:
            cfg["rope_parameters.rope_theta"] = nested["rope_theta"]
        vocab = _require(cfg, "vocab_size", int)
        hidden = _require(cfg, "hidden_size", int)
        layers = _require(cfg, "num_hidden_layers", int)
        heads = _require(cfg, "num_attention_heads", int)
        kv_heads = _alias(cfg, ("num_key_value_heads",), int, heads)
        head_dim = _alias(cfg, ("head_dim",), int, hidden // heads if heads > 0 else 0)
        rope_theta = _alias(cfg, ("rope_theta", "rope_parameters.rope_theta"), float, None)
        if rope_theta is None:
            raise ConfigError("config.json: required key 'rope_theta' is missing")
        conv_l = _require(cfg, "conv_L_cache", int)
        max_pos = _require(cfg, "max_position_embeddings", int)
        auto_adjust = _alias(cfg, ("block_auto_adjust_ff_dim",), bool, False)
        intermediate = _alias(cfg, ("intermediate_size", "block_ff_dim"), int, None)
        kinds = cls._layer_kinds(cfg, layers, tensor_shapes)
        if intermediate is None:
            w1 = (tensor_shapes or {}).get("model.layers.0.feed_forward.w1.weight")
            if w1 is None:
                raise ConfigError("config.json: required key 'intermediate_size' is missing")
            # the width itself: no adjustment is applied to a size read off the weights
            intermediate, auto_adjust = int(w1[0]), False
        eos = cfg.get("eos_token_id", 0)
        if isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        if "block_ffn_dim_multiplier" not in cfg:
            multiplier = 1.0
        elif cfg["block_ffn_dim_multiplier"] is None:
            multiplier = None
        else:
            multiplier = _typed(cfg, "block_ffn_dim_multiplier", float)
        out = cls(
            vocab_size=vocab, hidden_size=hidden, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            intermediate_size=intermediate, layer_types=tuple(kinds),
            conv_L_cache=conv_l,
            conv_bias=_alias(cfg, ("conv_bias",), bool, False),
            rope_theta=rope_theta,
            norm_eps=_alias(cfg, ("norm_eps", "rms_norm_eps"), float, 1e-6),
            max_position_embeddings=max_pos,
            block_auto_adjust_ff_dim=auto_adjust,
            block_multiple_of=_alias(cfg, ("block_multiple_of",), int, 256),
            block_ffn_dim_multiplier=multiplier,
            tie_word_embeddings=_alias(cfg, ("tie_word_embeddings", "tie_embedding"), bool, True),
            bos_token_id=_alias(cfg, ("bos_token_id",), int, 0),
            eos_token_ids=eos_ids,
            pad_token_id=_alias(cfg, ("pad_token_id",), int, 1),
        )
        out.validate()
        return out

    @staticmethod
    def _layer_kinds(cfg, layers: int, tensor_shapes) -> Tuple[str, ...]:
        """``layer_types`` if given; else from ``full_attn_idxs``; else from the tensors each
        layer has.  Whatever the source, tensors that say otherwise are an error."""
        from_tensors = None
        if tensor_shapes is not None:
            from_tensors = []
            for i in range(layers):
                conv = f"model.layers.{i}.conv.in_proj.weight" in tensor_shapes
                attn = f"model.layers.{i}.self_attn.q_proj.weight" in tensor_shapes
                from_tensors.append("conv" if conv and not attn else
                                    "full_attention" if attn and not conv else None)
        kinds = cfg.get("layer_types")
        if kinds is not None:
            if not isinstance(kinds, (list, tuple)) or not all(isinstance(k, str) for k in kinds):
                raise ConfigError("config.json: 'layer_types' must be a list of strings")
            kinds = tuple(kinds)
        elif cfg.get("full_attn_idxs") is not None:
            idxs = cfg["full_attn_idxs"]
            if not isinstance(idxs, (list, tuple)) or \
                    not all(isinstance(i, int) and not isinstance(i, bool) for i in idxs):
                raise ConfigError("config.json: 'full_attn_idxs' must be a list of integers")
            if any(not 0 <= i < layers for i in idxs):
                raise ConfigError(f"config.json: 'full_attn_idxs' names a layer outside [0, {layers})")
            kinds = tuple("full_attention" if i in set(idxs) else "conv" for i in range(layers))
        elif from_tensors is not None:
            unknown = [i for i, k in enumerate(from_tensors) if k is None]
            if unknown:
                raise ConfigError("config.json has no 'layer_types' and the tensors of layer(s) "
                                  f"{unknown} tell neither a convolution nor an attention layer")
            return tuple(from_tensors)
        else:
            raise ConfigError("config.json: required key 'layer_types' is missing")
        if from_tensors is not None and len(kinds) == layers:
            for i, (said, found) in enumerate(zip(kinds, from_tensors)):
                if found is not None and said in _LAYER_KINDS and said != found:
                    raise ConfigError(f"config.json: 'layer_types'[{i}] is {said!r} but the "
                                      f"checkpoint's tensors of layer {i} are those of {found!r}")
        return kinds

    def validate(self) -> None:
        """GQA divisibility, even head size and kv width as in
        src/model/inference/rules_attention.cpp:194-204; positive cache length as
        in src/model/inference/rules.cpp:36-40."""
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                    "num_key_value_heads", "head_dim", "intermediate_size", "conv_L_cache",
                    "max_position_embeddings", "block_multiple_of"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive, got {getattr(self, key)}")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(f"config.json: 'layer_types' has {len(self.layer_types)} entries "
                              f"but 'num_hidden_layers' is {self.num_hidden_layers}")
        for i, kind in enumerate(self.layer_types):
            if kind not in _LAYER_KINDS:
                raise ConfigError(f"config.json: 'layer_types'[{i}] is {kind!r}; "
                                  f"known kinds are {list(_LAYER_KINDS)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError("config.json: 'num_attention_heads' must be a multiple of "
                              "'num_key_value_heads'")
        if self.head_dim % 2:
            raise ConfigError("config.json: 'head_dim' must be even")
        if self.num_key_value_heads * self.head_dim > self.hidden_size:
            raise ConfigError("config.json: 'num_key_value_heads' * 'head_dim' exceeds 'hidden_size'")
        if not self.rope_theta > 0:
            raise ConfigError("config.json: 'rope_theta' must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("config.json: 'norm_eps' must be positive")
        if self.block_ffn_dim_multiplier is not None and not self.block_ffn_dim_multiplier > 0:
            raise ConfigError("config.json: 'block_ffn_dim_multiplier' must be positive")

    # ------------------------------------------------------------------ derived
    @property
    def ff_dim(self) -> int:
        return feed_forward_width(self.intermediate_size, self.block_auto_adjust_ff_dim,
                                  self.block_multiple_of, self.block_ffn_dim_multiplier)

    def to_dict(self) -> Dict[str, Any]:
        """The keys of config.json that this class reads, for a written model folder."""
        return {
            "architectures": [self.architecture],
            "model_type": "lfm2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "layer_types": list(self.layer_types),
            "conv_L_cache": self.conv_L_cache,
            "conv_bias": self.conv_bias,
            "rope_theta": self.rope_theta,
            "norm_eps": self.norm_eps,
            "max_position_embeddings": self.max_position_embeddings,
            "block_auto_adjust_ff_dim": self.block_auto_adjust_ff_dim,
            "block_multiple_of": self.block_multiple_of,
            "block_ffn_dim_multiplier": self.block_ffn_dim_multiplier,
            "tie_word_embeddings": self.tie_word_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": list(self.eos_token_ids) if len(self.eos_token_ids) != 1
            else self.eos_token_ids[0],
            "pad_token_id": self.pad_token_id,
        }

    # ------------------------------------------------------------------ parts
    def to_spec(self) -> ModelSpec:
        """Tensor names: embedding and head src/model/inference/global_facts.cpp:41-73
        and layer_bindings.cpp:24-154; norms layer_bindings.cpp:276-303; short
        convolution src/model/inference/support.cpp:114-123; attention
        support.cpp:57-78 and rules_attention.cpp:72-92; feed-forward
        layer_bindings.cpp:439-473."""
        H = self.hidden_size
        norm = lambda name: PartSpec("rmsnorm", {"width": H, "eps": self.norm_eps},
                                     {"weight": name})
        layers = []
        for i, kind in enumerate(self.layer_types):
            p = f"model.layers.{i}."
            if kind == "conv":
                tensors = {"in_proj": p + "conv.in_proj.weight",
                           "conv": p + "conv.conv.weight",
                           "out_proj": p + "conv.out_proj.weight"}
                if self.conv_bias:
                    tensors.update({"in_proj_bias": p + "conv.in_proj.bias",
                                    "conv_bias": p + "conv.conv.bias",
                                    "out_proj_bias": p + "conv.out_proj.bias"})
                mixer = PartSpec("short_conv",
                                 {"width": H, "taps": self.conv_L_cache, "bias": self.conv_bias},
                                 tensors)
            else:
                mixer = PartSpec(
                    "gqa_attention",
                    {"width": H, "heads": self.num_attention_heads,
                     "kv_heads": self.num_key_value_heads, "head_dim": self.head_dim,
                     "qk_norm": True, "eps": self.norm_eps, "window": None,
                     "position": PartSpec("rope", {"theta": self.rope_theta,
                                                   "rotary_dim": self.head_dim,
                                                   "head_dim": self.head_dim})},
                    {"q_proj": p + "self_attn.q_proj.weight",
                     "k_proj": p + "self_attn.k_proj.weight",
                     "v_proj": p + "self_attn.v_proj.weight",
                     "out_proj": p + "self_attn.out_proj.weight",
                     "q_norm": p + "self_attn.q_layernorm.weight",
                     "k_norm": p + "self_attn.k_layernorm.weight"})
            ffn = PartSpec("swiglu", {"width": H, "ff": self.ff_dim},
                           {"gate": p + "feed_forward.w1.weight",
                            "up": p + "feed_forward.w3.weight",
                            "down": p + "feed_forward.w2.weight"})
            layers.append(LayerSpec(mixer=mixer, mixer_norm=norm(p + "operator_norm.weight"),
                                    ffn=ffn, ffn_norm=norm(p + "ffn_norm.weight")))
        embedding = PartSpec("embedding", {"vocab": self.vocab_size, "width": H},
                             {"table": "model.embed_tokens.weight"})
        if self.tie_word_embeddings:
            head = PartSpec("tied_head", {"vocab": self.vocab_size, "width": H}, {})
        else:
            head = PartSpec("linear_head", {"vocab": self.vocab_size, "width": H},
                            {"weight": "lm_head.weight"})
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=H,
            max_context=self.max_position_embeddings, embedding=embedding,
            layers=tuple(layers),
            order=tuple(RunStep(i) for i in range(self.num_hidden_layers)),
            final_norm=norm("model.embedding_norm.weight"), head=head,
            eos_token_ids=self.eos_token_ids, bos_token_id=self.bos_token_id)
        spec.validate()
        return spec

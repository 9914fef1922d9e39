"""Typed configuration of LFM2 (`Lfm2ForCausalLM`, model_type `lfm2`).

Keys, their precedence and defaults follow the reference's family spec
(arch/families/lfm2.json5:27-57).  Where the reference decides by
which tensors a checkpoint holds (layer kind :78-80, tied head :91, vocabulary :35),
the same rule is used when the tensor table of the checkpoint is at hand, and
config.json's own keys (`layer_types`, `full_attn_idxs`, `tie_embedding`) otherwise.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Sequence, Tuple

from .base import ArchConfig, ConfigError, first, require
from .spec import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec,
                   PositionSpec)

CONV = "conv"
ATTENTION = "full_attention"


def feed_forward_width(ff_raw: int, auto_adjust: bool, multiplier: float, multiple_of: int) -> int:
    """The SwiGLU width (lfm2.json5:38-41): with `block_auto_adjust_ff_dim`, two thirds of
    the raw width, rounded up to `block_multiple_of` only when a multiplier is given
    (`int()` truncates, src/arch/expr.rs:820); else the raw width."""
    if not auto_adjust:
        return ff_raw
    ff_23 = ff_raw * 2 // 3
    if multiplier > 0:
        return multiple_of * math.ceil(int(multiplier * ff_23) / multiple_of)
    return ff_23


@dataclass(frozen=True)
class Lfm2Config(ArchConfig):
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    ff_raw: int                         # intermediate_size | block_ff_dim | 4 * hidden
    ff_raw_key: str                     # which key gave it (kept for to_dict)
    block_auto_adjust_ff_dim: bool
    block_ffn_dim_multiplier: float     # 0 = absent
    block_multiple_of: int
    norm_eps: float
    rope_theta: float
    conv_L_cache: int
    conv_bias: bool
    max_position_embeddings: int
    layer_types: Tuple[str, ...]
    tie_embedding: bool
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    architecture = "Lfm2ForCausalLM"

    # ------------------------------------------------------------------ derived sizes
    @property
    def intermediate_size(self) -> int:
        return feed_forward_width(self.ff_raw, self.block_auto_adjust_ff_dim,
                                  self.block_ffn_dim_multiplier, self.block_multiple_of)

    @property
    def full_attn_idxs(self) -> Tuple[int, ...]:
        return tuple(i for i, t in enumerate(self.layer_types) if t == ATTENTION)

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any],
                  tensors: Optional[Mapping[str, Sequence[int]]] = None) -> "Lfm2Config":
        """`tensors` (name -> shape of the checkpoint), when given, decides what the
        reference decides by tensor presence."""
        hidden = int(require(cfg, "hidden_size"))
        layers = int(require(cfg, "num_hidden_layers"))
        heads = int(require(cfg, "num_attention_heads", "num_heads"))
        kv_heads = int(first(cfg, "num_key_value_heads", default=heads))
        head_dim = int(first(cfg, "head_dim", default=hidden // heads))
        embed = tensors.get("model.embed_tokens.weight") if tensors else None
        vocab = int(embed[0]) if embed is not None else int(require(cfg, "vocab_size"))
        ff_key = "intermediate_size" if first(cfg, "intermediate_size") is not None else (
            "block_ff_dim" if first(cfg, "block_ff_dim") is not None else "")
        ff_raw = int(first(cfg, "intermediate_size", "block_ff_dim", default=4 * hidden))
        conv_k = first(cfg, "conv_L_cache")
        if conv_k is None or int(conv_k) < 2:
            raise ConfigError(f"LFM2 short-conv kernel (conv_L_cache) {conv_k} must be >= 2")
        if heads % kv_heads:
            raise ConfigError(f"num_attention_heads {heads} is not a multiple of num_key_value_heads {kv_heads}")

        layer_types = cls._layer_types(cfg, layers, tensors)
        tie = first(cfg, "tie_embedding", "tie_word_embeddings")
        if tensors is not None:
            tie = "lm_head.weight" not in tensors
        elif tie is None:
            tie = True
        eos = first(cfg, "eos_token_id", default=())
        eos = tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        bos = first(cfg, "bos_token_id")
        return cls(
            hidden_size=hidden, num_hidden_layers=layers, num_attention_heads=heads,
            num_key_value_heads=kv_heads, head_dim=head_dim, vocab_size=vocab,
            ff_raw=ff_raw, ff_raw_key=ff_key,
            block_auto_adjust_ff_dim=first(cfg, "block_auto_adjust_ff_dim", default=False) is True,
            block_ffn_dim_multiplier=float(first(cfg, "block_ffn_dim_multiplier", default=0)),
            block_multiple_of=int(first(cfg, "block_multiple_of", default=256)),
            norm_eps=float(first(cfg, "norm_eps", "rms_norm_eps", default=1e-5)),
            rope_theta=float(first(cfg, "rope_theta", "rope_parameters.rope_theta", default=10000)),
            conv_L_cache=int(conv_k), conv_bias=first(cfg, "conv_bias", default=False) is True,
            max_position_embeddings=int(first(cfg, "max_position_embeddings", default=2048)),
            layer_types=layer_types, tie_embedding=bool(tie), eos_token_ids=eos,
            bos_token_id=None if bos is None else int(bos))

    @staticmethod
    def _layer_types(cfg, layers, tensors) -> Tuple[str, ...]:
        from_types = first(cfg, "layer_types")
        from_idxs = first(cfg, "full_attn_idxs")
        kinds = None
        if from_types is not None:
            if len(from_types) != layers:
                raise ConfigError(f"layer_types has {len(from_types)} entries for {layers} layers")
            for t in from_types:
                if t not in (CONV, ATTENTION):
                    raise ConfigError(f"layer_types entry {t!r} is neither {CONV!r} nor {ATTENTION!r}")
            kinds = tuple(from_types)
        if from_idxs is not None:
            bad = [i for i in from_idxs if not 0 <= int(i) < layers]
            if bad:
                raise ConfigError(f"full_attn_idxs {bad} outside 0..{layers - 1}")
            idx = {int(i) for i in from_idxs}
            by_idx = tuple(ATTENTION if i in idx else CONV for i in range(layers))
            if kinds is not None and kinds != by_idx:
                raise ConfigError("layer_types and full_attn_idxs disagree")
            kinds = by_idx
        if tensors is not None:
            by_tensor = tuple(CONV if f"model.layers.{i}.conv.in_proj.weight" in tensors else ATTENTION
                              for i in range(layers))
            if kinds is None:
                kinds = by_tensor
            elif kinds != by_tensor:
                # (a layer without the convolution's in-projection counts as attention, as the reference's
                # spec decides it, arch/families/lfm2.json5:78-80)
                wrong = [i for i in range(layers) if kinds[i] != by_tensor[i]]
                raise ConfigError(
                    "config.json and the checkpoint's tensors disagree about the kind of layers "
                    f"{wrong}: config.json says {[kinds[i] for i in wrong]}, the tensors say {[by_tensor[i] for i in wrong]}")
        if kinds is None:
            raise ConfigError("config.json lacks layer_types / full_attn_idxs")
        return kinds

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> dict:
        d = {
            "architectures": [self.architecture], "model_type": "lfm2",
            "hidden_size": self.hidden_size, "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "block_auto_adjust_ff_dim": self.block_auto_adjust_ff_dim,
            "block_multiple_of": self.block_multiple_of,
            "norm_eps": self.norm_eps, "rope_theta": self.rope_theta,
            "conv_L_cache": self.conv_L_cache, "conv_bias": self.conv_bias,
            "max_position_embeddings": self.max_position_embeddings,
            "layer_types": list(self.layer_types), "full_attn_idxs": list(self.full_attn_idxs),
            "tie_embedding": self.tie_embedding,
        }
        d[self.ff_raw_key or "block_ff_dim"] = self.ff_raw
        if self.block_ffn_dim_multiplier > 0:
            d["block_ffn_dim_multiplier"] = self.block_ffn_dim_multiplier
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d

    # ------------------------------------------------------------------ the model it describes
    def model_spec(self) -> ModelSpec:
        """Pre-norm decoder (lfm2.json5:66-95): RMSNorm -> short conv or attention ->
        residual -> RMSNorm -> SwiGLU -> residual; final norm `embedding_norm`."""
        H, hd = self.hidden_size, self.head_dim
        rope = PositionSpec("rope", {"variant": "half_split", "rotary_dim": hd, "theta": self.rope_theta,
                                     "precision": "f32"})                      # lfm2.json5:45-47,64
        layers = []
        for i, kind in enumerate(self.layer_types):
            p = f"model.layers.{i}"
            if kind == CONV:
                tensors = {"in_proj": f"{p}.conv.in_proj.weight", "conv": f"{p}.conv.conv.weight",
                           "out_proj": f"{p}.conv.out_proj.weight"}
                if self.conv_bias:
                    tensors["conv_bias"] = f"{p}.conv.conv.bias"
                mixer = MixerSpec("short_conv", {"width": H, "kernel": self.conv_L_cache,
                                                 "bias": self.conv_bias}, tensors)
            else:
                mixer = MixerSpec("attention", {
                    "heads": self.num_attention_heads, "kv_heads": self.num_key_value_heads,
                    "head_dim": hd, "scale": 1.0 / math.sqrt(hd),                 # lfm2.json5:48
                    "qk_norm": "before", "qk_norm_eps": self.norm_eps, "window": None,
                }, {"q_proj": f"{p}.self_attn.q_proj.weight", "k_proj": f"{p}.self_attn.k_proj.weight",
                    "v_proj": f"{p}.self_attn.v_proj.weight", "out_proj": f"{p}.self_attn.out_proj.weight",
                    "q_norm": f"{p}.self_attn.q_layernorm.weight",
                    "k_norm": f"{p}.self_attn.k_layernorm.weight"}, position=rope)
            ffn = FeedForwardSpec("glu", {"inter": self.intermediate_size, "activation": "silu"},
                                  {"gate": f"{p}.feed_forward.w1.weight", "up": f"{p}.feed_forward.w3.weight",
                                   "down": f"{p}.feed_forward.w2.weight"})
            layers.append(LayerSpec(p, "pre_norm",
                                    NormSpec("rms", self.norm_eps, f"{p}.operator_norm.weight"), mixer,
                                    NormSpec("rms", self.norm_eps, f"{p}.ffn_norm.weight"), ffn))
        return ModelSpec(
            architecture=self.architecture, hidden=H, vocab=self.vocab_size, layers=tuple(layers),
            order=tuple(range(len(layers))), embedding="model.embed_tokens.weight",
            final_norm=NormSpec("rms", self.norm_eps, "model.embedding_norm.weight"),
            head=None if self.tie_embedding else "lm_head.weight",
            max_position=self.max_position_embeddings, eos_token_ids=self.eos_token_ids,
            bos_token_id=self.bos_token_id)

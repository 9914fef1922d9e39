"""Configuration and registry (no GPU)."""
import pytest

from gibbs_amd.config import (ConfigError, Lfm2Config, config_from_dict, find_architecture, register_architecture)
from gibbs_amd.config.base import ArchConfig
from tests import helpers as H

BASE = dict(architectures=["Lfm2ForCausalLM"], hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
            vocab_size=100, conv_L_cache=3, layer_types=["conv", "full_attention"])


def test_keys_precedence_and_defaults():
    c = config_from_dict(BASE)
    assert isinstance(c, Lfm2Config)
    assert (c.num_key_value_heads, c.head_dim, c.intermediate_size) == (4, 16, 256)     # defaults: nh, H/nh, 4H
    assert (c.norm_eps, c.rope_theta, c.max_position_embeddings) == (1e-5, 10000.0, 2048)
    assert c.tie_embedding and not c.conv_bias and c.block_multiple_of == 256
    c = config_from_dict({**BASE, "num_heads": 8, "num_attention_heads": None, "rms_norm_eps": 1e-6,
                          "rope_parameters": {"rope_theta": 5e5}, "intermediate_size": 99, "block_ff_dim": 500})
    assert (c.num_attention_heads, c.head_dim, c.norm_eps, c.rope_theta, c.intermediate_size) == (8, 8, 1e-6, 5e5, 99)
    c = config_from_dict({**BASE, "norm_eps": 1e-4, "rms_norm_eps": 1e-6, "rope_theta": 7.0,
                          "rope_parameters": {"rope_theta": 9.0}})
    assert (c.norm_eps, c.rope_theta) == (1e-4, 7.0)                                  # the first key wins


@pytest.mark.parametrize("raw,kw,want", [
    (12288, dict(block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0), 8192),
    (6656, dict(block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0), 4608),
    (10752, dict(block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0), 7168),
    (384, dict(block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0, block_multiple_of=64), 256),
    (6656, dict(block_auto_adjust_ff_dim=True), 4437),
    (384, dict(block_auto_adjust_ff_dim=False), 384),
])
def test_feed_forward_width_rule(raw, kw, want):
    assert config_from_dict({**BASE, "block_ff_dim": raw, **kw}).intermediate_size == want


def test_layer_kinds():
    assert config_from_dict({**BASE, "layer_types": None, "full_attn_idxs": [0]}).layer_types == ("full_attention", "conv")
    with pytest.raises(ConfigError, match="disagree"):
        config_from_dict({**BASE, "full_attn_idxs": [0]})
    with pytest.raises(ConfigError, match="neither"):
        config_from_dict({**BASE, "layer_types": ["conv", "sliding"]})
    with pytest.raises(ConfigError, match="2 layers|entries"):
        config_from_dict({**BASE, "layer_types": ["conv"]})
    with pytest.raises(ConfigError, match="lacks layer_types"):
        config_from_dict({**BASE, "layer_types": None})
    # with the checkpoint's table at hand, tensor presence decides, as in the reference
    tensors = {"model.embed_tokens.weight": (77, 64), "model.layers.1.conv.in_proj.weight": (192, 64),
               "lm_head.weight": (77, 64)}
    c = Lfm2Config.from_dict({**BASE, "layer_types": None}, tensors)
    assert c.layer_types == ("full_attention", "conv") and c.vocab_size == 77 and not c.tie_embedding
    # config.json names the kinds and the checkpoint holds other layers: one error that names them
    with pytest.raises(ConfigError, match=r"disagree about the kind of layers \[0, 1\].*'conv', 'full_attention'.*'full_attention', 'conv'"):
        Lfm2Config.from_dict(BASE, tensors)
    assert Lfm2Config.from_dict({**BASE, "layer_types": ["full_attention", "conv"]}, tensors).layer_types == c.layer_types


def test_refusals():
    with pytest.raises(ConfigError, match=r"conv_L_cache\) 1 must be >= 2"):
        config_from_dict({**BASE, "conv_L_cache": 1})
    with pytest.raises(ConfigError, match="lacks hidden_size"):
        config_from_dict({k: v for k, v in BASE.items() if k != "hidden_size"})
    with pytest.raises(ConfigError, match="not a multiple"):
        config_from_dict({**BASE, "num_key_value_heads": 3})


def test_registry():
    assert find_architecture({"model_type": "lfm2"}).name == "Lfm2ForCausalLM"
    assert find_architecture({"architectures": ["Other", "Lfm2ForCausalLM"]}).name == "Lfm2ForCausalLM"
    assert find_architecture({"architectures": ["LlamaForCausalLM"]}, arch="lfm2").name == "Lfm2ForCausalLM"
    with pytest.raises(ConfigError, match="no architecture spec matches this checkpoint"):
        find_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(ConfigError, match="unknown architecture"):
        find_architecture({}, arch="nope")

    class Toy(ArchConfig):
        architecture = "ToyForCausalLM"

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls()
    register_architecture("ToyForCausalLM", Toy, aliases=("toy",))
    assert isinstance(config_from_dict({"model_type": "toy"}), Toy)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_round_trip_and_spec(name):
    c = config_from_dict(H.TINY[name])
    assert Lfm2Config.from_dict(c.to_dict()) == c
    spec = c.model_spec()
    assert len(spec.layers) == c.num_hidden_layers and spec.order == tuple(range(c.num_hidden_layers))
    kinds = [l.mixer.kind for l in spec.layers]
    assert kinds == ["attention" if t == "full_attention" else "short_conv" for t in c.layer_types]
    assert (spec.head is None) == c.tie_embedding
    attn = next(l.mixer for l in spec.layers if l.mixer.kind == "attention")
    assert abs(attn.params["scale"] - c.head_dim ** -0.5) < 1e-15 and attn.position.params["theta"] == c.rope_theta
    assert all(l.ffn.params["inter"] == c.intermediate_size for l in spec.layers)


def test_1p2b_shape_and_parameter_count():
    c = config_from_dict(dict(architectures=["Lfm2ForCausalLM"], hidden_size=2048, num_hidden_layers=16,
                              num_attention_heads=32, num_key_value_heads=8, vocab_size=65536, block_ff_dim=12288,
                              block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0, conv_L_cache=3,
                              full_attn_idxs=[2, 5, 8, 10, 12, 14], rope_theta=1e6, max_position_embeddings=128000))
    assert (c.head_dim, c.intermediate_size, len(c.full_attn_idxs)) == (64, 8192, 6)
    from gibbs_amd.parts import DecoderModel
    decls = DecoderModel(c.model_spec()).tensor_decls()
    n = sum(int(__import__("numpy").prod(d.shape)) for d in decls)
    assert n == 1_170_340_608

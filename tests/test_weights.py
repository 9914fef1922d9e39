"""Weights: the container, the declared-tensor check and its one error, random-weights mode."""
import json
import os

import numpy as np
import pytest
import torch

from gibbs_amd.config import config_from_dict
from gibbs_amd.parts import DecoderModel
from gibbs_amd.weights import (TensorDecl, WeightError, check_table, load_weights, open_checkpoint, table_of,
                               write_random_model, write_safetensors)
from tests import helpers as H
from tests.plain import golden_fixture as G
from tests.plain import lfm2_plain as P


def test_container_round_trip(tmp_path):
    t = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.randn(5).to(torch.bfloat16),
         "c": torch.tensor([[1, 2], [3, 4]], dtype=torch.int32)}
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), t)
    table, files = open_checkpoint(str(tmp_path / "m"))
    assert {n: (e.dtype, e.shape) for n, e in table.items()} == {"a": ("F32", (2, 3)), "b": ("BF16", (5,)), "c": ("I32", (2, 2))}
    for n, e in table.items():
        assert torch.equal(files[e.file].read(n), t[n])
    # the plain reader (written from the reference's description of the layout) agrees
    plain = P.read_safetensors(str(tmp_path / "m" / "model.safetensors"))
    np.testing.assert_array_equal(plain["b"], t["b"].double().numpy())
    # and a file written in the reference's test-writer manner is read by ours
    G.write_safetensors_f32(str(tmp_path / "m" / "model.safetensors"), {"x": np.ones((3, 2), np.float32)})
    assert table_of(str(tmp_path / "m")) == {"x": (3, 2)}
    with open(tmp_path / "m" / "model.safetensors", "wb") as f:
        f.write(b"\x05")
    with pytest.raises(ValueError, match="not a safetensors file"):
        open_checkpoint(str(tmp_path / "m"))


def test_sharded_index(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}, f)
    assert table_of(str(tmp_path)) == {"a": (2,), "b": (3,)}


def test_one_error_lists_everything(tmp_path):
    decls = [TensorDecl("w.q", (4, 8)), TensorDecl("w.k", (2, 8)), TensorDecl("norm", (8,), init="gain"),
             TensorDecl("conv", (8, 1, 3), alt_shapes=((8, 3),))]
    table = {"w.q": (4, 8), "norm": (9,), "conv": (8, 3), "stray.a": (1,), "stray.b": (2, 2)}
    with pytest.raises(WeightError) as ei:
        check_table(decls, table, "somewhere")
    e = ei.value
    assert e.missing == ["w.k"] and e.unexpected == ["stray.a", "stray.b"] and e.wrong_shape == [("norm", (9,), (8,))]
    msg = str(e)
    for needle in ("missing tensors (1): w.k", "no part reads (2): stray.a, stray.b", "norm is [9], expected [8]"):
        assert needle in msg
    check_table(decls, {"w.q": (4, 8), "w.k": (2, 8), "norm": (8,), "conv": (8, 1, 3)})     # fits: no error


@pytest.mark.parametrize("name", ["A", "B"])
def test_random_weights_mode(tmp_path, name):
    d = H.make_model_dir(str(tmp_path), name, seed=3)
    cfg = config_from_dict(json.load(open(os.path.join(d, "config.json"))), tensors=table_of(d))
    assert cfg == config_from_dict(H.TINY[name])
    model = DecoderModel(cfg.model_spec())
    table, _ = open_checkpoint(d)
    check_table(model.tensor_decls(), {n: e.shape for n, e in table.items()})
    # matrices bfloat16, gains and biases float32
    assert table["model.layers.0.feed_forward.w1.weight"].dtype == "BF16"
    assert table["model.embedding_norm.weight"].dtype == "F32"
    # the same seed gives the same tensors whatever the order; another seed gives others
    d2 = H.make_model_dir(str(tmp_path / "again"), name, seed=3)
    d3 = H.make_model_dir(str(tmp_path / "other"), name, seed=4)
    a, b, c = (P.read_safetensors(os.path.join(x, "model.safetensors")) for x in (d, d2, d3))
    assert all(np.array_equal(a[k], b[k]) for k in a)
    assert not np.array_equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    w = a["model.layers.1.feed_forward.w2.weight"]
    assert abs(w.std() - 0.1) < 0.01 and abs(w.mean()) < 0.01
    gains = a["model.layers.1.ffn_norm.weight"]
    assert (np.all(gains == 1.0)) == (H.GAIN_STD[name] == 0.0)


def test_load_dtype_policy_and_errors(tmp_path):
    d = H.make_model_dir(str(tmp_path), "B", seed=1)
    cfg = config_from_dict(H.TINY["B"])
    decls = DecoderModel(cfg.model_spec()).tensor_decls()
    for dtype in (torch.float32, torch.bfloat16):
        ws = load_weights(d, decls, dtype, "cpu")
        assert ws["model.layers.0.self_attn.q_proj.weight"].dtype == dtype          # matrices: compute dtype
        assert ws["model.layers.0.operator_norm.weight"].dtype == torch.float32     # rank 1: float32
        assert ws["model.layers.1.conv.conv.weight"].dtype == torch.float32         # pinned by its part
        assert ws["model.layers.1.conv.conv.weight"].shape == (96, 1, 4)
    # a checkpoint of another shape fails once, naming everything
    other = config_from_dict({**H.TINY["B"], "num_hidden_layers": 5, "full_attn_idxs": [0, 3], "hidden_size": 64,
                              "num_attention_heads": 2})
    with pytest.raises(WeightError) as ei:
        load_weights(d, DecoderModel(other.model_spec()).tensor_decls(), torch.float32, "cpu")
    assert "model.layers.5.feed_forward.w1.weight" in ei.value.unexpected
    assert any(n == "model.embed_tokens.weight" for n, _, _ in ei.value.wrong_shape)
    assert "model.layers.2.conv.in_proj.weight" in ei.value.missing        # layer 2 is a conv layer there
    assert "model.layers.2.self_attn.q_proj.weight" in ei.value.unexpected


def test_golden_fixture_loads(tmp_path):
    """The reference's fixture (all float32, config with `intermediate_size` and `layer_types`)."""
    G.write_golden_model(str(tmp_path / "g"))
    cfg = config_from_dict(G.golden_config(), tensors=table_of(str(tmp_path / "g")))
    assert cfg.layer_types == ("conv", "full_attention", "conv") and cfg.intermediate_size == 64 and cfg.tie_embedding
    ws = load_weights(str(tmp_path / "g"), DecoderModel(cfg.model_spec()).tensor_decls(), torch.float32, "cpu")
    np.testing.assert_array_equal(ws["model.embed_tokens.weight"].numpy(), G.golden_weights()["model.embed_tokens.weight"])

"""Shared pieces of the tests: tiny LFM2 configurations that differ in every size and option,
model folders made from them in temporary directories, and comparisons with the plain
implementation."""
from __future__ import annotations

import os

import numpy as np

from tests.plain import lfm2_plain as P

# Tiny A: GQA 2:1, head size 16, no auto-adjust, tied head, K 3, no conv bias, theta 1e4,
# eps 1e-5, layer kinds through `layer_types`, norm gains 1.
TINY_A = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 4, "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "block_ff_dim": 128, "block_auto_adjust_ff_dim": False, "vocab_size": 256, "tie_embedding": True,
    "conv_L_cache": 3, "conv_bias": False, "rope_theta": 10000.0, "norm_eps": 1e-5,
    "max_position_embeddings": 512,
}
# Tiny B: MQA 3:1, head size 32, width 384 auto-adjusted to 256 (multiple of 64), untied head,
# K 4, conv bias, theta 1e6, eps 1e-6, layer kinds through `full_attn_idxs`, gains 1 + N(0, 0.1).
TINY_B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 6, "full_attn_idxs": [0, 2, 5],
    "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "block_ff_dim": 384, "block_auto_adjust_ff_dim": True, "block_ffn_dim_multiplier": 1.0,
    "block_multiple_of": 64, "vocab_size": 512, "tie_embedding": False,
    "conv_L_cache": 4, "conv_bias": True, "rope_theta": 1000000.0, "norm_eps": 1e-6,
    "max_position_embeddings": 1024,
}
# Tiny C: no size is a power of two: 7 heads of 48 on a width of 112 (so heads * head size is not
# the width), 7 kv heads (no grouping), width 200, vocabulary 331, K 2.
TINY_C = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 3, "layer_types": ["full_attention", "conv", "full_attention"],
    "hidden_size": 112, "num_attention_heads": 7, "num_key_value_heads": 7, "head_dim": 48,
    "intermediate_size": 200, "block_auto_adjust_ff_dim": False, "vocab_size": 331, "tie_embedding": False,
    "conv_L_cache": 2, "conv_bias": True, "rope_theta": 500000.0, "norm_eps": 1e-6,
    "max_position_embeddings": 2048,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
GAIN_STD = {"A": 0.0, "B": 0.1, "C": 0.1}


def make_model_dir(folder: str, name: str, seed: int = 0, std: float = 0.1, dtype: str = "bfloat16") -> str:
    """Writes tiny model `name` through the framework's random-weights mode.  Matrices are stored
    in bfloat16 so that the 32-bit path, the bfloat16 path and the plain implementation all start
    from the same values."""
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    cfg = config_from_dict(TINY[name])
    decls = DecoderModel(cfg.model_spec()).tensor_decls()
    path = os.path.join(folder, f"tiny_{name}_{seed}")
    write_random_model(path, cfg, decls, seed=seed, dtype=dtype, std=std, gain_std=GAIN_STD[name], bias_std=0.1)
    return path


def tokens(seed: int, n: int, vocab: int) -> list[int]:
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


_plain_cache: dict = {}


def plain_logits(model_dir: str, ids) -> np.ndarray:
    """[T, vocab] logits of the whole sequence from the plain implementation (cached per call)."""
    key = (model_dir, tuple(ids))
    if key not in _plain_cache:
        weights, cfg = P.load_model_dir(model_dir)
        _plain_cache[key] = P.forward(weights, cfg, list(ids))
    return _plain_cache[key]


def tolerance(dtype: str) -> float:
    """Largest allowed max|engine - plain| as a fraction of max|plain|.  32-bit: the reference's own
    CPU tolerance of 1e-5 x scale (/root/reference/src/runtime/lm.rs:1497-1511).  bfloat16: the
    reference allows its reduced-precision GPU path 3e-3 x scale with float32 activations (same
    lines); bfloat16 activations round to 2^-9 = 2e-3 per value at every layer boundary, for which
    2e-2 x scale is allowed here."""
    return {"float32": 1e-5, "bfloat16": 2e-2}[dtype]


def assert_close(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "") -> None:
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    scale = np.abs(want).max()
    err = np.abs(got - want).max(axis=-1) if got.ndim > 1 else np.abs(got - want)
    worst = int(np.argmax(err))
    assert err.max() <= tolerance(dtype) * scale, (
        f"{what}: max error {err.max():.3e} at row {worst} exceeds {tolerance(dtype)} x scale {scale:.3e}; "
        f"first bad row {int(np.argmax(err > tolerance(dtype) * scale))}")

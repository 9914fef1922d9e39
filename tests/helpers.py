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
# Tiny D: sizes that the fast kernels refuse, so that every fallback runs: a width of 100 and a
# feed-forward width of 150 (no multiples of 8; 226 auto-adjusted to two thirds without rounding),
# heads of 24 (no multiple of 16), an odd vocabulary, K 5.
TINY_D = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 3, "layer_types": ["conv", "full_attention", "conv"],
    "hidden_size": 100, "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 24,
    "block_ff_dim": 226, "block_auto_adjust_ff_dim": True, "vocab_size": 131, "tie_embedding": True,
    "conv_L_cache": 5, "conv_bias": False, "rope_theta": 10000.0, "norm_eps": 1e-5,
    "max_position_embeddings": 512,
}
# Medium M: the serving shapes in small: heads of 64, grouping 4:1, every size aligned, so that the
# engine takes its fast kernels (matrix-core attention for prompts and decoding, packed weights, the
# library product above 64 rows) on sequences long enough for key slices and many pages.
MEDIUM_M = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 4, "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "hidden_size": 512, "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64,
    "block_ff_dim": 1536, "block_auto_adjust_ff_dim": False, "vocab_size": 4096, "tie_embedding": True,
    "conv_L_cache": 3, "conv_bias": False, "rope_theta": 1000000.0, "norm_eps": 1e-5,
    "max_position_embeddings": 8192,
}
# Wide W: the decode products' other launch shapes in small: a feed-forward width of 6,144 (a workgroup
# of the gated product takes two tiles of features from 33 rows on; the down projection with its inner
# size of 4,096 or more is cut along k and summed by a second kernel), K 4, three layers.
WIDE_W = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 3, "layer_types": ["conv", "full_attention", "conv"],
    "hidden_size": 512, "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64,
    "block_ff_dim": 6144, "block_auto_adjust_ff_dim": False, "vocab_size": 3000, "tie_embedding": True,
    "conv_L_cache": 4, "conv_bias": True, "rope_theta": 1000000.0, "norm_eps": 1e-5,
    "max_position_embeddings": 4096,
}
# Big L: three layers (convolution, attention, convolution) of the LFM2-1.2B layer sizes, vocabulary and all.
BIG_L = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "num_hidden_layers": 3, "layer_types": ["conv", "full_attention", "conv"],
    "hidden_size": 2048, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "block_ff_dim": 12288, "block_auto_adjust_ff_dim": True, "block_ffn_dim_multiplier": 1.0, "block_multiple_of": 256,
    "vocab_size": 65536, "tie_embedding": True, "conv_L_cache": 3, "conv_bias": False, "rope_theta": 1000000.0,
    "norm_eps": 1e-5, "max_position_embeddings": 128000,
}
# Tiny G: Tiny A's sizes with norm gains spread widely (1 + N(0, 0.5)): a gain that is multiplied into
# the wrong matrix, or left out, changes the logits by tens of percent.
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "M": MEDIUM_M, "G": TINY_A, "W": WIDE_W, "L": BIG_L}
GAIN_STD = {"A": 0.0, "B": 0.1, "C": 0.1, "D": 0.1, "M": 0.1, "G": 0.5, "W": 0.2, "L": 0.2}


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
_plain_model: list = [None, None]          # the folder whose weights were read last, and what was read


def plain_logits(model_dir: str, ids) -> np.ndarray:
    """[T, vocab] logits of the whole sequence from the plain implementation (cached per call)."""
    key = (model_dir, tuple(ids))
    if key not in _plain_cache:
        if _plain_model[0] != model_dir:
            _plain_model[:] = [model_dir, P.load_model_dir(model_dir)]
        weights, cfg = _plain_model[1]
        _plain_cache[key] = P.forward(weights, cfg, list(ids))
    return _plain_cache[key]


def tolerance(dtype: str) -> float:
    """Largest allowed max|engine - plain| as a fraction of max|plain| in 32-bit: the reference's own
    CPU tolerance of 1e-5 x scale (src/runtime/lm.rs:1497-1511); the engine measures about 2e-6.
    bfloat16 runs are held to per-model bounds instead (`assert_close`, `BF16_REL_L2`, `max_logit_error`)."""
    return {"float32": 1e-5}[dtype]


# Largest error of a single bfloat16 logit against the plain implementation, as a fraction of the
# largest plain logit: 1.3 x the worst measured over every test of that model (A 2.2 %, B 3.8 %, C 2.0 %).  Every activation that a
# matrix product reads or writes is rounded to 8 bits of mantissa (relative error up to 2^-9 each), about
# five such roundings lie on the path through each half of a layer, and what a layer inherits through the
# residual stream adds to its own.
BF16_MAX_ERR = {"A": 0.029, "B": 0.050, "C": 0.027}


def max_logit_error(dtype: str, model: str) -> float:
    """How far one logit of the engine may lie from the plain implementation's, as a fraction of the
    largest plain logit."""
    return 1e-5 if dtype == "float32" else BF16_MAX_ERR[model]


def consistency(dtype: str) -> float:
    """Largest allowed difference, as a fraction of the scale, between the logits that two ways of
    cutting or batching the same tokens give in the same precision.  32-bit: the ways differ only
    in the order of float32 additions.  bfloat16: prompt portions and decoded tokens take different
    attention kernels (the matrix-core kernel rounds the softmax weights to bfloat16 for its second
    product, the decode kernel keeps them in float32) and different matrix-product kernels, so the
    ways differ by rounding noise of the same kind as each differs from the plain implementation,
    amplified through the layers in the same way (measured up to 2.7 %: decoded tokens of the 4-layer model against
    its whole prompt; 2.4 % for the 6-layer model's portions, whose feed-forwards take the fused few-row kernels);
    what pins the fast kernels' indexing tightly is their own tests against exact references."""
    return {"float32": 2e-6, "bfloat16": 4e-2}[dtype]


# Largest per-row relative L2 error of bfloat16 logits against the plain implementation: 1.5 x the worst
# row measured over every test of that model (4 layers: A, M, G; 6 layers of width 96: B; 3 layers: C, D).
# A gain folded into the wrong matrix, a norm in the wrong place or a wrong key shows as tens of percent.
# (measured worst rows: A 2.4 %, B 4.9 %, C 2.5 %, D 4.5 %, G 4.5 %, M 2.4 %, W 1.6 %, L 1.3 %; models that tests put
# together themselves up to 4.7 %; the cosine over all rows of a comparison was never below 0.9998)
BF16_REL_L2 = {"A": 0.036, "B": 0.074, "C": 0.037, "D": 0.067, "M": 0.035, "G": 0.067, "W": 0.024, "L": 0.019}
BF16_REL_L2_OTHER = 0.07
BF16_COSINE = 0.9995


def model_of(model_dir: str) -> str:
    """The tiny model's name from a folder that `make_model_dir` made."""
    parts = os.path.basename(model_dir.rstrip("/")).split("_")
    return parts[1] if len(parts) >= 3 and parts[0] == "tiny" else ""


def _record(what: str, model: str, dtype: str, rel: float, cos: float, err: float) -> None:
    path = os.environ.get("GIBBS_TEST_RECORD")
    if path:
        import json
        with open(path, "a") as f:
            f.write(json.dumps({"what": what, "model": model, "dtype": dtype, "rel_l2": rel, "cos": cos, "max_err": err}) + "\n")


def assert_close(got: np.ndarray, want: np.ndarray, dtype: str, what: str = "", tol: float | None = None,
                 model: str = "") -> None:
    """32-bit, or with `tol` given: the largest difference as a fraction of the largest wanted value.
    bfloat16 against the plain implementation: every row's relative L2 error within the model's
    measured bound and the cosine over all rows at least 0.9995."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    g2, w2 = np.atleast_2d(got), np.atleast_2d(want)
    norm = np.sqrt((w2 * w2).sum(-1)) + 1e-300
    rel = np.sqrt(((g2 - w2) ** 2).sum(-1)) / norm
    cos = (g2 * w2).sum(-1) / (norm * (np.sqrt((g2 * g2).sum(-1)) + 1e-300))
    scale = np.abs(want).max()
    err = np.abs(g2 - w2).max(axis=-1)
    _record(what, model, dtype, float(rel.max()), float((g2 * w2).sum() / np.sqrt((g2 * g2).sum() * (w2 * w2).sum() + 1e-300)),
            float(err.max() / scale))
    if dtype == "bfloat16" and tol is None:
        bound = BF16_REL_L2.get(model, BF16_REL_L2_OTHER)
        worst = int(np.argmax(rel))
        all_cos = (g2 * w2).sum() / np.sqrt((g2 * g2).sum() * (w2 * w2).sum() + 1e-300)
        assert rel.max() <= bound and all_cos >= BF16_COSINE, (
            f"{what}: relative L2 error {rel.max():.3e} at row {worst} (bound {bound}), cosine over all rows "
            f"{all_cos:.6f} (bound {BF16_COSINE}); first bad row {int(np.argmax(rel > bound))}")
        return
    tol = tolerance(dtype) if tol is None else tol
    worst = int(np.argmax(err))
    assert err.max() <= tol * scale, (
        f"{what}: max error {err.max():.3e} at row {worst} exceeds {tol} x scale {scale:.3e}; "
        f"first bad row {int(np.argmax(err > tol * scale))}")

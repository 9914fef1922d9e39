"""The reference's tiny LFM2 golden fixture, regenerated bit for bit.

Weights come from one SplitMix64 stream in call order (tests/golden/util.rs:18-95);
the model and its draw order are those of `graphlm_lfm2` (tests/golden/lm.rs:262-309);
the expected logits are the reference's committed tests/golden/lm_graphlm_lfm2.json.  Its numbers
(float32 logits and the greedy ids) are kept beside this file as golden_lfm2_expected.npz, so
that the check also runs where the reference is not mounted; when it is mounted, the copy is
compared with the original.
"""
from __future__ import annotations

import json
import os

import numpy as np

MASK = (1 << 64) - 1
# the reference's checkout, if there is one here: $GIBBS_REFERENCE, else a `reference` folder beside the repository
REFERENCE = os.environ.get("GIBBS_REFERENCE") or os.path.join(
    os.path.dirname(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))), "reference")
GOLDEN_JSON = os.path.join(REFERENCE, "tests", "golden", "lm_graphlm_lfm2.json")
GOLDEN_NPZ = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden_lfm2_expected.npz")

PROMPT = [5, 17, 42, 99, 133, 200]            # tests/golden/lm.rs:13
DECODE = [7, 64, 250]                         # tests/golden/lm.rs:15
LONG_PROMPT = [(i * 37 + 11) % 252 + 4 for i in range(20)]   # tests/golden/lm.rs:18-20


class SplitMix64:
    """tests/golden/util.rs:18-46."""

    def __init__(self, seed: int):
        self.s = seed & MASK

    def next_u64(self) -> int:
        self.s = (self.s + 0x9E3779B97F4A7C15) & MASK
        z = self.s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
        return z ^ (z >> 31)

    def unit(self) -> np.float32:
        """Uniform in [-1, 1), float32 arithmetic as written (util.rs:34-36)."""
        return np.float32(np.float32(self.next_u64() >> 40) / np.float32(1 << 24)) * np.float32(2.0) - np.float32(1.0)

    def vec(self, n: int, scale) -> np.ndarray:
        scale = np.float32(scale)
        return np.array([self.unit() * scale for _ in range(n)], dtype=np.float32)

    def around(self, n: int, center, spread) -> np.ndarray:
        center, spread = np.float32(center), np.float32(spread)
        return np.array([center + self.unit() * spread for _ in range(n)], dtype=np.float32)


class Weights:
    """tests/golden/util.rs:51-95."""

    def __init__(self, seed: int):
        self.rng = SplitMix64(seed)
        self.tensors: dict[str, np.ndarray] = {}

    def w(self, name, shape):
        n = int(np.prod(shape))
        scale = np.float32(1.0) / np.sqrt(np.float32(shape[-1])) if len(shape) >= 2 else np.float32(0.5)
        self.tensors[name] = self.rng.vec(n, scale).reshape(shape)

    def s(self, name, shape, scale):
        self.tensors[name] = self.rng.vec(int(np.prod(shape)), scale).reshape(shape)

    def norm(self, name, n, center):
        self.tensors[name] = self.rng.around(n, center, 0.1)


def golden_config() -> dict:
    """tests/golden/lm.rs:39-52 (base) and :273-283 (LFM2 extras)."""
    return {
        "model_type": "lfm2", "architectures": ["Lfm2ForCausalLM"], "vocab_size": 256,
        "hidden_size": 32, "num_hidden_layers": 3, "num_attention_heads": 4,
        "num_key_value_heads": 2, "head_dim": 8, "intermediate_size": 64,
        "rms_norm_eps": 1e-5, "rope_theta": 1000000.0, "hidden_act": "silu",
        "max_position_embeddings": 128, "bos_token_id": 1, "eos_token_id": 2,
        "tie_word_embeddings": True,
        "norm_eps": 1e-5, "conv_L_cache": 3, "conv_bias": False,
        "block_auto_adjust_ff_dim": False,
        "layer_types": ["conv", "full_attention", "conv"],
    }


def golden_weights() -> dict:
    """tests/golden/lm.rs:284-307, seed 13."""
    V, h, heads, kv, hd, inter, k = 256, 32, 4, 2, 8, 64, 3
    w = Weights(13)
    w.s("model.embed_tokens.weight", [V, h], 0.05)
    w.norm("model.embedding_norm.weight", h, 1.0)
    for l, is_conv in enumerate([True, False, True]):
        p = f"model.layers.{l}"
        w.norm(f"{p}.operator_norm.weight", h, 1.0)
        w.norm(f"{p}.ffn_norm.weight", h, 1.0)
        if is_conv:
            w.w(f"{p}.conv.in_proj.weight", [3 * h, h])
            w.w(f"{p}.conv.conv.weight", [h, 1, k])
            w.w(f"{p}.conv.out_proj.weight", [h, h])
        else:
            a, kvd = heads * hd, kv * hd
            w.w(f"{p}.self_attn.q_proj.weight", [a, h])
            w.w(f"{p}.self_attn.k_proj.weight", [kvd, h])
            w.w(f"{p}.self_attn.v_proj.weight", [kvd, h])
            w.w(f"{p}.self_attn.out_proj.weight", [h, a])
            w.norm(f"{p}.self_attn.q_layernorm.weight", hd, 1.0)
            w.norm(f"{p}.self_attn.k_layernorm.weight", hd, 1.0)
        w.w(f"{p}.feed_forward.w1.weight", [inter, h])
        w.w(f"{p}.feed_forward.w3.weight", [inter, h])
        w.w(f"{p}.feed_forward.w2.weight", [h, inter])
    return w.tensors


def golden_expected():
    """The reference's committed outputs: {"f32": {name: logits}, "ids": {"greedy8": [...]}}."""
    data = np.load(GOLDEN_NPZ, allow_pickle=False)
    out = {"f32": {k: data[k].astype(np.float64) for k in data.files if k != "greedy8"},
           "ids": {"greedy8": data["greedy8"].tolist()}}
    if os.path.exists(GOLDEN_JSON):                     # the copy must be the original's numbers
        with open(GOLDEN_JSON) as f:
            orig = json.load(f)
        assert orig["ids"]["greedy8"] == out["ids"]["greedy8"]
        for k, v in orig["f32"].items():
            assert np.array_equal(np.asarray(v, dtype=np.float64), out["f32"][k]), k
    return out


def write_safetensors_f32(path: str, tensors: dict) -> None:
    """A minimal F32 safetensors writer in the manner of tests/golden/util.rs:111-143
    (header padded to a multiple of 8 with spaces)."""
    header, blobs, off = {}, [], 0
    for name, arr in tensors.items():
        if arr.dtype.kind == "i":
            b, tag = np.ascontiguousarray(arr, dtype=np.int32).tobytes(), "I32"
        else:
            b, tag = np.ascontiguousarray(arr, dtype=np.float32).tobytes(), "F32"
        header[name] = {"dtype": tag, "shape": list(arr.shape), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header, separators=(",", ":")).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(path, "wb") as f:
        f.write(len(hj).to_bytes(8, "little"))
        f.write(hj)
        for b in blobs:
            f.write(b)


def write_golden_model(folder: str) -> None:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(golden_config(), f)
    write_safetensors_f32(os.path.join(folder, "model.safetensors"), golden_weights())


def rel_l2(a, b) -> float:
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def cosine(a, b) -> float:
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(a @ b / max(np.linalg.norm(a) * np.linalg.norm(b), 1e-30))

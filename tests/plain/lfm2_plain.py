"""Plain LFM2 forward pass: whole sequences, no cache, one function per part.

Everything here is written from the text of the reference (MisterTK/gibbs);
each function names the file:line it was read from.  Arithmetic is float64
except where the reference pins a float32 step (RoPE frequencies and angles),
so the result is an arbiter for both the engine's 32-bit and bfloat16 paths.
Nothing from the product package is imported.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- config
def _first(*vals):
    """`first(a, b, ...)` of the spec language: the first value that is not null
    (src/arch/expr.rs:723)."""
    for v in vals:
        if v is not None:
            return v
    return None


def resolve_config(cfg: dict, embed_rows: int | None = None) -> dict:
    """Sizes and constants of an LFM2 checkpoint, from config.json keys with the
    reference's precedence (arch/families/lfm2.json5:27-51)."""
    hidden = cfg["hidden_size"]                                                   # :29
    layers = cfg["num_hidden_layers"]                                             # :30
    heads = _first(cfg.get("num_attention_heads"), cfg.get("num_heads"))          # :31
    kv_heads = _first(cfg.get("num_key_value_heads"), heads)                      # :33
    head_dim = _first(cfg.get("head_dim"), hidden // heads)                       # :34
    vocab = _first(embed_rows, cfg.get("vocab_size"))                             # :35
    ff_raw = _first(cfg.get("intermediate_size"), cfg.get("block_ff_dim"), 4 * hidden)  # :38
    ff_23 = ff_raw * 2 // 3                                                       # :39
    ff_multiple = _first(cfg.get("block_multiple_of"), 256)                       # :40
    if cfg.get("block_auto_adjust_ff_dim") is True:                               # :41
        mult = _first(cfg.get("block_ffn_dim_multiplier"), 0)
        if mult > 0:
            # int() truncates (src/arch/expr.rs:820), `/` is float division, ceil rounds up.
            inter = ff_multiple * math.ceil(int(mult * ff_23) / ff_multiple)
        else:
            inter = ff_23
    else:
        inter = ff_raw
    eps = _first(cfg.get("norm_eps"), cfg.get("rms_norm_eps"), 1e-5)              # :42
    rp = cfg.get("rope_parameters") or {}
    theta = _first(cfg.get("rope_theta"), rp.get("rope_theta"), 10000)            # :45
    conv_k = cfg.get("conv_L_cache")                                              # :49
    if conv_k is None or conv_k < 2:                                              # :54
        raise ValueError(f"LFM2 short-conv kernel (conv_L_cache) {conv_k} must be >= 2")
    return dict(hidden=hidden, layers=layers, heads=heads, kv_heads=kv_heads, head_dim=head_dim,
                vocab=vocab, inter=inter, eps=float(eps), theta=float(theta), conv_k=conv_k,
                attn_scale=1.0 / math.sqrt(head_dim))                             # :48


# --------------------------------------------------------------------------- parts
def embedding(table: np.ndarray, ids) -> np.ndarray:
    """x[t,:] = E[ids[t],:]; an id beyond the table is an error, no scaling
    (src/graph/cpu.rs:161-248, id check :174)."""
    table = np.asarray(table, dtype=F64)
    ids = np.asarray(ids, dtype=np.int64)
    if ids.size and (ids.min() < 0 or ids.max() >= table.shape[0]):
        raise IndexError(f"token id {int(ids.max())} out of range for {table.shape[0]} rows")
    return table[ids].copy()


def rms_norm(x: np.ndarray, gain: np.ndarray, eps: float) -> np.ndarray:
    """out = x * (1/sqrt(sum(x^2)/n + eps)) * gain over the last axis; eps inside
    the root, gain multiplied last, no (1 + gain) offset (src/model/simd.rs:75-110,
    src/graph/cpu.rs:358-377)."""
    x = np.asarray(x, dtype=F64)
    gain = np.asarray(gain, dtype=F64)
    n = x.shape[-1]
    assert gain.shape == (n,)
    sum_sq = np.sum(x * x, axis=-1, keepdims=True)
    scale = 1.0 / np.sqrt(sum_sq / n + eps)
    return x * scale * gain


def rope_inv_freq(dim: int, theta: float) -> np.ndarray:
    """inv_freq[i] = 1 / theta^(2i/dim), computed in float32 as LFM2's spec asks
    (`precision: 'f32'`, arch/families/lfm2.json5:64; src/arch/gen.rs:162-164)."""
    half = dim // 2
    t = np.float32(theta)
    out = np.empty(half, dtype=np.float32)
    for i in range(half):
        expo = np.float32(2 * i) / np.float32(dim)
        out[i] = np.float32(1.0) / np.power(t, expo, dtype=np.float32)
    return out


def rope_half_split(x: np.ndarray, positions, inv_freq: np.ndarray) -> np.ndarray:
    """HalfSplit rotation of x[T, heads, head_dim]: pair (j, j + half) turned by the
    angle float32(pos) * inv_freq[j] (a float32 product), mscale 1
    (src/graph/cpu.rs:602-719: angle :673, HalfSplit pairing :686-695)."""
    x = np.asarray(x, dtype=F64)
    T, heads, hd = x.shape
    half = len(inv_freq)
    assert 2 * half <= hd
    out = x.copy()
    for t in range(T):
        for j in range(half):
            angle = np.float32(np.float32(positions[t]) * np.float32(inv_freq[j]))
            c, s = math.cos(float(angle)), math.sin(float(angle))
            x0 = x[t, :, j]
            x1 = x[t, :, j + half]
            out[t, :, j] = x0 * c - x1 * s
            out[t, :, j + half] = x0 * s + x1 * c
    return out


def causal_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                     window: int | None = None, positions=None) -> np.ndarray:
    """Causal grouped-query attention of q[T,nh,hd] over k,v[T,nkv,hd]: query head h
    reads kv head h // (nh/nkv); key i is visible to query t iff i <= t (and, with a
    window w, i + w > t); softmax subtracts the maximum over the visible keys
    (src/graph/cpu.rs:826-951: grouping :845/:886, mask :889-899, softmax :907-921)."""
    q = np.asarray(q, dtype=F64)
    k = np.asarray(k, dtype=F64)
    v = np.asarray(v, dtype=F64)
    T, nh, hd = q.shape
    nkv = k.shape[1]
    rep = nh // nkv
    out = np.zeros((T, nh, v.shape[2]), dtype=F64)
    for t in range(T):
        lo = 0 if window is None else max(0, t - window + 1)
        for h in range(nh):
            g = h // rep
            scores = (k[lo:t + 1, g, :] @ q[t, h, :]) * scale
            w = np.exp(scores - scores.max())
            w = w / w.sum()
            out[t, h, :] = w @ v[lo:t + 1, g, :]
    return out


def causal_conv1d(x: np.ndarray, taps: np.ndarray, bias: np.ndarray | None = None,
                  state: np.ndarray | None = None):
    """Depthwise causal convolution of x[T,C] with taps[C,K]: the window is the state
    ([K-1, C], oldest row first, zeros at a sequence start) followed by x; tap K-1
    multiplies the current row and tap j the row K-1-j steps back; the new state is
    the window's last K-1 rows (src/graph/cpu.rs:952-994: taps :976-983, state :987).
    The reference refuses a bias (arch/families/lfm2.json5:53); here it is added after
    the tap sum, as a depthwise convolution's bias is.  Returns (out, new_state)."""
    x = np.asarray(x, dtype=F64)
    taps = np.asarray(taps, dtype=F64)
    T, C = x.shape
    K = taps.shape[1]
    assert taps.shape == (C, K)
    hist = K - 1
    if state is None:
        state = np.zeros((hist, C), dtype=F64)
    window = np.concatenate([np.asarray(state, dtype=F64), x], axis=0)
    out = np.zeros((T, C), dtype=F64)
    for t in range(T):
        for j in range(K):
            back = K - 1 - j
            out[t] += taps[:, j] * window[hist + t - back]
        if bias is not None:
            out[t] += np.asarray(bias, dtype=F64)
    return out, window[T:].copy()


def linear(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """y = x @ w^T with w stored [out, in] (src/graph/cpu.rs:249-274, src/model/nn.rs:516-527)."""
    return np.asarray(x, dtype=F64) @ np.asarray(w, dtype=F64).T


def short_conv_mixer(h, w_in, taps, w_out, bias=None):
    """[B | C | x] = thirds of in_proj(h) in that order; out_proj(C * conv(B * x))
    (arch/lib/transformer.json5:140-151)."""
    bcx = linear(h, w_in)
    cw = bcx.shape[1] // 3
    b, c, xs = bcx[:, :cw], bcx[:, cw:2 * cw], bcx[:, 2 * cw:3 * cw]
    taps = np.asarray(taps, dtype=F64).reshape(cw, -1)       # [H,1,K] -> [H,K] (lfm2.json5:61)
    cv, _ = causal_conv1d(b * xs, taps, bias)
    return linear(c * cv, w_out)


def attention_mixer(h, wq, wk, wv, wo, q_gain, k_gain, *, heads, kv_heads, head_dim, eps,
                    inv_freq, positions, scale, window=None):
    """q,k,v projections; RMSNorm of every head of q and k with one [head_dim] gain,
    before RoPE; RoPE on q and k; causal GQA; out_proj
    (arch/lib/transformer.json5:46-87 with qk_norm 'before', arch/families/lfm2.json5:80-83)."""
    T = h.shape[0]
    q = linear(h, wq).reshape(T, heads, head_dim)
    k = linear(h, wk).reshape(T, kv_heads, head_dim)
    v = linear(h, wv).reshape(T, kv_heads, head_dim)
    q = rms_norm(q, q_gain, eps)
    k = rms_norm(k, k_gain, eps)
    q = rope_half_split(q, positions, inv_freq)
    k = rope_half_split(k, positions, inv_freq)
    a = causal_attention(q, k, v, scale, window)
    return linear(a.reshape(T, heads * head_dim), wo)


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """(g * 1/(1+exp(-g))) * u (src/graph/cpu.rs:378-390)."""
    gate = np.asarray(gate, dtype=F64)
    return (gate * (1.0 / (1.0 + np.exp(-gate)))) * np.asarray(up, dtype=F64)


def swiglu_ffn(h, w1, w3, w2):
    """down(silu(gate(h)) * up(h)) with gate = w1, up = w3, down = w2
    (arch/lib/transformer.json5:117-130, arch/families/lfm2.json5:86-87)."""
    return linear(swiglu(linear(h, w1), linear(h, w3)), w2)


# --------------------------------------------------------------------------- whole model
def forward(weights: dict, cfg: dict, ids, positions=None) -> np.ndarray:
    """Logits [T, vocab] of the whole sequence `ids` from a fresh state
    (arch/families/lfm2.json5:66-95).  A layer is a conv layer iff it has
    `conv.in_proj.weight` (:78-80); the head is `lm_head.weight` if present, else the
    embedding (:91)."""
    emb = weights["model.embed_tokens.weight"]
    c = resolve_config(cfg, embed_rows=emb.shape[0])
    T = len(ids)
    if positions is None:
        positions = list(range(T))
    inv_freq = rope_inv_freq(c["head_dim"], c["theta"])
    x = embedding(emb, ids)
    for i in range(c["layers"]):
        p = f"model.layers.{i}"
        h = rms_norm(x, weights[f"{p}.operator_norm.weight"], c["eps"])
        if f"{p}.conv.in_proj.weight" in weights:
            a = short_conv_mixer(h, weights[f"{p}.conv.in_proj.weight"], weights[f"{p}.conv.conv.weight"],
                                 weights[f"{p}.conv.out_proj.weight"], weights.get(f"{p}.conv.conv.bias"))
        else:
            a = attention_mixer(h, weights[f"{p}.self_attn.q_proj.weight"], weights[f"{p}.self_attn.k_proj.weight"],
                                weights[f"{p}.self_attn.v_proj.weight"], weights[f"{p}.self_attn.out_proj.weight"],
                                weights[f"{p}.self_attn.q_layernorm.weight"], weights[f"{p}.self_attn.k_layernorm.weight"],
                                heads=c["heads"], kv_heads=c["kv_heads"], head_dim=c["head_dim"], eps=c["eps"],
                                inv_freq=inv_freq, positions=positions, scale=c["attn_scale"])
        x = x + a
        h = rms_norm(x, weights[f"{p}.ffn_norm.weight"], c["eps"])
        m = swiglu_ffn(h, weights[f"{p}.feed_forward.w1.weight"], weights[f"{p}.feed_forward.w3.weight"],
                       weights[f"{p}.feed_forward.w2.weight"])
        x = x + m
    x = rms_norm(x, weights["model.embedding_norm.weight"], c["eps"])
    head = weights.get("lm_head.weight", emb)
    return linear(x, head)


# --------------------------------------------------------------------------- sampling
def argmax_first(logits) -> int:
    """Index of the first largest element; NaN never wins; 0 when nothing is above
    -inf (src/runtime/lm.rs:1043-1057)."""
    vals = [float(v) for v in np.asarray(logits, dtype=np.float32)]
    mx = -math.inf
    for v in vals:
        if not math.isnan(v) and v > mx:
            mx = v
    for i, v in enumerate(vals):
        if v == mx:
            return i
    return 0


def nucleus(logits, temperature: float, top_k: int, top_p: float):
    """Candidates of a sampled draw: top-k (<= 64) by (logit desc, id asc), softmax at
    `temperature` in float32, cut at the shortest prefix whose cumulative probability
    reaches clamp(top_p, 0.01, 1) (src/runtime/lm.rs:1153-1240).  Returns (ids, probs)."""
    logits = np.asarray(logits, dtype=np.float32)
    assert top_k <= 64
    k = min(max(top_k, 1), len(logits))
    order = sorted(range(len(logits)), key=lambda i: (-float(logits[i]) if not math.isnan(logits[i]) else math.inf, i))
    cand = order[:k]
    scaled = np.array([np.float32(logits[i]) / np.float32(temperature) for i in cand], dtype=np.float32)
    mx = scaled.max()
    e = np.exp((scaled - mx).astype(np.float32)).astype(np.float32)
    denom = max(np.float32(e.sum(dtype=np.float32)), np.float32(1e-12))
    probs = (e / denom).astype(np.float32)
    thresh = min(max(top_p, 0.01), 1.0)
    cum, cut = np.float32(0.0), k
    for i, p in enumerate(probs):
        cum = np.float32(cum + p)
        if cum >= np.float32(thresh):
            cut = i + 1
            break
    return cand[:cut], probs[:cut]


def repetition_penalty(logits, recent, penalty: float, greedy: bool) -> np.ndarray:
    """The logits as the reference's sampler sees them with a repetition penalty > 1 over the
    recent tokens: a token that occurs c times is, c times over, divided by the penalty if its
    value is positive and multiplied by it if not.  The greedy rule then takes 1.5 c off
    (src/runtime/lm.rs:1089-1105); the sampling rule takes 1.5 off after each of the c steps, so a
    value can change sign on the way (src/runtime/lm.rs:1176-1189).  A penalty <= 1 or no recent
    tokens change nothing (src/runtime/lm.rs:1072, :1163)."""
    out = np.array(logits, dtype=np.float32)
    if not penalty > 1.0 or len(recent) == 0:
        return out
    p = np.float32(penalty)
    for tok in sorted(set(int(t) for t in recent)):
        if not 0 <= tok < len(out):
            continue
        c = sum(1 for t in recent if int(t) == tok)
        v = out[tok]
        for _ in range(c):
            v = np.float32(v / p) if v > 0 else np.float32(v * p)
            if not greedy:
                v = np.float32(v - np.float32(1.5))
        if greedy:
            v = np.float32(v - np.float32(c) * np.float32(1.5))
        out[tok] = v
    return out


def draw(cand, probs, u: float) -> int:
    """Pick the first candidate whose cumulative probability reaches u * sum(probs)
    (src/runtime/lm.rs:1137-1145)."""
    r = np.float32(u) * np.float32(np.sum(probs, dtype=np.float32))
    cum = np.float32(0.0)
    for i, p in enumerate(probs):
        cum = np.float32(cum + p)
        if cum >= r or i == len(probs) - 1:
            return cand[i]
    return cand[0]


# --------------------------------------------------------------------------- files
_ST_DTYPES = {"F32": np.float32, "F16": np.float16, "I32": np.int32, "F64": np.float64}


def read_safetensors(path: str) -> dict:
    """name -> float64/int array.  Layout: u64 LE header length, JSON header
    {name: {dtype, shape, data_offsets}}, then the data (src/model/loaders/safetensors.rs:15-64)."""
    with open(path, "rb") as f:
        raw = f.read()
    n = int.from_bytes(raw[:8], "little")
    header = json.loads(raw[8:8 + n])
    data = raw[8 + n:]
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        buf = data[lo:hi]
        if meta["dtype"] == "BF16":
            u16 = np.frombuffer(buf, dtype=np.uint16).astype(np.uint32) << 16
            arr = u16.view(np.float32)
        else:
            arr = np.frombuffer(buf, dtype=_ST_DTYPES[meta["dtype"]])
        arr = arr.reshape(meta["shape"])
        out[name] = arr.astype(F64) if arr.dtype.kind == "f" else arr.copy()
    return out


def load_model_dir(path: str):
    """(weights, config.json dict) of a model folder."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    return read_safetensors(os.path.join(path, "model.safetensors")), cfg

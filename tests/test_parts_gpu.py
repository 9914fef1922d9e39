"""Each part alone against the plain implementation; parts chosen layer by layer; a layer order
that names a layer twice and a layer that reads another layer's cache; a windowed attention
whose cache group gives pages back; and a toy mixer with state of its own, defined here and
registered without a change to the framework's files."""
import json
import math
import os

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import lfm2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [("float32", torch.float32), ("bfloat16", torch.bfloat16)]


def bf16_exact(a: np.ndarray) -> np.ndarray:
    """Rounds to values bfloat16 holds exactly, so every precision starts from the same numbers."""
    return torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).double().numpy()


def store(tensors: dict, decls, dtype):
    from gibbs_amd.weights import WeightStore
    out = {}
    for d in decls:
        out[d.name] = torch.tensor(tensors[d.name]).reshape(d.shape).to(DEV, d.resolved_dtype(dtype)).contiguous()
    return WeightStore(out, dtype, torch.device(DEV))


def run_mixer(mixer, hs, chunks, dtype, page_size=8):
    """Feeds h (a list of [T_r, hidden] arrays, one per request) through a bound mixer in the given
    chunks [(request, a, b), ...] per step; returns the concatenated outputs per request."""
    from gibbs_amd.cache import CacheManager, DeviceCache
    from gibbs_amd.engine.batch import BatchStager
    cm = CacheManager([mixer.cache_need()], [tuple(mixer.state_needs())], page_size, 64, 4)
    dc = DeviceCache(cm, dtype, torch.device(DEV))
    view = dc.layer_view(0)
    stager = BatchStager(torch.device(DEV))
    outs = {r: [] for r in range(len(hs))}
    for step in chunks:
        rids = [r for r, _, _ in step]
        for r, a, b in step:
            if r not in cm:
                assert cm.admit(r)
            assert cm.reserve(r, b - a)
        dc.clear_fresh_slots()
        q = np.array([b - a for _, a, b in step], dtype=np.int32)
        cu = np.concatenate([[0], np.cumsum(q)]).astype(np.int32)
        ctx = np.array([cm.tokens(r) for r in rids], dtype=np.int32)
        row_req = np.repeat(np.arange(len(step), dtype=np.int32), q)
        pos = (np.arange(cu[-1], dtype=np.int32) - cu[:-1][row_req] + ctx[row_req]).astype(np.int32)
        batch = stager.stage(np.zeros(cu[-1], np.int32), pos, row_req, cu, ctx,
                             np.array([cm.slot(r) for r in rids], np.int32), np.zeros(0, np.int32),
                             [cm.block_table(rids, g) for g in range(cm.n_groups)])
        h = torch.tensor(np.concatenate([hs[r][a:b] for r, a, b in step])).to(DEV, dtype).contiguous()
        y = mixer.forward(h, batch, view)
        if y.dim() == 3:
            y = y.sum(0)
        y = y.float().cpu().numpy()
        for i, (r, a, b) in enumerate(step):
            outs[r].append(y[cu[i]:cu[i + 1]])
            cm.commit(r, b - a)
        cm.check()
    return {r: np.concatenate(v) for r, v in outs.items()}, cm


def close(got, want, name, what):
    tol = {"float32": 1e-5, "bfloat16": 2e-2}[name]
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= tol * scale, f"{what}: {np.abs(got - want).max():.3e} > {tol} x {scale:.3e}"


# two requests fed in ragged steps: portions of one beside single tokens of the other
STEPS = [[(0, 0, 5)], [(0, 5, 7), (1, 0, 9)], [(0, 7, 8), (1, 9, 11)], [(0, 8, 9), (1, 11, 12)], [(0, 9, 26), (1, 12, 13)],
         [(1, 13, 14), (0, 26, 27)]]


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_norm_part(name, dtype):
    from gibbs_amd.config import NormSpec
    from gibbs_amd.parts import Runtime, build_norm
    rng = np.random.default_rng(0)
    norm = build_norm(NormSpec("rms", 3e-6, "g"), 72)
    gain = rng.normal(size=72) + 1
    norm.bind(store({"g": gain}, norm.tensor_decls(), dtype), Runtime(torch.device(DEV), dtype))
    x = rng.normal(size=(5, 72)).astype(np.float32)
    delta = bf16_exact(rng.normal(size=(5, 72)))
    xt = torch.tensor(x, device=DEV)
    out = norm.forward(xt, torch.tensor(delta).to(DEV, dtype))
    close(out.float().cpu().numpy(), P.rms_norm(x.astype(np.float64) + delta, gain, 3e-6), name, "norm")
    np.testing.assert_allclose(xt.cpu().numpy(), x + delta.astype(np.float32), rtol=1e-6)


def test_rope_part_table():
    from gibbs_amd.config import PositionSpec
    from gibbs_amd.parts import Runtime, build_position
    for theta, dim in [(1e4, 16), (1e6, 64), (5e5, 48)]:
        pos = build_position(PositionSpec("rope", {"theta": theta, "rotary_dim": dim, "precision": "f32"}), dim)
        pos.bind(None, Runtime(torch.device(DEV), torch.float32))
        np.testing.assert_array_equal(pos.inv_freq.cpu().numpy(), P.rope_inv_freq(dim, theta))
    assert build_position(None, 16) is None and build_position(PositionSpec("none"), 16) is None
    with pytest.raises(ValueError, match="rotary_dim"):
        build_position(PositionSpec("rope", {"theta": 1e4, "rotary_dim": 18}), 16)


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,hd,hidden,window", [(4, 2, 16, 40, None), (3, 1, 48, 72, None), (4, 4, 32, 64, 6)])
def test_attention_part(name, dtype, heads, kv, hd, hidden, window):
    from gibbs_amd.config import MixerSpec, PositionSpec
    from gibbs_amd.parts import Runtime, build_mixer
    rng = np.random.default_rng(1)
    names = {k: k for k in ("q_proj", "k_proj", "v_proj", "out_proj", "q_norm", "k_norm")}
    spec = MixerSpec("attention", {"heads": heads, "kv_heads": kv, "head_dim": hd, "scale": 1 / math.sqrt(hd),
                                   "qk_norm": "before", "qk_norm_eps": 1e-6, "window": window}, names,
                     PositionSpec("rope", {"theta": 1e4, "rotary_dim": hd, "precision": "f32"}))
    mixer = build_mixer(spec, hidden, 0)
    w = {"q_proj": bf16_exact(rng.normal(size=(heads * hd, hidden)) * 0.3), "k_proj": bf16_exact(rng.normal(size=(kv * hd, hidden)) * 0.3),
         "v_proj": bf16_exact(rng.normal(size=(kv * hd, hidden)) * 0.3), "out_proj": bf16_exact(rng.normal(size=(hidden, heads * hd)) * 0.2),
         "q_norm": rng.normal(size=hd) * 0.1 + 1, "k_norm": rng.normal(size=hd) * 0.1 + 1}
    mixer.bind(store(w, mixer.tensor_decls(), dtype), Runtime(torch.device(DEV), dtype))
    hs = [bf16_exact(rng.normal(size=(27, hidden))), bf16_exact(rng.normal(size=(14, hidden)))]
    got, cm = run_mixer(mixer, hs, STEPS, dtype)
    for r, h in enumerate(hs):
        want = P.attention_mixer(h, w["q_proj"], w["k_proj"], w["v_proj"], w["out_proj"], w["q_norm"], w["k_norm"],
                                 heads=heads, kv_heads=kv, head_dim=hd, eps=1e-6, inv_freq=P.rope_inv_freq(hd, 1e4),
                                 positions=list(range(len(h))), scale=1 / math.sqrt(hd), window=window)
        close(got[r], want, name, f"attention part request {r}")
    if window is not None:
        # pages of 8 tokens behind a window of 6: request 0 (27 tokens) holds at most 2 pages at the end
        table = cm.block_table([0], 0)[0]
        assert (table >= 0).sum() <= 2 and (table[:2] == -1).all(), table


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("width,kernel,bias", [(40, 3, False), (72, 4, True), (16, 2, True)])
def test_shortconv_part(name, dtype, width, kernel, bias):
    from gibbs_amd.config import MixerSpec
    from gibbs_amd.parts import Runtime, build_mixer
    rng = np.random.default_rng(2)
    names = {"in_proj": "in", "conv": "taps", "out_proj": "out", "conv_bias": "b"}
    mixer = build_mixer(MixerSpec("short_conv", {"width": width, "kernel": kernel, "bias": bias}, names), width, 0)
    w = {"in": bf16_exact(rng.normal(size=(3 * width, width)) * 0.3), "taps": rng.normal(size=(width, 1, kernel)),
         "out": bf16_exact(rng.normal(size=(width, width)) * 0.3), "b": rng.normal(size=width) * 0.1}
    mixer.bind(store(w, mixer.tensor_decls(), dtype), Runtime(torch.device(DEV), dtype))
    hs = [bf16_exact(rng.normal(size=(27, width))), bf16_exact(rng.normal(size=(14, width)))]
    got, _ = run_mixer(mixer, hs, STEPS, dtype)
    taps32 = w["taps"].astype(np.float32).astype(np.float64)
    for r, h in enumerate(hs):
        want = P.short_conv_mixer(h, w["in"], taps32, w["out"], w["b"].astype(np.float32) if bias else None)
        close(got[r], want, name, f"short conv part request {r}")


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_glu_part(name, dtype):
    from gibbs_amd.config import FeedForwardSpec
    from gibbs_amd.parts import Runtime, build_feed_forward
    rng = np.random.default_rng(3)
    ffn = build_feed_forward(FeedForwardSpec("glu", {"inter": 200, "activation": "silu"},
                                             {"gate": "w1", "up": "w3", "down": "w2"}), 72)
    w = {"w1": bf16_exact(rng.normal(size=(200, 72)) * 0.2), "w3": bf16_exact(rng.normal(size=(200, 72)) * 0.2),
         "w2": bf16_exact(rng.normal(size=(72, 200)) * 0.2)}
    ffn.bind(store(w, ffn.tensor_decls(), dtype), Runtime(torch.device(DEV), dtype))
    h = bf16_exact(rng.normal(size=(9, 72)))
    y = ffn.forward(torch.tensor(h).to(DEV, dtype), None)
    y = y.sum(0) if y.dim() == 3 else y
    close(y.float().cpu().numpy(), P.swiglu_ffn(h, w["w1"], w["w3"], w["w2"]), name, "glu part")
    with pytest.raises(ValueError, match="activation"):
        build_feed_forward(FeedForwardSpec("glu", {"inter": 8, "activation": "softsign"}, {}), 8)
    with pytest.raises(KeyError, match="no feed-forward of kind"):
        build_feed_forward(FeedForwardSpec("experts", {}, {}), 8)


def run_block(block, xs, chunks, dtype, page_size=8):
    """Feeds residual rows xs (one [T_r, hidden] array per request) through a bound block in the given
    chunks per step; returns the stream after the block, and how many steps took the fused decode
    kernels in both halves."""
    from gibbs_amd.cache import CacheManager, DeviceCache
    from gibbs_amd.engine.batch import BatchStager
    cm = CacheManager([block.mixer.cache_need()], [tuple(block.mixer.state_needs())], page_size, 64, 4)
    dc = DeviceCache(cm, dtype, torch.device(DEV))
    views = {"mixer": dc.layer_view(0)}
    stager = BatchStager(torch.device(DEV))
    outs = {r: [] for r in range(len(xs))}
    fused_steps = 0
    for step in chunks:
        rids = [r for r, _, _ in step]
        for r, a, b in step:
            if r not in cm:
                assert cm.admit(r)
            assert cm.reserve(r, b - a)
        dc.clear_fresh_slots()
        q = np.array([b - a for _, a, b in step], dtype=np.int32)
        cu = np.concatenate([[0], np.cumsum(q)]).astype(np.int32)
        ctx = np.array([cm.tokens(r) for r in rids], dtype=np.int32)
        row_req = np.repeat(np.arange(len(step), dtype=np.int32), q)
        pos = (np.arange(cu[-1], dtype=np.int32) - cu[:-1][row_req] + ctx[row_req]).astype(np.int32)
        batch = stager.stage(np.zeros(cu[-1], np.int32), pos, row_req, cu, ctx,
                             np.array([cm.slot(r) for r in rids], np.int32), np.zeros(0, np.int32),
                             [cm.block_table(rids, g) for g in range(cm.n_groups)])
        x = torch.tensor(np.concatenate([xs[r][a:b] for r, a, b in step]), dtype=torch.float32, device=DEV).contiguous()
        y = block.forward(x, batch, views).cpu().numpy()
        plan = next(iter(block._solos.values()))[0]
        fused_steps += plan.last_fused() == 2
        for i, (r, a, b) in enumerate(step):
            outs[r].append(y[cu[i]:cu[i + 1]])
            cm.commit(r, b - a)
    return {r: np.concatenate(v) for r, v in outs.items()}, fused_steps


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("kind,hidden,inter", [("short_conv", 64, 128), ("attention", 64, 128), ("short_conv", 40, 72), ("short_conv", 36, 68)])
def test_block_part(name, dtype, kind, hidden, inter):
    """The arrangement alone: x + mixer(norm(x)), then + feed-forward(norm(.)), with norms whose gains
    and eps differ, through ragged steps.  In bfloat16 the gains are folded into the matrices, and the
    steps that hold single tokens only take the fused decode kernels where the sizes allow them (the
    widths of 64 and 40 do, 36 is no multiple of 8 and does not): both ways give the plain block."""
    from gibbs_amd.config import FeedForwardSpec, LayerSpec, MixerSpec, NormSpec, PositionSpec
    from gibbs_amd.parts import Runtime, build_block
    rng = np.random.default_rng(7)
    heads, kv, hd = 4, 2, 16
    if kind == "short_conv":
        mixer = MixerSpec("short_conv", {"width": hidden, "kernel": 3, "bias": False}, {"in_proj": "in", "conv": "taps", "out_proj": "out"})
        w = {"in": bf16_exact(rng.normal(size=(3 * hidden, hidden)) * 0.3), "taps": rng.normal(size=(hidden, 1, 3)),
             "out": bf16_exact(rng.normal(size=(hidden, hidden)) * 0.3)}
    else:
        mixer = MixerSpec("attention", {"heads": heads, "kv_heads": kv, "head_dim": hd, "scale": hd ** -0.5, "qk_norm": "before",
                                        "qk_norm_eps": 1e-6, "window": None},
                          {k: k for k in ("q_proj", "k_proj", "v_proj", "out_proj", "q_norm", "k_norm")},
                          PositionSpec("rope", {"theta": 1e4, "rotary_dim": hd, "precision": "f32"}))
        w = {"q_proj": bf16_exact(rng.normal(size=(heads * hd, hidden)) * 0.3), "k_proj": bf16_exact(rng.normal(size=(kv * hd, hidden)) * 0.3),
             "v_proj": bf16_exact(rng.normal(size=(kv * hd, hidden)) * 0.3), "out_proj": bf16_exact(rng.normal(size=(hidden, heads * hd)) * 0.2),
             "q_norm": rng.normal(size=hd) * 0.1 + 1, "k_norm": rng.normal(size=hd) * 0.1 + 1}
    w.update({"n1": rng.normal(size=hidden) * 0.2 + 1, "n2": rng.normal(size=hidden) * 0.2 + 1,
              "w1": bf16_exact(rng.normal(size=(inter, hidden)) * 0.2), "w3": bf16_exact(rng.normal(size=(inter, hidden)) * 0.2),
              "w2": bf16_exact(rng.normal(size=(hidden, inter)) * 0.2)})
    spec = LayerSpec("l0", "pre_norm", NormSpec("rms", 1e-5, "n1"), mixer, NormSpec("rms", 1e-6, "n2"),
                     FeedForwardSpec("glu", {"inter": inter, "activation": "silu"}, {"gate": "w1", "up": "w3", "down": "w2"}))
    block = build_block(spec, hidden, 0)
    block.bind(store(w, block.tensor_decls(), dtype), Runtime(torch.device(DEV), dtype))
    xs = [rng.normal(size=(27, hidden)), rng.normal(size=(14, hidden))]
    steps = STEPS + [[(0, 27, 28), (1, 14, 15)], [(1, 15, 16)]]
    xs = [np.concatenate([x, rng.normal(size=(2, hidden))]) for x in xs]
    got, fused = run_block(block, xs, steps, dtype)
    n1, n2 = w["n1"].astype(np.float32).astype(np.float64), w["n2"].astype(np.float32).astype(np.float64)
    for r, x in enumerate(xs):
        x = x.astype(np.float32).astype(np.float64)[:len(got[r])]
        h = P.rms_norm(x, n1, 1e-5)
        if kind == "short_conv":
            a = P.short_conv_mixer(h, w["in"], w["taps"].astype(np.float32).astype(np.float64), w["out"])
        else:
            a = P.attention_mixer(h, w["q_proj"], w["k_proj"], w["v_proj"], w["out_proj"], w["q_norm"].astype(np.float32), w["k_norm"].astype(np.float32),
                                  heads=heads, kv_heads=kv, head_dim=hd, eps=1e-6, inv_freq=P.rope_inv_freq(hd, 1e4),
                                  positions=list(range(len(x))), scale=hd ** -0.5)
        y = x + a
        want = y + P.swiglu_ffn(P.rms_norm(y, n2, 1e-6), w["w1"], w["w3"], w["w2"])
        close(got[r], want, name, f"block {kind} request {r}")
    if name == "bfloat16":
        assert (fused >= 3) == (hidden % 8 == 0), f"{fused} steps took the fused decode kernels"
    else:
        assert fused == 0


# --------------------------------------------------------------------------- whole specs built by hand
def plain_spec_forward(spec, weights, ids):
    """Plain forward of a hand-built ModelSpec from the plain part functions: handles a run order
    that repeats layers and attention layers that read an earlier run's keys and values."""
    T = len(ids)
    x = P.embedding(weights[spec.embedding], ids)
    kv_of_layer = {}
    for i in spec.order:
        L = spec.layers[i]
        h = P.rms_norm(x, weights[L.mixer_norm.weight], L.mixer_norm.eps)
        m, t = L.mixer, L.mixer.tensors
        if m.kind == "short_conv":
            a = P.short_conv_mixer(h, weights[t["in_proj"]], weights[t["conv"]], weights[t["out_proj"]],
                                   weights.get(t.get("conv_bias", "")))
        else:
            p = m.params
            nh, nkv, hd = p["heads"], p["kv_heads"], p["head_dim"]
            inv = P.rope_inv_freq(hd, m.position.params["theta"])
            q = P.rope_half_split(P.rms_norm(P.linear(h, weights[t["q_proj"]]).reshape(T, nh, hd), weights[t["q_norm"]], p["qk_norm_eps"]), range(T), inv)
            if p.get("kv_source") is None:
                k = P.rope_half_split(P.rms_norm(P.linear(h, weights[t["k_proj"]]).reshape(T, nkv, hd), weights[t["k_norm"]], p["qk_norm_eps"]), range(T), inv)
                v = P.linear(h, weights[t["v_proj"]]).reshape(T, nkv, hd)
                kv_of_layer[i] = (k, v)
            else:
                k, v = kv_of_layer[p["kv_source"]]
            a = P.linear(P.causal_attention(q, k, v, p["scale"], p.get("window")).reshape(T, nh * hd), weights[t["out_proj"]])
        x = x + a
        h = P.rms_norm(x, weights[L.ffn_norm.weight], L.ffn_norm.eps)
        f = L.ffn.tensors
        x = x + P.swiglu_ffn(h, weights[f["gate"]], weights[f["up"]], weights[f["down"]])
    x = P.rms_norm(x, weights[spec.final_norm.weight], spec.final_norm.eps)
    return P.linear(x, weights[spec.head or spec.embedding])


def hand_spec(hidden=48, vocab=97):
    """Layer 0 attention (owns a cache), layer 1 short conv, layer 2 attention that reads layer 0's
    cache, run order 0, 1, 2, 1: layer 1 runs twice with the same weights and a state per run."""
    from gibbs_amd.config import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec
    rope = PositionSpec("rope", {"theta": 1e4, "rotary_dim": 16, "precision": "f32"})
    layers = []
    for i, kind in enumerate(["attention", "short_conv", "shared"]):
        p = f"l{i}"
        if kind == "short_conv":
            mixer = MixerSpec("short_conv", {"width": hidden, "kernel": 3, "bias": False},
                              {"in_proj": f"{p}.in", "conv": f"{p}.taps", "out_proj": f"{p}.out"})
        else:
            params = {"heads": 3, "kv_heads": 1, "head_dim": 16, "scale": 0.25, "qk_norm": "before", "qk_norm_eps": 1e-5,
                      "window": None}
            tensors = {"q_proj": f"{p}.q", "out_proj": f"{p}.o", "q_norm": f"{p}.qn"}
            if kind == "shared":
                params["kv_source"] = 0
            else:
                tensors.update({"k_proj": f"{p}.k", "v_proj": f"{p}.v", "k_norm": f"{p}.kn"})
            mixer = MixerSpec("attention", params, tensors, rope)
        ffn = FeedForwardSpec("glu", {"inter": 64, "activation": "silu"}, {"gate": f"{p}.w1", "up": f"{p}.w3", "down": f"{p}.w2"})
        layers.append(LayerSpec(p, "pre_norm", NormSpec("rms", 1e-5, f"{p}.n1"), mixer, NormSpec("rms", 1e-5, f"{p}.n2"), ffn))
    return ModelSpec("Hand", hidden, vocab, tuple(layers), (0, 1, 2, 1), "emb", NormSpec("rms", 1e-5, "fn"), "head", 256)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_layer_order_and_shared_cache(name, dtype, tmp_path):
    from gibbs_amd import Engine, Entry
    from gibbs_amd.config.base import ArchConfig
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import random_tensor
    spec = hand_spec()
    decls = DecoderModel(spec).tensor_decls()
    assert not any(d.name in ("l2.k", "l2.v", "l2.kn") for d in decls), "a layer that reads a cache projects no k, v"
    tensors = {d.name: random_tensor(d, 5, torch.bfloat16, std=0.15, gain_std=0.1) for d in decls}

    class Hand(ArchConfig):
        def model_spec(self):
            return spec
    ws = store({k: v.float().numpy() for k, v in tensors.items()}, decls, dtype)
    eng = Engine(config=Hand(), weights=ws, dtype=name, max_tokens=256, max_requests=2, page_size=8)
    assert eng.cache.group_layers == [[0]] and len(eng.cache.state_layout) == 2, "one cache, one state per run of layer 1"
    ids = H.tokens(4, 40, spec.vocab)
    want = plain_spec_forward(spec, {k: v.double().numpy() for k, v in tensors.items()}, ids)
    got = []
    for a, b in [(0, 9), (9, 11), (11, 12), (12, 13), (13, 40)]:
        got.append(eng.step([Entry("r", ids[a:b], list(range(b - a)))]).cpu().numpy())
    H.assert_close(np.concatenate(got), want, name, "hand-built spec")


def window_spec(hidden=40, vocab=83, window=20):
    """Layer 0 attends to all keys, layer 1 to a window of them (other head counts, so a cache group of
    its own), layer 2 is a short convolution."""
    from gibbs_amd.config import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec
    rope = PositionSpec("rope", {"theta": 1e4, "rotary_dim": 16, "precision": "f32"})
    layers = []
    for i, kind in enumerate(["full", "window", "short_conv"]):
        p = f"l{i}"
        if kind == "short_conv":
            mixer = MixerSpec("short_conv", {"width": hidden, "kernel": 3, "bias": False},
                              {"in_proj": f"{p}.in", "conv": f"{p}.taps", "out_proj": f"{p}.out"})
        else:
            heads, kv = (4, 2) if kind == "full" else (3, 1)
            mixer = MixerSpec("attention", {"heads": heads, "kv_heads": kv, "head_dim": 16, "scale": 0.25, "qk_norm": "before",
                                            "qk_norm_eps": 1e-5, "window": window if kind == "window" else None},
                              {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o",
                               "q_norm": f"{p}.qn", "k_norm": f"{p}.kn"}, rope)
        ffn = FeedForwardSpec("glu", {"inter": 56, "activation": "silu"}, {"gate": f"{p}.w1", "up": f"{p}.w3", "down": f"{p}.w2"})
        layers.append(LayerSpec(p, "pre_norm", NormSpec("rms", 1e-5, f"{p}.n1"), mixer, NormSpec("rms", 1e-5, f"{p}.n2"), ffn))
    return ModelSpec("Windowed", hidden, vocab, tuple(layers), (0, 1, 2), "emb", NormSpec("rms", 1e-5, "fn"), None, 512)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_window_group_gives_pages_back_and_they_are_used_again(name, dtype):
    """A model whose layers need different caches: all keys in one group, a window of 20 in another.
    Three requests through the engine, portions beside decoded tokens, in pools of 8-token pages of
    different sizes: 24 pages for the group that keeps every key, 12 for the window's group, which hands
    out 29 pages over the run, so pages that a window has passed are in use again while their first
    owner still runs; the logits equal the plain model's."""
    from gibbs_amd import Engine, Entry
    from gibbs_amd.config.base import ArchConfig
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import random_tensor
    spec = window_spec()
    decls = DecoderModel(spec).tensor_decls()
    tensors = {d.name: random_tensor(d, 9, torch.bfloat16, std=0.15, gain_std=0.1) for d in decls}

    class Windowed(ArchConfig):
        def model_spec(self):
            return spec
    ws = store({k: v.float().numpy() for k, v in tensors.items()}, decls, dtype)
    eng = Engine(config=Windowed(), weights=ws, dtype=name, max_tokens=24 * 8, max_requests=2, page_size=8,
                 group_pages=[24, 12])
    cm = eng.cache
    assert cm.n_groups == 2 and cm.group_layers == [[0], [1]]
    assert [t.shape[1] for t in eng.device_cache.kpages] == [24 + 1, 12 + 1], "every group has the pages of its own pool (and a scratch page)"
    win = 1                                                     # the window's group
    seqs = {"a": H.tokens(1, 150, spec.vocab), "b": H.tokens(2, 40, spec.vocab), "c": H.tokens(3, 40, spec.vocab)}
    plain = {r: plain_spec_forward(spec, {k: v.double().numpy() for k, v in tensors.items()}, ids) for r, ids in seqs.items()}
    got = {r: [] for r in seqs}
    at = {r: 0 for r in seqs}
    owners, used_again = {}, 0                                   # page of the window group -> (request, index in its table)
    def step(parts):
        nonlocal used_again
        entries = [Entry(r, seqs[r][at[r]:at[r] + n], list(range(n))) for r, n in parts]
        rows = eng.step(entries).cpu().numpy()
        i = 0
        for r, n in parts:
            got[r].append(rows[i:i + n]); i += n; at[r] += n
            table = cm.block_table([r], win)[0]
            held = [(j, int(pg)) for j, pg in enumerate(table) if pg >= 0]
            assert len(held) <= 20 // 8 + 2, f"request {r} holds {len(held)} pages of the window group"
            for j, pg in held:
                if pg in owners and owners[pg] != (r, j):
                    used_again += 1
                owners[pg] = (r, j)
            if at[r] == len(seqs[r]):
                eng.release(r)
        cm.check()
    step([("a", 37)])
    step([("a", 1), ("b", 9)])
    for _ in range(15):
        step([("a", 1), ("b", 2)])
    step([("a", 40), ("b", 1)])                                 # b ends (40 tokens)
    step([("a", 2), ("c", 33)])
    for _ in range(7):
        step([("a", 1), ("c", 1)])                              # c ends
    step([("a", 150 - at["a"])])
    assert not any(r in cm for r in seqs) and [cm.free_pages(g) for g in range(2)] == [24, 12]
    assert used_again >= 5, "the pool was meant to be so small that pages a window has passed are used again"
    for r in seqs:
        H.assert_close(np.concatenate(got[r]), plain[r], name, f"windowed model request {r}")


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_captured_decode_loop_past_the_pages_of_a_window_group(name, dtype):
    """The captured decode loop on the model with a window's cache group whose pool (12 pages of 8 tokens) is
    smaller than a request's count of logical pages: the request decodes to 150 tokens (19 logical pages, of
    which the window's group holds 4 at a time), so the loop's block tables must be as wide as the context,
    not as the pool.  Same greedy tokens as stepping the same engine from the host."""
    from gibbs_amd import Engine
    from gibbs_amd.config.base import ArchConfig
    from gibbs_amd.engine.decode import DecodeLoop
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import random_tensor
    spec = window_spec()
    decls = DecoderModel(spec).tensor_decls()
    tensors = {d.name: random_tensor(d, 9, torch.bfloat16, std=0.15, gain_std=0.1) for d in decls}

    class Windowed(ArchConfig):
        def model_spec(self):
            return spec
    prompt = H.tokens(5, 21, spec.vocab)
    tokens = {}
    for mode in ("loop", "steps"):
        ws = store({k: v.float().numpy() for k, v in tensors.items()}, decls, dtype)
        eng = Engine(config=Windowed(), weights=ws, dtype=name, max_tokens=24 * 8, max_requests=2, page_size=8,
                     group_pages=[24, 12], ctx=192)
        first = int(eng.step([("r", prompt, [len(prompt) - 1])]).argmax(-1).item())
        if mode == "loop":
            loop = DecodeLoop(eng, ["r"], [first])
            assert loop.width == [24, 24], "one table entry per logical page of the context"
            for n in (9, 40, 40, 39):                      # past 12 logical pages during the third run
                loop.run(n)
            tokens[mode] = [first] + loop.tokens()[0]
            assert eng.cache.tokens("r") == 21 + 128
            assert (eng.cache.block_table(["r"], 1)[0] >= 0).sum() <= 20 // 8 + 2
        else:
            out = [first]
            for _ in range(128):
                out.append(int(eng.step([("r", [out[-1]], [0])]).argmax(-1).item()))
            tokens[mode] = out
        eng.cache.check()
    assert tokens["loop"] == tokens["steps"]


# --------------------------------------------------------------------------- a toy mixer with its own state
def register_toy():
    """An exponential moving average over time of a projection of the input: state [hidden] per
    request.  Written with framework operations and plain tensor code; nothing in the framework
    knows about it."""
    from gibbs_amd.cache import StateNeed
    from gibbs_amd.ops.linear import linear
    from gibbs_amd.parts import Mixer, register_mixer
    from gibbs_amd.weights import TensorDecl

    @register_mixer("toy_ema")
    class ToyEma(Mixer):
        def state_needs(self):
            # (a float32 average, a count of the request's tokens so far as an integer, and that count modulo 7, 5
            # and 3 in bfloat16: states of other types than float32, one of an odd size)
            return (StateNeed("ema", (self.hidden,)), StateNeed("seen", (1,), "int32"), StateNeed("last", (3,), "bfloat16"))

        def tensor_decls(self):
            return [TensorDecl(self.spec.tensors["proj"], (self.hidden, self.hidden))]

        def bind(self, weights, rt):
            self.rt, self.w = rt, weights[self.spec.tensors["proj"]]

        def forward(self, h, batch, cache):
            u = linear(h, self.w).float()
            decay = self.spec.params["decay"]
            state, seen, last = cache.states["ema"], cache.states["seen"], cache.states["last"]
            assert seen.dtype == torch.int32 and last.dtype == torch.bfloat16 and last.shape[1:] == (3,)
            out = torch.empty_like(u)
            row = 0
            for q, slot in zip(batch.q_lens, batch.slots):
                s = state[slot].clone()
                mods = torch.tensor([7, 5, 3], device=u.device)
                for t in range(q):
                    s = decay * s + u[row + t]
                    out[row + t] = s
                    # (the count of tokens so far and its remainders, as the states hold them)
                    out[row + t, :3] += 0.05 * int(seen[slot, 0]) + 0.5 * last[slot].float()
                    seen[slot, 0] += 1
                    last[slot] = (seen[slot, 0] % mods).bfloat16()
                state[slot] = s
                row += q
            return out.to(self.rt.act_dtype)
    return ToyEma


def toy_config_class():
    from gibbs_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                  register_architecture)
    from gibbs_amd.config.base import ArchConfig

    class ToyConfig(ArchConfig):
        architecture = "ToyEmaForCausalLM"

        def __init__(self, cfg):
            self.cfg = dict(cfg)

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls(cfg)

        def to_dict(self):
            return dict(self.cfg)

        def model_spec(self):
            c, layers = self.cfg, []
            H_, hd = c["width"], c["head_size"]
            for i, kind in enumerate(c["mixers"]):
                p = f"blocks.{i}"
                if kind == "ema":
                    mixer = MixerSpec("toy_ema", {"decay": c["decay"]}, {"proj": f"{p}.ema.proj"})
                else:
                    mixer = MixerSpec("attention", {"heads": c["heads"], "kv_heads": c["heads"], "head_dim": hd,
                                                    "scale": hd ** -0.5, "qk_norm": None, "window": None},
                                      {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o"},
                                      PositionSpec("rope", {"theta": c["theta"], "rotary_dim": hd, "precision": "f32"}))
                ffn = FeedForwardSpec("glu", {"inter": c["ff"], "activation": "silu"},
                                      {"gate": f"{p}.g", "up": f"{p}.u", "down": f"{p}.d"})
                layers.append(LayerSpec(p, "pre_norm", NormSpec("rms", c["eps"], f"{p}.n1"), mixer,
                                        NormSpec("rms", c["eps"], f"{p}.n2"), ffn))
            return ModelSpec(self.architecture, H_, c["vocab"], tuple(layers), tuple(range(len(layers))), "tok",
                             NormSpec("rms", c["eps"], "out_norm"), None, c["max_len"])
    register_architecture("ToyEmaForCausalLM", ToyConfig, aliases=("toy_ema",))
    return ToyConfig


def toy_plain(cfg, w, ids):
    T, hd, nh = len(ids), cfg["head_size"], cfg["heads"]
    x = P.embedding(w["tok"], ids)
    for i, kind in enumerate(cfg["mixers"]):
        p = f"blocks.{i}"
        h = P.rms_norm(x, w[f"{p}.n1"], cfg["eps"])
        if kind == "ema":
            u, s, a = P.linear(h, w[f"{p}.ema.proj"]), np.zeros(cfg["width"]), []
            for t in range(T):
                s = cfg["decay"] * s + u[t]
                a.append(s.copy())
                a[-1][:3] += 0.05 * t + 0.5 * np.array([t % 7, t % 5, t % 3])
            a = np.stack(a)
        else:
            inv = P.rope_inv_freq(hd, cfg["theta"])
            q = P.rope_half_split(P.linear(h, w[f"{p}.q"]).reshape(T, nh, hd), range(T), inv)
            k = P.rope_half_split(P.linear(h, w[f"{p}.k"]).reshape(T, nh, hd), range(T), inv)
            v = P.linear(h, w[f"{p}.v"]).reshape(T, nh, hd)
            a = P.linear(P.causal_attention(q, k, v, hd ** -0.5).reshape(T, nh * hd), w[f"{p}.o"])
        x = x + a
        x = x + P.swiglu_ffn(P.rms_norm(x, w[f"{p}.n2"], cfg["eps"]), w[f"{p}.g"], w[f"{p}.u"], w[f"{p}.d"])
    return P.linear(P.rms_norm(x, w["out_norm"], cfg["eps"]), w["tok"])


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_toy_mixer_with_state_registers_builds_and_steps(name, dtype, tmp_path):
    from gibbs_amd import Engine, Entry
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    register_toy()
    Toy = toy_config_class()
    cfg = {"architectures": ["ToyEmaForCausalLM"], "width": 40, "heads": 2, "head_size": 16, "ff": 56, "vocab": 83,
           "mixers": ["ema", "attn", "ema"], "decay": 0.75, "theta": 1e4, "eps": 1e-5, "max_len": 128}
    folder = str(tmp_path / "toy")
    config = Toy.from_dict(cfg)
    write_random_model(folder, config, DecoderModel(config.model_spec()).tensor_decls(), seed=2, std=0.15, gain_std=0.1)
    assert json.load(open(os.path.join(folder, "config.json")))["mixers"] == ["ema", "attn", "ema"]
    eng = Engine(folder, dtype=name, max_tokens=128, max_requests=2, page_size=8)     # the class is chosen by config.json
    assert [type(b.mixer).__name__ for b in eng.model.blocks] == ["ToyEma", "AttentionMixer", "ToyEma"]
    assert eng.plan.op_count() == 6, "the toy mixer is a part of the native step's program like any other"
    assert set(eng.cache.state_layout) == {(i, n) for i in (0, 2) for n in ("ema", "seen", "last")}
    assert eng.cache.slot_floats == 2 * (40 + 1 + 2), "a float32 row, an integer and three bfloat16 values in two words"
    weights, _ = P.load_model_dir(folder)
    seqs = {"a": H.tokens(1, 30, 83), "b": H.tokens(2, 17, 83)}
    got = {}
    # a (portions) beside b (tokens one by one), b ends first and c takes its slot: the state must be cleared
    plan = [[("a", 0, 6), ("b", 0, 4)], [("a", 6, 8), ("b", 4, 5)], [("a", 8, 9), ("b", 5, 17)], [("a", 9, 30)]]
    for step in plan:
        out = eng.step([Entry(r, seqs[r][a:b], list(range(b - a))) for r, a, b in step]).cpu().numpy()
        at = 0
        for r, a, b in step:
            got.setdefault(r, []).append(out[at:at + b - a]); at += b - a
    eng.release("b")
    seqs["c"] = H.tokens(3, 9, 83)
    got["c"] = [eng.step([Entry("c", seqs["c"], list(range(9)))]).cpu().numpy()]
    assert eng.cache.slot("c") != eng.cache.slot("a")
    for r, ids in seqs.items():
        H.assert_close(np.concatenate(got[r]), toy_plain(cfg, weights, ids), name, f"toy model request {r}")


# --------------------------------------------------------------------------- a toy routed feed-forward and a toy position encoding
def register_toy_routed():
    """A feed-forward that routes every token to its two best of E small gated experts (router
    logits and their softmax in float32, the two weights renormalised), and a rotary encoding whose
    positions are stretched by a factor.  Both are written with framework operations and plain
    tensor code and are registered from here."""
    from gibbs_amd import ops
    from gibbs_amd.ops.linear import linear
    from gibbs_amd.parts import FeedForward, PositionEncoding, Rotation, register_feed_forward, register_position
    from gibbs_amd.weights import TensorDecl

    @register_feed_forward("toy_routed")
    class ToyRouted(FeedForward):
        def tensor_decls(self):
            p, t = self.spec.params, self.spec.tensors
            decls = [TensorDecl(t["router"], (p["experts"], self.hidden))]
            for e in range(p["experts"]):
                decls += [TensorDecl(t["gate"].format(e=e), (p["inter"], self.hidden)),
                          TensorDecl(t["up"].format(e=e), (p["inter"], self.hidden)),
                          TensorDecl(t["down"].format(e=e), (self.hidden, p["inter"]))]
            return decls

        def bind(self, weights, rt):
            self.rt, t = rt, self.spec.tensors
            self.router = weights[t["router"]]
            self.experts = [(torch.cat([weights[t["gate"].format(e=e)], weights[t["up"].format(e=e)]]).contiguous(),
                             weights[t["down"].format(e=e)]) for e in range(self.spec.params["experts"])]

        def forward(self, h, batch):
            logits = linear(h, self.router, out_dtype=torch.float32)
            top, idx = torch.softmax(logits, dim=-1).topk(2, dim=-1)
            top = top / top.sum(-1, keepdim=True)
            out = torch.zeros((h.shape[0], self.hidden), dtype=torch.float32, device=h.device)
            for e, (w_gate_up, w_down) in enumerate(self.experts):
                rows, which = (idx == e).nonzero(as_tuple=True)
                if rows.numel():
                    y = linear(ops.glu(linear(h[rows].contiguous(), w_gate_up)), w_down).float()
                    out.index_add_(0, rows, y * top[rows, which, None])
            return out.to(self.rt.act_dtype)

    @register_position("toy_stretched_rope")
    class StretchedRope(PositionEncoding):
        """Pairs (2j, 2j + 1) turned by pos / stretch * theta^(-2j/dim): a rotation, which the attention
        mixer's kernels apply themselves from the tables that `rotation()` hands over."""
        def bind(self, weights, rt):
            p = self.spec.params
            self.rt = rt
            inv = np.array([p["theta"] ** (-2.0 * j / self.head_dim) / p["stretch"] for j in range(self.head_dim // 2)])
            self.inv_freq = torch.tensor(inv, dtype=torch.float32, device=rt.device)
            self.cos_sin = ops.rope_table(self.inv_freq, rt.max_positions) if rt.max_positions > 0 else None

        def rotation(self):
            return Rotation(self.inv_freq, self.head_dim, "interleaved", self.cos_sin)


def routed_config_class():
    from gibbs_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                  register_architecture)
    from gibbs_amd.config.base import ArchConfig

    class RoutedConfig(ArchConfig):
        architecture = "ToyRoutedForCausalLM"

        def __init__(self, cfg):
            self.cfg = dict(cfg)

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls(cfg)

        def to_dict(self):
            return dict(self.cfg)

        def model_spec(self):
            c, layers = self.cfg, []
            H_, hd = c["width"], c["head_size"]
            for i, routed in enumerate(c["routed"]):
                p = f"l.{i}"
                mixer = MixerSpec("attention", {"heads": c["heads"], "kv_heads": 1, "head_dim": hd, "scale": hd ** -0.5,
                                                "qk_norm": None, "window": None},
                                  {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o"},
                                  PositionSpec("toy_stretched_rope", {"theta": c["theta"], "stretch": c["stretch"]}))
                if routed:
                    ffn = FeedForwardSpec("toy_routed", {"experts": c["experts"], "inter": c["expert_ff"]},
                                          {"router": f"{p}.router", "gate": p + ".e{e}.g", "up": p + ".e{e}.u",
                                           "down": p + ".e{e}.d"})
                else:
                    ffn = FeedForwardSpec("glu", {"inter": c["ff"], "activation": "silu"},
                                          {"gate": f"{p}.g", "up": f"{p}.u", "down": f"{p}.d"})
                layers.append(LayerSpec(p, "pre_norm", NormSpec("rms", c["eps"], f"{p}.n1"), mixer,
                                        NormSpec("rms", c["eps"], f"{p}.n2"), ffn))
            return ModelSpec(self.architecture, H_, c["vocab"], tuple(layers), tuple(range(len(layers))), "tok",
                             NormSpec("rms", c["eps"], "out_norm"), None, c["max_len"])
    register_architecture("ToyRoutedForCausalLM", RoutedConfig, aliases=("toy_routed",))
    return RoutedConfig


def routed_plain(cfg, w, ids):
    """Whole sequence, float64; also returns the smallest gap between a token's second and third
    router probability (a routing decision that close could fall either way in lower precision)."""
    T, hd, nh = len(ids), cfg["head_size"], cfg["heads"]
    inv = np.array([cfg["theta"] ** (-2.0 * j / hd) / cfg["stretch"] for j in range(hd // 2)], dtype=np.float32)

    def turn(x):       # pairs (2j, 2j + 1), angle = float32(pos) * inv_freq[j] as a float32 product
        out = x.copy()
        for t in range(T):
            for j in range(hd // 2):
                a = float(np.float32(np.float32(t) * inv[j]))
                c, s = math.cos(a), math.sin(a)
                out[t, :, 2 * j] = x[t, :, 2 * j] * c - x[t, :, 2 * j + 1] * s
                out[t, :, 2 * j + 1] = x[t, :, 2 * j] * s + x[t, :, 2 * j + 1] * c
        return out
    x, gap = P.embedding(w["tok"], ids), np.inf
    for i, routed in enumerate(cfg["routed"]):
        p = f"l.{i}"
        h = P.rms_norm(x, w[f"{p}.n1"], cfg["eps"])
        q = turn(P.linear(h, w[f"{p}.q"]).reshape(T, nh, hd))
        k = turn(P.linear(h, w[f"{p}.k"]).reshape(T, 1, hd))
        v = P.linear(h, w[f"{p}.v"]).reshape(T, 1, hd)
        x = x + P.linear(P.causal_attention(q, k, v, hd ** -0.5).reshape(T, nh * hd), w[f"{p}.o"])
        h = P.rms_norm(x, w[f"{p}.n2"], cfg["eps"])
        if routed:
            logits = P.linear(h, w[f"{p}.router"])
            prob = np.exp(logits - logits.max(-1, keepdims=True))
            prob /= prob.sum(-1, keepdims=True)
            m = np.zeros_like(x)
            for t in range(T):
                order = np.argsort(-prob[t], kind="stable")
                gap = min(gap, prob[t, order[1]] - prob[t, order[2]])
                for e in order[:2]:
                    y = P.swiglu_ffn(h[t:t + 1], w[f"{p}.e{e}.g"], w[f"{p}.e{e}.u"], w[f"{p}.e{e}.d"])[0]
                    m[t] += prob[t, e] / (prob[t, order[0]] + prob[t, order[1]]) * y
        else:
            m = P.swiglu_ffn(h, w[f"{p}.g"], w[f"{p}.u"], w[f"{p}.d"])
        x = x + m
    return P.linear(P.rms_norm(x, w["out_norm"], cfg["eps"]), w["tok"]), gap


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_toy_routed_feed_forward_and_position_encoding(name, dtype, tmp_path):
    """Parts of other kinds than the architecture's own, chosen layer by layer: a routed feed-forward
    in one layer beside the dense one in the other, and a position encoding of the test's own in
    both attention mixers.  Registered, built from config.json and stepped in portions and single
    tokens (general path and fused decode path) without a change to the framework's files."""
    from gibbs_amd import Engine, Entry
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    register_toy_routed()
    Routed = routed_config_class()
    cfg = {"architectures": ["ToyRoutedForCausalLM"], "width": 48, "heads": 3, "head_size": 16, "ff": 72, "vocab": 91,
           "routed": [True, False], "experts": 4, "expert_ff": 24, "theta": 500.0, "stretch": 1.75, "eps": 1e-6,
           "max_len": 96}
    folder = str(tmp_path / "routed")
    config = Routed.from_dict(cfg)
    write_random_model(folder, config, DecoderModel(config.model_spec()).tensor_decls(), seed=9, std=0.2, gain_std=0.1)
    eng = Engine(folder, dtype=name, max_tokens=128, max_requests=2, page_size=8)
    assert [type(b.ffn).__name__ for b in eng.model.blocks] == ["ToyRouted", "GluFeedForward"]
    assert all(type(b.mixer.position).__name__ == "StretchedRope" for b in eng.model.blocks)
    weights, _ = P.load_model_dir(folder)
    ids = H.tokens(4, 40, 91)
    want, gap = routed_plain(cfg, weights, ids)
    assert gap > 1e-2, f"routing decisions too close to call in bfloat16 (gap {gap:.3e}): take another seed"
    got = []
    for a, b in [(0, 11), (11, 13), (13, 14), (14, 15), (15, 37), (37, 38), (38, 39), (39, 40)]:
        got.append(eng.step([Entry("r", ids[a:b], list(range(b - a)))]).cpu().numpy())
    H.assert_close(np.concatenate(got), want, name, "toy routed feed-forward, stretched positions")


# --------------------------------------------------------------------------- positions that are no rotation, values wider than keys, other activations
def register_toy_positions_and_wide_values():
    """Two position encodings that are no rotation (a linear bias on the scores by distance; a learned
    vector per position added to q and k), and an attention mixer of the test's own whose values have
    another head size than its keys and whose pages it reads and writes with plain tensor code.  All
    registered from here; the framework's attention mixer, cache manager and kernels take them as they are."""
    from gibbs_amd.cache import CacheNeed
    from gibbs_amd.ops.linear import linear
    from gibbs_amd.parts import Mixer, PositionEncoding, register_mixer, register_position
    from gibbs_amd.weights import TensorDecl
    from gibbs_amd.weights.loader import FLOAT32

    @register_position("toy_distance_bias")
    class DistanceBias(PositionEncoding):
        """score(q at p, key at k) += slope_h * (k - p), slope_h = base^-(h + 1)."""
        def score_slopes(self, heads):
            base = float(self.spec.params["base"])
            return torch.tensor([base ** -(h + 1) for h in range(heads)], dtype=torch.float32, device=self.rt.device)

    @register_position("toy_learned_offsets")
    class LearnedOffsets(PositionEncoding):
        """q and k of position p get row p of a learned table [positions, head_dim] added (every head the same)."""
        def tensor_decls(self):
            return [TensorDecl(self.spec.tensors["table"], (self.spec.params["positions"], self.head_dim), FLOAT32)]

        def bind(self, weights, rt):
            self.rt, self.table = rt, weights[self.spec.tensors["table"]]

        def apply(self, q, k, batch):
            rows = self.table[batch.pos[:q.shape[0]].long()].to(q.dtype)[:, None, :]
            q += rows
            if k is not None:
                k += rows

    @register_mixer("toy_wide_values")
    class WideValues(Mixer):
        """Causal attention without position encoding, keys of `head_dim`, values of `v_head_dim`."""
        def __init__(self, spec, hidden, layer_index):
            super().__init__(spec, hidden, layer_index)
            p = spec.params
            self.heads, self.hd, self.vd = p["heads"], p["head_dim"], p["v_head_dim"]

        def cache_need(self):
            return CacheNeed(self.heads, self.hd, v_head_dim=self.vd)

        def tensor_decls(self):
            t, n = self.spec.tensors, self.heads
            return [TensorDecl(t["q"], (n * self.hd, self.hidden)), TensorDecl(t["k"], (n * self.hd, self.hidden)),
                    TensorDecl(t["v"], (n * self.vd, self.hidden)), TensorDecl(t["o"], (self.hidden, n * self.vd))]

        def bind(self, weights, rt):
            self.rt = rt
            self.w = {r: weights[self.spec.tensors[r]] for r in "qkvo"}

        def forward(self, h, batch, cache):
            n, ps = self.heads, cache.kpages.shape[2]
            assert cache.kpages.shape[3] == self.hd and cache.vpages.shape[3] == self.vd
            q = linear(h, self.w["q"]).unflatten(1, (n, self.hd))
            k = linear(h, self.w["k"]).unflatten(1, (n, self.hd))
            v = linear(h, self.w["v"]).unflatten(1, (n, self.vd))
            table = batch.tables[cache.group]
            out = torch.empty((h.shape[0], n, self.vd), dtype=torch.float32, device=h.device)
            row = 0
            for r, (q_len, ctx) in enumerate(zip(batch.q_lens, batch.ctx_lens)):
                pos = torch.arange(ctx, ctx + q_len, device=h.device)
                pages = table[r, pos // ps].long()
                cache.kpages[pages, :, pos % ps] = k[row:row + q_len]
                cache.vpages[pages, :, pos % ps] = v[row:row + q_len]
                held = table[r, :-(-(ctx + q_len) // ps)].long()
                keys = cache.kpages[held].transpose(1, 2).reshape(-1, n, self.hd)[:ctx + q_len].float()
                vals = cache.vpages[held].transpose(1, 2).reshape(-1, n, self.vd)[:ctx + q_len].float()
                s = torch.einsum("thd,lhd->htl", q[row:row + q_len].float(), keys) * self.hd ** -0.5
                s = s.masked_fill(torch.arange(ctx + q_len, device=h.device)[None, None, :] > pos[None, :, None], -torch.inf)
                out[row:row + q_len] = torch.einsum("htl,lhd->thd", s.softmax(-1), vals)
                row += q_len
            return linear(out.flatten(1).to(self.rt.act_dtype).contiguous(), self.w["o"])


def wide_config_class():
    from gibbs_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                  register_architecture)
    from gibbs_amd.config.base import ArchConfig

    class WideConfig(ArchConfig):
        architecture = "ToyWideForCausalLM"

        def __init__(self, cfg):
            self.cfg = dict(cfg)

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls(cfg)

        def to_dict(self):
            return dict(self.cfg)

        def model_spec(self):
            c, layers = self.cfg, []
            H_, hd = c["width"], c["head_size"]
            attn = {"heads": c["heads"], "kv_heads": c["kv_heads"], "head_dim": hd, "scale": hd ** -0.5,
                    "qk_norm": "before", "qk_norm_eps": c["eps"], "window": None}
            for i, kind in enumerate(c["mixers"]):
                p = f"l.{i}"
                names = {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o",
                         "q_norm": f"{p}.qn", "k_norm": f"{p}.kn"}
                if kind == "bias":
                    mixer = MixerSpec("attention", attn, names, PositionSpec("toy_distance_bias", {"base": c["slope_base"]}))
                elif kind == "learned":
                    mixer = MixerSpec("attention", attn, names,
                                      PositionSpec("toy_learned_offsets", {"positions": c["max_len"]}, {"table": f"{p}.pos"}))
                else:
                    mixer = MixerSpec("toy_wide_values", {"heads": c["heads"], "head_dim": hd, "v_head_dim": c["v_head_size"]},
                                      {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"})
                ffn = FeedForwardSpec("glu", {"inter": c["ff"], "activation": c["activations"][i]},
                                      {"gate": f"{p}.g", "up": f"{p}.u", "down": f"{p}.d"})
                layers.append(LayerSpec(p, "pre_norm", NormSpec("rms", c["eps"], f"{p}.n1"), mixer,
                                        NormSpec("rms", c["eps"], f"{p}.n2"), ffn))
            return ModelSpec(self.architecture, H_, c["vocab"], tuple(layers), tuple(range(len(layers))), "tok",
                             NormSpec("rms", c["eps"], "out_norm"), None, c["max_len"])
    register_architecture("ToyWideForCausalLM", WideConfig, aliases=("toy_wide",))
    return WideConfig


def wide_plain(cfg, w, ids):
    T, hd, vd, nh, nkv = len(ids), cfg["head_size"], cfg["v_head_size"], cfg["heads"], cfg["kv_heads"]
    acts = {"silu": lambda g: g / (1 + np.exp(-g)), "relu": lambda g: np.maximum(g, 0.0),
            "gelu_tanh": lambda g: 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))),
            "gelu": lambda g: 0.5 * g * (1 + np.vectorize(math.erf)(g / math.sqrt(2)))}
    x = P.embedding(w["tok"], ids)
    for i, kind in enumerate(cfg["mixers"]):
        p = f"l.{i}"
        h = P.rms_norm(x, w[f"{p}.n1"], cfg["eps"])
        if kind == "wide":
            q, k = (P.linear(h, w[f"{p}.{r}"]).reshape(T, nh, hd) for r in "qk")
            v = P.linear(h, w[f"{p}.v"]).reshape(T, nh, vd)
            a = P.causal_attention(q, k, v, hd ** -0.5).reshape(T, nh * vd)
        else:
            q = P.rms_norm(P.linear(h, w[f"{p}.q"]).reshape(T, nh, hd), w[f"{p}.qn"], cfg["eps"])
            k = P.rms_norm(P.linear(h, w[f"{p}.k"]).reshape(T, nkv, hd), w[f"{p}.kn"], cfg["eps"])
            v = P.linear(h, w[f"{p}.v"]).reshape(T, nkv, hd)
            if kind == "learned":
                q, k = q + w[f"{p}.pos"][:T, None, :], k + w[f"{p}.pos"][:T, None, :]
                a = P.causal_attention(q, k, v, hd ** -0.5)
            else:   # scores biased by the distance
                a = np.zeros((T, nh, hd))
                for t in range(T):
                    for hh in range(nh):
                        g = hh // (nh // nkv)
                        s = (k[:t + 1, g] @ q[t, hh]) * hd ** -0.5 + cfg["slope_base"] ** -(hh + 1) * (np.arange(t + 1) - t)
                        e = np.exp(s - s.max())
                        a[t, hh] = (e / e.sum()) @ v[:t + 1, g]
            a = a.reshape(T, nh * hd)
        x = x + P.linear(a, w[f"{p}.o"])
        h = P.rms_norm(x, w[f"{p}.n2"], cfg["eps"])
        x = x + P.linear(acts[cfg["activations"][i]](P.linear(h, w[f"{p}.g"])) * P.linear(h, w[f"{p}.u"]), w[f"{p}.d"])
    return P.linear(P.rms_norm(x, w["out_norm"], cfg["eps"]), w["tok"])


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_positions_that_are_no_rotation_and_values_wider_than_keys(name, dtype, tmp_path):
    """The attention mixer with a position encoding that biases the scores by distance and with one that
    changes q and k itself (a learned table of its own in the checkpoint), a mixer from outside whose
    cache group has values of another head size than keys, and feed-forwards with three other
    activations (general path and the fused decode epilogue): registered, built from config.json and
    stepped in portions and single tokens of two requests, against a plain implementation."""
    from gibbs_amd import Engine, Entry
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    register_toy_positions_and_wide_values()
    Wide = wide_config_class()
    cfg = {"architectures": ["ToyWideForCausalLM"], "width": 64, "heads": 4, "kv_heads": 2, "head_size": 16,
           "v_head_size": 24, "ff": 96, "vocab": 77, "mixers": ["bias", "wide", "learned", "bias"],
           "activations": ["gelu_tanh", "relu", "gelu", "silu"], "slope_base": 1.6, "eps": 1e-5, "max_len": 96}
    folder = str(tmp_path / "wide")
    config = Wide.from_dict(cfg)
    write_random_model(folder, config, DecoderModel(config.model_spec()).tensor_decls(), seed=4, std=0.2, gain_std=0.2)
    eng = Engine(folder, dtype=name, max_tokens=160, max_requests=2, page_size=8)
    needs = eng.cache.group_needs
    assert len(needs) == 2 and {n.value_dim for n in needs} == {16, 24}, "values of another head size are a group of their own"
    assert [tuple(t.shape[-2:]) for t in eng.device_cache.vpages] == [(8, n.value_dim) for n in needs]
    weights, _ = P.load_model_dir(folder)
    seqs = {"a": H.tokens(5, 41, 77), "b": H.tokens(6, 23, 77)}
    plan = [[("a", 0, 9)], [("a", 9, 10), ("b", 0, 13)], [("a", 10, 11), ("b", 13, 14)], [("a", 11, 12), ("b", 14, 15)],
            [("a", 12, 35), ("b", 15, 16)], [("a", 35, 36), ("b", 16, 23)]] + [[("a", t, t + 1)] for t in range(36, 41)]
    got = {}
    for step in plan:
        out = eng.step([Entry(r, seqs[r][a:b], list(range(b - a))) for r, a, b in step]).cpu().numpy()
        at = 0
        for r, a, b in step:
            got.setdefault(r, []).append(out[at:at + b - a]); at += b - a
    for r, ids in seqs.items():
        H.assert_close(np.concatenate(got[r]), wide_plain(cfg, weights, ids), name, f"toy positions / wide values request {r}")


# --------------------------------------------------------------------------- other arrangements of a block's parts
def test_an_arrangement_from_outside_is_a_program_of_the_native_step(tmp_path):
    """A block in which mixer and feed-forward read the same normed rows and both add to the stream
    (x += mixer(norm(x)) + ffn(norm(x))), registered from here: one norm and two bodies by role, laid
    down as norm, body, body, add, add, drop operations of the native step.  It knows nothing of how
    deltas travel (pending deltas, float32 partial sums).  Both precisions, portions and single tokens."""
    from gibbs_amd import Engine, Entry
    from gibbs_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                  register_architecture)
    from gibbs_amd.config.base import ArchConfig
    from gibbs_amd.parts import Block, DecoderModel, register_arrangement
    from gibbs_amd.weights import write_random_model

    @register_arrangement("toy_parallel")
    class Parallel(Block):
        def emit(self, plan, caches):
            h = plan.normed(self.norm.emit(plan))
            a = plan.apply(self.mixer.emit(plan, caches["mixer"]), h)
            m = plan.apply(self.ffn.emit(plan), h)
            plan.add(a)
            plan.add(m)
            plan.drop(h)

    class ParallelConfig(ArchConfig):
        architecture = "ToyParallelForCausalLM"

        def __init__(self, cfg):
            self.cfg = dict(cfg)

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls(cfg)

        def to_dict(self):
            return dict(self.cfg)

        def model_spec(self):
            c, layers = self.cfg, []
            for i, kind in enumerate(c["mixers"]):
                p = f"b{i}"
                if kind == "conv":
                    mixer = MixerSpec("short_conv", {"width": c["width"], "kernel": 3, "bias": False},
                                      {"in_proj": f"{p}.in", "conv": f"{p}.taps", "out_proj": f"{p}.out"})
                else:
                    mixer = MixerSpec("attention", {"heads": 2, "kv_heads": 1, "head_dim": 16, "scale": 0.25, "qk_norm": None,
                                                    "window": None},
                                      {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o"},
                                      PositionSpec("rope", {"theta": 1e4, "rotary_dim": 16, "precision": "f32"}))
                ffn = FeedForwardSpec("glu", {"inter": c["ff"], "activation": "silu"}, {"gate": f"{p}.g", "up": f"{p}.u", "down": f"{p}.d"})
                layers.append(LayerSpec(p, "toy_parallel", parts=[("norm", NormSpec("rms", c["eps"], f"{p}.n")), ("mixer", mixer),
                                                                  ("ffn", ffn)]))
            return ModelSpec(self.architecture, c["width"], c["vocab"], tuple(layers), tuple(range(len(layers))), "tok",
                             NormSpec("rms", c["eps"], "out_norm"), None, 128)
    register_architecture("ToyParallelForCausalLM", ParallelConfig)
    cfg = {"architectures": ["ToyParallelForCausalLM"], "width": 48, "ff": 80, "vocab": 61, "mixers": ["conv", "attn", "conv"],
           "eps": 1e-5}
    config = ParallelConfig(cfg)
    folder = str(tmp_path / "parallel")
    write_random_model(folder, config, DecoderModel(config.model_spec()).tensor_decls(), seed=6, std=0.2, gain_std=0.2)
    w, _ = P.load_model_dir(folder)
    ids = H.tokens(8, 50, 61)
    T = len(ids)
    x = P.embedding(w["tok"], ids)
    for i, kind in enumerate(cfg["mixers"]):
        p = f"b{i}"
        h = P.rms_norm(x, w[f"{p}.n"], cfg["eps"])
        if kind == "conv":
            a = P.short_conv_mixer(h, w[f"{p}.in"], w[f"{p}.taps"], w[f"{p}.out"])
        else:
            inv = P.rope_inv_freq(16, 1e4)
            q = P.rope_half_split(P.linear(h, w[f"{p}.q"]).reshape(T, 2, 16), range(T), inv)
            k = P.rope_half_split(P.linear(h, w[f"{p}.k"]).reshape(T, 1, 16), range(T), inv)
            a = P.linear(P.causal_attention(q, k, P.linear(h, w[f"{p}.v"]).reshape(T, 1, 16), 0.25).reshape(T, 32), w[f"{p}.o"])
        x = x + a + P.swiglu_ffn(h, w[f"{p}.g"], w[f"{p}.u"], w[f"{p}.d"])
    want = P.linear(P.rms_norm(x, w["out_norm"], cfg["eps"]), w["tok"])
    for name in ("float32", "bfloat16"):
        eng = Engine(folder, dtype=name, max_tokens=128, max_requests=1, page_size=8)
        assert [type(b).__name__ for b in eng.model.blocks] == ["Parallel"] * 3
        assert eng.plan.op_count() == 3 * 6, "the step is the native program that the blocks laid down"
        got = [eng.step([Entry("r", ids[a:b], list(range(b - a)))]).cpu().numpy()
               for a, b in [(0, 21), (21, 23), (23, 24), (24, 25), (25, 49), (49, 50)]]
        H.assert_close(np.concatenate(got), want, name, f"parallel arrangement {name}")


def test_layers_with_two_mixers_and_layers_without_a_feed_forward(tmp_path):
    """A layer is whatever parts its spec names, by role: here layers of the kind "mix" hold a norm and
    TWO mixers that read the same normed rows (a short convolution with its state and an attention with
    its cache pages: two cache owners in one layer) and no feed-forward; layers of the kind "ff" hold a
    norm and a feed-forward and no mixer.  The arrangement, registered from here, lays down whichever
    parts a layer has.  Cache manager, step function and scheduler take the model as it is."""
    from gibbs_amd import Engine, Entry, generate
    from gibbs_amd.config import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                  register_architecture)
    from gibbs_amd.config.base import ArchConfig
    from gibbs_amd.parts import Block, DecoderModel, register_arrangement
    from gibbs_amd.weights import write_random_model

    @register_arrangement("toy_all_of_them")
    class AllOfThem(Block):
        """x += sum of every body's delta of norm(x)."""
        def emit(self, plan, caches):
            h = plan.normed(self.norm.emit(plan))
            deltas = [plan.apply(part.emit(plan, caches[role]) if role in caches else part.emit(plan), h)
                      for role, part in self.named.items() if role != "norm"]
            for d in deltas:
                plan.add(d)
            plan.drop(h)

    class MixConfig(ArchConfig):
        architecture = "ToyTwoMixersForCausalLM"

        def __init__(self, cfg):
            self.cfg = dict(cfg)

        @classmethod
        def from_dict(cls, cfg, tensors=None):
            return cls(cfg)

        def to_dict(self):
            return dict(self.cfg)

        def model_spec(self):
            c, layers = self.cfg, []
            for i, kind in enumerate(c["layers"]):
                p = f"l{i}"
                parts = [("norm", NormSpec("rms", c["eps"], f"{p}.n"))]
                if kind == "mix":
                    parts.append(("local", MixerSpec("short_conv", {"width": c["width"], "kernel": 4, "bias": True},
                                                     {"in_proj": f"{p}.in", "conv": f"{p}.taps", "out_proj": f"{p}.out",
                                                      "conv_bias": f"{p}.cb"})))
                    parts.append(("global", MixerSpec("attention", {"heads": 4, "kv_heads": 2, "head_dim": 16, "scale": 0.25,
                                                                     "qk_norm": None, "window": None},
                                                      {"q_proj": f"{p}.q", "k_proj": f"{p}.k", "v_proj": f"{p}.v", "out_proj": f"{p}.o"},
                                                      PositionSpec("rope", {"theta": 1e4, "rotary_dim": 16, "precision": "f32"}))))
                else:
                    parts.append(("ffn", FeedForwardSpec("glu", {"inter": c["ff"], "activation": "silu"},
                                                         {"gate": f"{p}.g", "up": f"{p}.u", "down": f"{p}.d"})))
                layers.append(LayerSpec(p, "toy_all_of_them", parts=parts))
            return ModelSpec(self.architecture, c["width"], c["vocab"], tuple(layers), tuple(range(len(layers))), "tok",
                             NormSpec("rms", c["eps"], "out_norm"), None, 128)
    register_architecture("ToyTwoMixersForCausalLM", MixConfig)
    cfg = {"architectures": ["ToyTwoMixersForCausalLM"], "width": 64, "ff": 96, "vocab": 67, "layers": ["mix", "ff", "mix"],
           "eps": 1e-5}
    config = MixConfig(cfg)
    folder = str(tmp_path / "two_mixers")
    write_random_model(folder, config, DecoderModel(config.model_spec()).tensor_decls(), seed=3, std=0.2, gain_std=0.2, bias_std=0.1)
    w, _ = P.load_model_dir(folder)

    def plain(ids):
        T = len(ids)
        x = P.embedding(w["tok"], ids)
        for i, kind in enumerate(cfg["layers"]):
            p = f"l{i}"
            h = P.rms_norm(x, w[f"{p}.n"], cfg["eps"])
            if kind == "mix":
                inv = P.rope_inv_freq(16, 1e4)
                q = P.rope_half_split(P.linear(h, w[f"{p}.q"]).reshape(T, 4, 16), range(T), inv)
                k = P.rope_half_split(P.linear(h, w[f"{p}.k"]).reshape(T, 2, 16), range(T), inv)
                att = P.linear(P.causal_attention(q, k, P.linear(h, w[f"{p}.v"]).reshape(T, 2, 16), 0.25).reshape(T, 64), w[f"{p}.o"])
                x = x + P.short_conv_mixer(h, w[f"{p}.in"], w[f"{p}.taps"], w[f"{p}.out"], w[f"{p}.cb"]) + att
            else:
                x = x + P.swiglu_ffn(h, w[f"{p}.g"], w[f"{p}.u"], w[f"{p}.d"])
        return P.linear(P.rms_norm(x, w["out_norm"], cfg["eps"]), w["tok"])
    seqs = {"a": H.tokens(8, 45, 67), "b": H.tokens(9, 20, 67)}
    steps = [[("a", 0, 17)], [("a", 17, 19), ("b", 0, 9)], [("a", 19, 20), ("b", 9, 10)], [("a", 20, 21), ("b", 10, 11)],
             [("a", 21, 44), ("b", 11, 12)], [("a", 44, 45), ("b", 12, 20)]]
    for name in ("float32", "bfloat16"):
        eng = Engine(folder, dtype=name, max_tokens=128, max_requests=2, page_size=8)
        # two cache owners in each "mix" layer: the convolution's state and the attention's pages
        assert eng.model.cache_owners() == [(0, "local"), (0, "global"), (2, "local"), (2, "global")]
        assert eng.cache.group_layers == [[1, 3]] and set(eng.cache.state_layout) == {(0, "conv"), (2, "conv")}
        got = {}
        for step in steps:
            out = eng.step([Entry(r, seqs[r][a:b], list(range(b - a))) for r, a, b in step]).cpu().numpy()
            at = 0
            for r, a, b in step:
                got.setdefault(r, []).append(out[at:at + b - a]); at += b - a
        for r, ids in seqs.items():
            H.assert_close(np.concatenate(got[r]), plain(ids), name, f"two mixers in a layer, request {r}, {name}")
        eng.release("a"); eng.release("b")
        if name == "float32":
            out = generate(eng, [seqs["b"][:7]], max_tokens=6, temperature=0.0, ignore_eos=True)[0].tokens
            seq = list(seqs["b"][:7])
            for t in out:
                assert t == P.argmax_first(plain(seq)[-1])
                seq.append(t)

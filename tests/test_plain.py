"""Pins of the plain implementation beside the reference's text: vectors the reference's
own tests hold, special cases that reduce to a library routine, and invariants.  Each is
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a
swapped gate) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests.plain import golden_fixture as G
from tests.plain import lfm2_plain as P

rng = np.random.default_rng(7)


def test_rmsnorm_reference_vector():
    # src/graph/cpu.rs:2579-2602: [1,2,3,4], eps 1e-5 -> x / sqrt(7.5 + 1e-5)
    out = P.rms_norm(np.array([[1.0, 2, 3, 4]]), np.ones(4), 1e-5)
    np.testing.assert_allclose(out[0], np.array([1.0, 2, 3, 4]) / math.sqrt(7.5 + 1e-5), rtol=1e-12)


def test_rmsnorm_library_and_gain_last():
    x, g = rng.normal(size=(5, 24)), rng.normal(size=24)
    ref = F.rms_norm(torch.tensor(x), (24,), torch.tensor(g), eps=1e-6).numpy()
    np.testing.assert_allclose(P.rms_norm(x, g, 1e-6), ref, rtol=1e-10)
    # eps sits inside the root: a zero row stays zero and finite
    assert np.all(P.rms_norm(np.zeros((1, 8)), np.ones(8), 1e-5) == 0)
    # per-head norm == the same routine on a [T*heads, hd] view
    xh = rng.normal(size=(3, 4, 16)); gh = rng.normal(size=16)
    np.testing.assert_allclose(P.rms_norm(xh, gh, 1e-5).reshape(12, 16), P.rms_norm(xh.reshape(12, 16), gh, 1e-5))


def test_inv_freq_pinned():
    # src/arch/gen.rs:843-844
    assert list(P.rope_inv_freq(4, 10000.0)) == [1.0, np.float32(0.01)]


def test_rope_identity_at_zero_and_complex_form():
    x = rng.normal(size=(6, 3, 16))
    inv = P.rope_inv_freq(16, 10000.0)
    # src/graph/cpu.rs:2688-2730: position 0 is the identity
    np.testing.assert_array_equal(P.rope_half_split(x[:1], [0], inv), x[:1])
    pos = [0, 1, 5, 17, 100, 1000]
    out = P.rope_half_split(x, pos, inv)
    # complex multiplication on pairs (j, j + half)
    z = x[..., :8] + 1j * x[..., 8:]
    ang = np.array([[float(np.float32(np.float32(p) * f)) for f in inv] for p in pos])
    zr = z * np.exp(1j * ang)[:, None, :]
    np.testing.assert_allclose(out[..., :8], zr.real, atol=1e-12)
    np.testing.assert_allclose(out[..., 8:], zr.imag, atol=1e-12)
    # norms are kept
    np.testing.assert_allclose(np.linalg.norm(out, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-12)


def test_rope_relative_positions_only():
    # q.k depends on the distance only: shifting all positions leaves scores unchanged
    # (small positions, where the float32 angle is exact enough)
    inv = P.rope_inv_freq(8, 100.0)
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    def score(pq, pk):
        return float((P.rope_half_split(q, [pq], inv) * P.rope_half_split(k, [pk], inv)).sum())
    assert abs(score(5, 2) - score(9, 6)) < 1e-5
    assert abs(score(5, 2) - score(2, 5)) > 1e-3     # the sign of the rotation matters


def test_attention_library_and_special_cases():
    T, nh, nkv, hd = 9, 6, 2, 16
    q, k, v = rng.normal(size=(T, nh, hd)), rng.normal(size=(T, nkv, hd)), rng.normal(size=(T, nkv, hd))
    scale = 1 / math.sqrt(hd)
    out = P.causal_attention(q, k, v, scale)
    tq = torch.tensor(q).transpose(0, 1)[None]
    tk = torch.tensor(k).transpose(0, 1).repeat_interleave(nh // nkv, dim=0)[None]
    tv = torch.tensor(v).transpose(0, 1).repeat_interleave(nh // nkv, dim=0)[None]
    ref = F.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=scale)[0].transpose(0, 1).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-12)
    # src/graph/cpu.rs:2748-2780: a single key returns its value
    np.testing.assert_allclose(out[0], np.repeat(v[0], nh // nkv, axis=0), atol=1e-12)
    # a window of 1 sees only itself; a window >= T is no window
    np.testing.assert_allclose(P.causal_attention(q, k, v, scale, window=1),
                               np.repeat(v, nh // nkv, axis=1), atol=1e-12)
    np.testing.assert_allclose(P.causal_attention(q, k, v, scale, window=T), out, atol=1e-12)
    # window 3 == library attention with a banded mask
    mask = torch.tensor([[0 <= t - i < 3 for i in range(T)] for t in range(T)])
    refw = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=scale)[0].transpose(0, 1).numpy()
    np.testing.assert_allclose(P.causal_attention(q, k, v, scale, window=3), refw, atol=1e-12)


def test_conv_reference_vector_and_library():
    # src/graph/cpu.rs:2783-2808: taps [0.5, 1.0] on [2,4,6] -> [2,5,8]
    out, st = P.causal_conv1d(np.array([[2.0], [4.0], [6.0]]), np.array([[0.5, 1.0]]))
    assert out[:, 0].tolist() == [2.0, 5.0, 8.0] and st[:, 0].tolist() == [6.0]
    T, C, K = 11, 5, 4
    x, w, b = rng.normal(size=(T, C)), rng.normal(size=(C, K)), rng.normal(size=C)
    out, st = P.causal_conv1d(x, w, b)
    ref = F.conv1d(torch.tensor(x.T)[None], torch.tensor(w)[:, None, :], torch.tensor(b), groups=C, padding=K - 1)[0, :, :T].T
    np.testing.assert_allclose(out, ref.numpy(), atol=1e-12)
    np.testing.assert_array_equal(st, x[-(K - 1):])


@pytest.mark.parametrize("cuts", [[1] * 11, [2, 2, 2, 2, 3], [5, 1, 2, 3], [11]])
def test_conv_chunk_invariance(cuts):
    # src/graph/cpu.rs:3007-3053: step by step equals whole, also for chunks shorter than K-1
    T, C, K = 11, 3, 4
    x, w = rng.normal(size=(T, C)), rng.normal(size=(C, K))
    whole, st_whole = P.causal_conv1d(x, w)
    outs, st, at = [], None, 0
    for c in cuts:
        o, st = P.causal_conv1d(x[at:at + c], w, state=st)
        outs.append(o); at += c
    np.testing.assert_allclose(np.concatenate(outs), whole, atol=1e-12)
    np.testing.assert_allclose(st, st_whole, atol=1e-12)


def test_swiglu_vectors():
    # src/graph/cpu.rs:2605-2622
    assert P.swiglu(np.array([0.0]), np.array([1.0]))[0] == 0.0
    np.testing.assert_allclose(P.swiglu(np.array([2.0]), np.array([3.0]))[0], 2 / (1 + math.exp(-2)) * 3, rtol=1e-12)
    g, u = rng.normal(size=20), rng.normal(size=20)
    np.testing.assert_allclose(P.swiglu(g, u), (F.silu(torch.tensor(g)) * torch.tensor(u)).numpy(), rtol=1e-12)


def test_ff_width_rule():
    base = dict(hidden_size=64, num_hidden_layers=1, num_attention_heads=4, conv_L_cache=3)
    def inter(**kw):
        return P.resolve_config({**base, **kw})["inter"]
    aa = dict(block_auto_adjust_ff_dim=True, block_ffn_dim_multiplier=1.0)
    assert inter(block_ff_dim=12288, **aa) == 8192
    assert inter(block_ff_dim=6656, **aa) == 4608
    assert inter(block_ff_dim=10752, **aa) == 7168
    assert inter(block_ff_dim=384, block_multiple_of=64, **aa) == 256
    assert inter(block_ff_dim=6656, block_auto_adjust_ff_dim=True) == 4437      # no multiplier: unrounded
    assert inter(block_ff_dim=384, block_auto_adjust_ff_dim=False) == 384
    assert inter(intermediate_size=100, block_ff_dim=384) == 100                # intermediate_size wins
    assert inter() == 256                                                       # 4 * hidden
    with pytest.raises(ValueError, match="must be >= 2"):
        P.resolve_config({**base, "conv_L_cache": 1})


def test_gate_order_matters():
    # thirds are [B | C | x]; swapping C with B changes the result (B and x commute)
    h = rng.normal(size=(6, 8)); w_in = rng.normal(size=(24, 8)); taps = rng.normal(size=(8, 1, 3)); w_out = rng.normal(size=(8, 8))
    out = P.short_conv_mixer(h, w_in, taps, w_out)
    bx = w_in.copy(); bx[0:8], bx[16:24] = w_in[16:24], w_in[0:8]
    np.testing.assert_allclose(P.short_conv_mixer(h, bx, taps, w_out), out, atol=1e-12)
    bc = w_in.copy(); bc[0:8], bc[8:16] = w_in[8:16], w_in[0:8]
    assert np.abs(P.short_conv_mixer(h, bc, taps, w_out) - out).max() > 1e-3


def test_tail_tied_equals_untied_copy():
    w, cfg = G.golden_weights(), G.golden_config()
    a = P.forward(w, cfg, G.PROMPT)
    w2 = dict(w); w2["lm_head.weight"] = w["model.embed_tokens.weight"].copy()
    np.testing.assert_array_equal(P.forward(w2, cfg, G.PROMPT), a)
    # causal: a row's logits do not depend on later tokens
    np.testing.assert_allclose(P.forward(w, cfg, G.PROMPT[:4]), a[:4], atol=1e-12)


def test_whole_model_golden_vector():
    """tests/golden/lm_graphlm_lfm2.json of the reference; tolerance of tests/golden/util.rs:257-260."""
    w, cfg, exp = G.golden_weights(), G.golden_config(), G.golden_expected()
    cases = {"prefill6": G.PROMPT, "prefill20": G.LONG_PROMPT}
    for i in range(3):
        cases[f"decode{i}"] = G.PROMPT + G.DECODE[:i + 1]
    for name, ids in cases.items():
        got = P.forward(w, cfg, ids)[-1]
        assert G.rel_l2(got, exp["f32"][name]) < 1e-3 and G.cosine(got, exp["f32"][name]) > 0.9999, name
    seq, out = list(G.PROMPT), []
    for _ in range(8):
        t = P.argmax_first(P.forward(w, cfg, seq)[-1]); out.append(t); seq.append(t)
    assert out == exp["ids"]["greedy8"]


def test_argmax_first_rules():
    # src/runtime/lm.rs:1244-1269: ties -> first; NaN never wins; all -inf -> 0
    assert P.argmax_first([1.0, 3.0, 3.0, 2.0]) == 1
    assert P.argmax_first([float("nan"), 1.0, float("nan"), 1.0]) == 1
    assert P.argmax_first([-math.inf] * 4) == 0
    assert P.argmax_first([float("nan")] * 3) == 0


def test_nucleus_against_full_sort():
    for seed in range(50):
        r = np.random.default_rng(seed)
        logits = r.normal(size=300).astype(np.float32) * 3
        ids, probs = P.nucleus(logits, 0.8, 50, 0.9)
        full = np.exp((logits.astype(np.float64) - logits.max()) / 0.8)
        order = np.argsort(-logits, kind="stable")[:50]
        p = full[order] / full[order].sum()
        cut = int(np.searchsorted(np.cumsum(p), 0.9 - 1e-7)) + 1
        assert abs(len(ids) - cut) <= 1 and list(order[:len(ids)]) == list(ids)
        np.testing.assert_allclose(probs, p[:len(ids)], rtol=1e-4)
    # temperature -> 0 puts all mass on the argmax
    ids, probs = P.nucleus(np.array([0.1, 0.5, 0.3], dtype=np.float32), 1e-3, 50, 0.9)
    assert ids == [1]
    assert P.draw([4, 9, 2], np.array([0.5, 0.3, 0.2], dtype=np.float32), 0.0) == 4
    assert P.draw([4, 9, 2], np.array([0.5, 0.3, 0.2], dtype=np.float32), 0.6) == 9
    assert P.draw([4, 9, 2], np.array([0.5, 0.3, 0.2], dtype=np.float32), 0.999) == 2


def test_repetition_penalty_rules():
    """Worked by hand from the reference's two loops (src/runtime/lm.rs:1089-1105, :1176-1189): the
    greedy rule divides c times and then subtracts 1.5 c; the sampling rule subtracts 1.5 after every
    division, so 4.0 seen twice at penalty 2 becomes 4/2/2 - 3 = -2 when greedy and
    (4/2 - 1.5)/2 - 1.5 = -1.25 when sampled; values that are not positive are multiplied."""
    logits = [4.0, -1.0, 0.5, 3.0, 0.0]
    recent = [0, 1, 0, 4, 99]                                  # 99: outside the vocabulary, ignored
    g = P.repetition_penalty(logits, recent, 2.0, greedy=True)
    s = P.repetition_penalty(logits, recent, 2.0, greedy=False)
    assert g.tolist() == [-2.0, -3.5, 0.5, 3.0, -1.5]
    assert s.tolist() == [-1.25, -3.5, 0.5, 3.0, -1.5]
    assert P.repetition_penalty(logits, recent, 1.0, greedy=True).tolist() == logits
    assert P.repetition_penalty(logits, [], 2.0, greedy=False).tolist() == logits
    # the best token, seen before, loses to the runner-up; unseen, it stays the best whatever the penalty
    assert P.argmax_first(g) == 3 and P.argmax_first(P.repetition_penalty(logits, [1, 2], 5.0, True)) == 0

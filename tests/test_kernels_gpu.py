"""Each kernel alone against a plain float32 PyTorch reference of the same operation, at sizes
other than the engine's tiny models use (sizes that are no power of two, several head sizes)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = [torch.float32, torch.bfloat16]


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def close(got, want, dtype, what="", f32=1e-5, bf16=1.2e-2):
    got, want = got.float().cpu(), want.float().cpu()
    tol = f32 if dtype == torch.float32 else bf16
    scale = want.abs().max().item() + 1e-30
    err = (got - want).abs().max().item()
    assert err <= tol * scale, f"{what}: error {err:.3e} > {tol} x {scale:.3e}"


@pytest.mark.parametrize("table_dtype", DT)
def test_embed(table_dtype):
    from gibbs_amd import ops
    table = rnd(331, 72, dtype=table_dtype)
    ids = i32([0, 330, 5, 5, 17])
    out = ops.embed(table, ids, 5)
    assert out.dtype == torch.float32
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("hidden", [48, 70, 200, 2048, 5000, 20000])   # 70 and 20000: the element-wise kernel
def test_add_rmsnorm(dtype, hidden):
    from gibbs_amd import ops
    x = rnd(7, hidden, scale=3.0)
    delta = rnd(7, hidden, dtype=dtype, seed=1)
    gain = rnd(hidden, seed=2) + 1.0
    x0 = x.clone()
    out = ops.add_rmsnorm(x, delta, gain, 1e-6, dtype)
    v = x0 + delta.float()
    assert torch.equal(x, v), "the residual stream must hold x + delta exactly"
    want = F.rms_norm(v.double(), (hidden,), gain.double(), eps=1e-6)
    close(out, want, dtype, "add_rmsnorm")
    # without delta; and on chosen rows only (x untouched)
    out2 = ops.add_rmsnorm(x, None, gain, 1e-6, dtype)
    close(out2, want, dtype, "rmsnorm")
    rows = i32([6, 0, 3])
    x1 = x.clone()
    out3 = ops.add_rmsnorm(x, delta, gain, 1e-6, dtype, rows)
    assert torch.equal(x, x1)
    want3 = F.rms_norm((x1 + delta.float())[rows.long()].double(), (hidden,), gain.double(), eps=1e-6)
    close(out3, want3, dtype, "rmsnorm rows")


@pytest.mark.parametrize("shape", [(1, 64, 32), (5, 331, 112), (130, 200, 72), (257, 129, 1000)])
def test_gemm_f32(shape):
    from gibbs_amd import ops
    n, o, i = shape
    a, w = rnd(n, i), rnd(o, i, seed=1)
    close(ops.gemm_f32(a, w), a.double() @ w.double().t(), torch.float32, f"gemm_f32 {shape}")
    # a row's result does not depend on the other rows of the call
    assert torch.equal(ops.gemm_f32(a[:1].contiguous(), w), ops.gemm_f32(a, w)[:1])


@pytest.mark.parametrize("out_dtype", DT)
@pytest.mark.parametrize("shape", [(1, 64, 32), (5, 331, 112), (130, 200, 72), (257, 129, 1000), (300, 512, 2048),
                                   (2048, 6144, 192), (1024, 12288, 64), (768, 16384, 320)])   # the 256 x 256 kernel: both tile orders
def test_gemm_bf16(shape, out_dtype):
    from gibbs_amd import ops
    n, o, i = shape
    a, w = rnd(n, i, dtype=torch.bfloat16), rnd(o, i, dtype=torch.bfloat16, seed=1)
    want = a.double() @ w.double().t()
    got = ops.gemm_bf16(a, w, out_dtype)
    assert got.dtype == out_dtype
    # float32 output: only the accumulation order differs from the exact product
    close(got, want, out_dtype, f"gemm_bf16 {shape}", f32=2e-5, bf16=4e-3)
    # a view with a row stride (the q part of a fused projection)
    big = rnd(n, i + 64, dtype=torch.bfloat16, seed=3)
    close(ops.gemm_bf16(big[:, :i], w, out_dtype), big[:, :i].double() @ w.double().t(), out_dtype, "strided", f32=2e-5, bf16=4e-3)


@pytest.mark.parametrize("shape", [(65, 64, 32), (130, 200, 72), (257, 129, 1000), (512, 6144, 2048), (2048, 2048, 512)])
def test_gemm_library(shape):
    """The library's product called directly (descriptors and algorithm kept per shape), also on a
    view with a row stride and into a strided output, and twice (the second call takes the kept plan)."""
    from gibbs_amd import ops
    n, o, i = shape
    a, w = rnd(n, i, dtype=torch.bfloat16), rnd(o, i, dtype=torch.bfloat16, seed=1)
    want = a.double() @ w.double().t()
    for _ in range(2):
        close(ops.gemm_library(a, w), want, torch.bfloat16, f"gemm_library {shape}", bf16=4e-3)
    big = rnd(n, i + 64, dtype=torch.bfloat16, seed=3)
    close(ops.gemm_library(big[:, :i], w), big[:, :i].double() @ w.double().t(), torch.bfloat16, "strided input", bf16=4e-3)
    wide = torch.zeros(n, o + 16, dtype=torch.bfloat16, device=DEV)
    ops.gemm_library(a, w, out=wide[:, :o])
    close(wide[:, :o], want, torch.bfloat16, "strided output", bf16=4e-3)
    assert float(wide[:, o:].abs().max()) == 0.0


@pytest.mark.parametrize("out_dtype", DT)
@pytest.mark.parametrize("n,o,i,splits", [(1, 64, 128, 1), (8, 331, 1000, 1), (16, 2048, 2048, 2), (17, 200, 8192, 8),
                                          (33, 48, 72, 1), (64, 515, 1024, 1), (5, 2048, 8192, 4), (64, 96, 4096, 3),
                                          (64, 2048, 2048, 8), (40, 8200, 512, 1), (50, 1000, 4096, 16)])   # 4 tiles a workgroup
def test_gemm_skinny(n, o, i, splits, out_dtype):
    from gibbs_amd import ops
    x, w = rnd(n, i, dtype=torch.bfloat16), rnd(o, i, dtype=torch.bfloat16, seed=1)
    want = x.double() @ w.double().t()
    if splits > 1 and out_dtype == torch.float32:          # partial sums are float32
        parts = ops.gemm_skinny(x, w, torch.float32, splits)
        assert parts.shape == (splits, n, o)
        close(parts.sum(0), want, torch.float32, "skinny partial sums", f32=2e-5)
    got = ops.gemm_skinny(x, w, out_dtype)
    assert got.dtype == out_dtype and got.shape == (n, o)
    close(got, want, out_dtype, f"gemm_skinny {(n, o, i)}", f32=2e-5, bf16=4e-3)
    # a strided view of x (rows of a wider buffer)
    big = rnd(n, i + 64, dtype=torch.bfloat16, seed=3)
    close(ops.gemm_skinny(big[:, :i], w, out_dtype), big[:, :i].double() @ w.double().t(), out_dtype, "strided",
          f32=2e-5, bf16=4e-3)


def test_packed_weight_layout():
    """Many rows: [group][16-row tile][32-k tile][lane = g * 16 + r][8]; few rows (workgroups of 8 features):
    [group][8-row tile][pair of k tiles][g][half][r8][8]; zeros beyond the matrix."""
    from gibbs_amd import ops
    rows = 4104                                             # 257 tiles of 16
    assert not ops.pair_layout(rows) and not ops.pair_layout(4081) and ops.pair_layout(4080) and ops.pair_layout(40)
    w = rnd(2 * rows, 72, dtype=torch.bfloat16)
    p = ops.PackedWeight(w, groups=2)
    assert p.shape == (2 * rows, 72) and p.stride(0) == 0 and tuple(p.data.shape) == (2, 257, 3, 4, 16, 8) and not p.pairs
    for q, ot, kt, g, r in [(0, 0, 0, 0, 0), (1, 2, 1, 3, 7), (0, 256, 2, 0, 15), (1, 256, 2, 1, 3), (1, 256, 0, 2, 8)]:
        row, k = ot * 16 + r, kt * 32 + g * 8
        want = torch.zeros(8, dtype=torch.bfloat16, device=DEV)
        if row < rows and k < 72:
            want[:min(8, 72 - k)] = w[q * rows + row, k:k + 8]
        assert torch.equal(p.data[q, ot, kt, g, r], want), (q, ot, kt, g, r)
    w = rnd(2 * 40, 72, dtype=torch.bfloat16)
    p = ops.PackedWeight(w, groups=2)
    assert p.shape == (80, 72) and p.stride(0) == 0 and tuple(p.data.shape) == (2, 6, 2, 4, 2, 8, 8) and p.pairs
    for q, o8, pair, g, half, r8 in [(0, 0, 0, 0, 0, 0), (1, 4, 1, 0, 0, 7), (0, 2, 1, 1, 1, 5), (1, 5, 0, 3, 1, 3), (0, 4, 0, 2, 1, 7)]:
        row, k = o8 * 8 + r8, pair * 64 + half * 32 + g * 8
        want = torch.zeros(8, dtype=torch.bfloat16, device=DEV)
        if row < 40 and k < 72:
            want[:min(8, 72 - k)] = w[q * 40 + row, k:k + 8]
        assert torch.equal(p.data[q, o8, pair, g, half, r8], want), (q, o8, pair, g, half, r8)
    x = rnd(5, 72, dtype=torch.bfloat16, seed=2)
    for splits in (1, 2):
        w1 = rnd(50, 256, dtype=torch.bfloat16, seed=3)
        x1 = rnd(5, 256, dtype=torch.bfloat16, seed=4)
        assert torch.equal(ops.gemm_skinny(x1, ops.PackedWeight(w1), torch.float32, splits), ops.gemm_skinny(x1, w1, torch.float32, splits))
        w2 = rnd(4200, 256, dtype=torch.bfloat16, seed=5)                    # 16-row tiles
        assert torch.equal(ops.gemm_skinny(x1, ops.PackedWeight(w2), torch.float32, splits), ops.gemm_skinny(x1, w2, torch.float32, splits))


def test_skinny_splits_cover_k():
    from gibbs_amd import ops
    for o, i in [(2048, 2048), (2048, 8192), (6144, 2048), (65536, 2048), (96, 96), (200, 1000), (64, 12800)]:
        s = ops.skinny_splits(o, i)
        per = -(-(-(-i // s)) // 128) * 128
        assert s >= 1 and -(-i // per) == s, (o, i, s)
        x, w = rnd(3, i, dtype=torch.bfloat16), rnd(min(o, 64), i, dtype=torch.bfloat16, seed=1)
        parts = ops.gemm_skinny(x, w, torch.float32, s)
        got = parts.sum(0) if s > 1 else parts
        close(got, x.double() @ w.double().t(), torch.float32, f"splits {s}", f32=2e-5)


@pytest.mark.parametrize("dtype", DT)
def test_add_partials_rmsnorm(dtype):
    from gibbs_amd import ops
    hidden, n, s = 200, 5, 3
    x = rnd(n, hidden, scale=2.0)
    parts = rnd(s, n, hidden, seed=4)
    gain = rnd(hidden, seed=2) + 1.0
    x0 = x.clone()
    out = ops.add_rmsnorm(x, parts, gain, 1e-6, dtype)
    v = x0 + (parts[0] + parts[1]) + parts[2]
    close(x, v, torch.float32, "x + partials", f32=1e-6)
    close(out, F.rms_norm(v.double(), (hidden,), gain.double(), eps=1e-6), dtype, "partials rmsnorm")
    rows = i32([4, 1])
    x1 = x.clone()
    out2 = ops.add_rmsnorm(x, parts, gain, 1e-6, dtype, rows)
    assert torch.equal(x, x1)
    close(out2, F.rms_norm((x1 + parts.sum(0))[rows.long()].double(), (hidden,), gain.double(), eps=1e-6), dtype, "rows")


def test_gemm_bf16_refuses_unaligned():
    from gibbs_amd import ops
    from gibbs_amd.ops.lib import KernelError
    with pytest.raises(KernelError, match="multiples of 8"):
        ops.gemm_bf16(rnd(3, 20, dtype=torch.bfloat16), rnd(4, 20, dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", DT)
def test_glu(dtype):
    from gibbs_amd import ops
    gu = rnd(9, 2 * 200, dtype=dtype, scale=2.0)
    want = F.silu(gu.double()[:, :200]) * gu.double()[:, 200:]
    close(ops.glu(gu), want, dtype, "glu")
    one = torch.tensor([[0.0, 2.0, 1.0, 3.0]], device=DEV)              # silu(0)*1 = 0, silu(2)*3
    out = ops.glu(one)
    assert out[0, 0].item() == 0.0 and abs(out[0, 1].item() - 2 / (1 + math.exp(-2)) * 3) < 1e-6


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("K,C,bias", [(3, 40, False), (4, 300, True), (2, 72, True), (7, 16, False)])
def test_shortconv_ragged_with_state(dtype, K, C, bias):
    """Three requests in one call: a fresh one, one with history shorter than K-1 before this chunk,
    one decoding a single token; against conv1d over each whole sequence."""
    from gibbs_amd import ops
    taps = rnd(C, K, seed=4)
    b = rnd(C, seed=5) if bias else None
    lens_before, lens_now = [0, 1, 9], [6, 2, 1]
    slots = [2, 0, 3]
    seqs = [rnd(lb + ln, 3 * C, dtype=dtype, seed=10 + i) for i, (lb, ln) in enumerate(zip(lens_before, lens_now))]
    state = torch.full((4, K - 1, C), 7.0, device=DEV)                   # stale content of a reused slot
    def reference(seq):
        s = seq.double()
        bx = s[:, :C] * s[:, 2 * C:]
        cv = F.conv1d(bx.t()[None], taps.double()[:, None, :], None if b is None else b.double(), groups=C,
                      padding=K - 1)[0, :, :seq.shape[0]].t()
        return s[:, C:2 * C] * cv, bx
    # first call: the histories (requests 1 and 2 only)
    cu = i32([0, lens_before[1], lens_before[1] + lens_before[2]])
    hist = torch.cat([seqs[1][:lens_before[1]], seqs[2][:lens_before[2]]])
    ops.shortconv(hist, taps, b, state, cu, i32([0, 0]), i32(slots[1:]), hist.shape[0], 2)
    # second call: all three together
    now = torch.cat([s[lb:] for s, lb in zip(seqs, lens_before)])
    cu = i32(np.concatenate([[0], np.cumsum(lens_now)]))
    y = ops.shortconv(now, taps, b, state, cu, i32(lens_before), i32(slots), now.shape[0], 3)
    at = 0
    for seq, lb, ln, slot in zip(seqs, lens_before, lens_now, slots):
        want, bx = reference(seq)
        close(y[at:at + ln], want[lb:], dtype, f"shortconv rows K={K}")
        at += ln
        full = torch.cat([torch.zeros(K - 1, C, device=DEV, dtype=torch.float64), bx])
        close(state[slot], full[-(K - 1):], torch.float32, "state", f32=1e-6)
    assert torch.all(state[1] == 7.0), "a slot of no request was written"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [24, 520])
@pytest.mark.parametrize("lens_now", [[1, 1, 1, 1, 1], [1, 1, 1, 40, 2], [1, 1, 70, 1, 1]])
def test_shortconv_decoded_rows_at_the_head(dtype, C, lens_now):
    """Requests that bring one row each at the head of the batch (decoded tokens) are found by their tile's number,
    the others by a walk over the requests behind them: the same result whatever the caller says about the head
    (nothing, its true length, less), and against conv1d over each whole sequence."""
    from gibbs_amd import ops
    K = 3
    taps, b = rnd(C, K, seed=4), rnd(C, seed=5)
    lens_before = [9, 1, 3, 0, 5]
    slots = [4, 0, 3, 1, 5]
    seqs = [rnd(lb + ln, 3 * C, dtype=dtype, seed=20 + i) for i, (lb, ln) in enumerate(zip(lens_before, lens_now))]
    lead = next((i for i, n in enumerate(lens_now) if n != 1), len(lens_now))
    results = []
    for say in (None, lead, max(lead - 1, 0), 0):
        state = torch.full((6, K - 1, C), 7.0, device=DEV)
        with_history = [i for i, lb in enumerate(lens_before) if lb]
        hist = torch.cat([seqs[i][:lens_before[i]] for i in with_history])
        cu = i32(np.concatenate([[0], np.cumsum([lens_before[i] for i in with_history])]))
        ops.shortconv(hist, taps, b, state, cu, i32([0] * len(with_history)), i32([slots[i] for i in with_history]),
                      hist.shape[0], len(with_history))
        now = torch.cat([s[lb:] for s, lb in zip(seqs, lens_before)])
        cu = i32(np.concatenate([[0], np.cumsum(lens_now)]))
        y = ops.shortconv(now, taps, b, state, cu, i32(lens_before), i32(slots), now.shape[0], len(lens_now), lead_single=say)
        results.append((y, state))
    for y, state in results[1:]:
        assert torch.equal(y, results[0][0]) and torch.equal(state, results[0][1])
    y, state = results[0]
    at = 0
    for seq, lb, ln, slot in zip(seqs, lens_before, lens_now, slots):
        s = seq.double()
        bx = s[:, :C] * s[:, 2 * C:]
        cv = F.conv1d(bx.t()[None], taps.double()[:, None, :], b.double(), groups=C, padding=K - 1)[0, :, :seq.shape[0]].t()
        close(y[at:at + ln], (s[:, C:2 * C] * cv)[lb:], dtype, "shortconv rows")
        at += ln
        full = torch.cat([torch.zeros(K - 1, C, device=DEV, dtype=torch.float64), bx])
        close(state[slot], full[-(K - 1):], torch.float32, "state", f32=1e-6)
    assert torch.all(state[2] == 7.0), "a slot of no request was written"
    with pytest.raises(ops.KernelError, match="leading single rows"):
        ops.shortconv(now, taps, b, state, cu, i32(lens_before), i32(slots), now.shape[0], len(lens_now), lead_single=6)


def paged_setup(dtype, nkv, hd, page_size, seq_lens, num_pages, seed=0):
    """Random keys and values of several requests scattered over shuffled pages (the rest of the
    pool holds large garbage)."""
    rng = np.random.default_rng(seed)
    kp = torch.full((num_pages, nkv, page_size, hd), 50.0, dtype=dtype, device=DEV)
    vp = torch.full((num_pages, nkv, page_size, hd), -50.0, dtype=dtype, device=DEV)
    free = rng.permutation(num_pages).tolist()
    width = max(-(-l // page_size) for l in seq_lens)
    table = np.full((len(seq_lens), width), -1, dtype=np.int32)
    ks, vs = [], []
    for r, l in enumerate(seq_lens):
        k, v = rnd(l, nkv, hd, dtype=dtype, seed=seed + 2 * r), rnd(l, nkv, hd, dtype=dtype, seed=seed + 2 * r + 1)
        ks.append(k); vs.append(v)
        for j in range(-(-l // page_size)):
            p = free.pop()
            table[r, j] = p
            n = min(page_size, l - j * page_size)
            kp[p, :, :n] = k[j * page_size:j * page_size + n].transpose(0, 1)
            vp[p, :, :n] = v[j * page_size:j * page_size + n].transpose(0, 1)
    return kp, vp, i32(table), ks, vs


def attention_reference(q, k, v, positions, scale, window):
    """q: [n, nh, hd] rows at `positions` of one request with keys k, v: [L, nkv, hd]."""
    nh, nkv = q.shape[1], k.shape[1]
    kk, vv = k.double().repeat_interleave(nh // nkv, 1), v.double().repeat_interleave(nh // nkv, 1)
    out = torch.zeros(q.shape, dtype=torch.float64, device=q.device)
    for i, p in enumerate(positions):
        lo = 0 if not window else max(0, p - window + 1)
        s = torch.einsum("hd,lhd->hl", q[i].double(), kk[lo:p + 1]) * scale
        out[i] = torch.einsum("hl,lhd->hd", s.softmax(-1), vv[lo:p + 1])
    return out


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,hd,page,window", [(4, 2, 16, 16, None), (6, 1, 48, 8, None), (5, 5, 80, 32, 37),
                                                   (8, 2, 128, 16, None), (2, 2, 256, 64, 100)])
def test_attention_plain_paged(dtype, nh, nkv, hd, page, window):
    from gibbs_amd import ops
    seq_lens = [150, 3, 77]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 40)
    # request 0: a portion of 20 rows ending at its last key; request 1: all 3 rows; request 2: one decoded row
    rows = [(0, list(range(130, 150))), (1, [0, 1, 2]), (2, [76])]
    pos = i32([p for _, ps in rows for p in ps])
    row_req = i32([r for r, ps in rows for _ in ps])
    n = pos.numel()
    q = rnd(n, nh * hd, dtype=dtype, seed=9)
    scale = 1 / math.sqrt(hd)
    out = ops.attention_plain(q, n, nh, nkv, hd, kp, vp, table, 3, pos, row_req, scale, window)
    at = 0
    for r, ps in rows:
        want = attention_reference(q[at:at + len(ps)].view(-1, nh, hd), ks[r], vs[r], ps, scale, window)
        close(out[at:at + len(ps)].view(-1, nh, hd), want, dtype, f"attention request {r}", f32=2e-5, bf16=1e-2)
        at += len(ps)


@pytest.mark.parametrize("kind", ["valu", "mfma", "valu-merge-pass", "mfma-merge-pass"])
@pytest.mark.parametrize("n_splits,waves", [(1, 4), (1, 8), (3, 8), (16, 4), (None, None)])
@pytest.mark.parametrize("nh,nkv,hd,page,window", [(4, 2, 16, 16, None), (6, 1, 48, 8, None), (5, 5, 80, 32, 37),
                                                   (32, 8, 64, 16, None), (16, 2, 128, 16, None), (2, 2, 256, 64, 100),
                                                   (24, 2, 32, 16, None), (3, 1, 24, 16, None)])
def test_attention_decode_split_keys(nh, nkv, hd, page, window, n_splits, waves, kind):
    """The key-splitting kernel against the float64 reference and against the plain kernel, for
    rows of different lengths (one key, a page edge, hundreds of keys) in one call."""
    from gibbs_amd import ops
    dtype = torch.bfloat16
    seq_lens = [700, 1, 33, 16]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 120, seed=7)
    positions = [l - 1 for l in seq_lens]
    pos, row_req = i32(positions), i32([0, 1, 2, 3])
    q = rnd(4, nh * hd, dtype=dtype, seed=9)
    scale = 1 / math.sqrt(hd)
    if kind.startswith("mfma") and (hd % 16 or hd > 128):
        with pytest.raises(ops.KernelError, match="matrix-core"):
            ops.attention_decode(q, 4, nh, nkv, hd, kp, vp, table, 4, pos, row_req, scale, window, max_seq=700,
                                 n_splits=n_splits, waves=waves, kind=kind)
        return
    out = ops.attention_decode(q, 4, nh, nkv, hd, kp, vp, table, 4, pos, row_req, scale, window, max_seq=700,
                               n_splits=n_splits, waves=waves, kind=kind)
    plain = ops.attention_plain(q, 4, nh, nkv, hd, kp, vp, table, 4, pos, row_req, scale, window)
    for r in range(4):
        want = attention_reference(q[r:r + 1].view(1, nh, hd), ks[r], vs[r], [positions[r]], scale, window)
        close(out[r].view(1, nh, hd), want, dtype, f"decode attention row {r}", bf16=1e-2)
    close(out, plain, dtype, "decode vs plain kernel", bf16=1e-2)


@pytest.mark.parametrize("kind", ["valu", "mfma"])
@pytest.mark.parametrize("n_splits", [1, 4])
@pytest.mark.parametrize("bound", [0, 64, 700])
def test_attention_decode_rows_as_requests_and_rows_beyond_the_bound(bound, n_splits, kind):
    """Without a row-to-request map row n is request n; and the caller's bound on the keys only steers the
    kernel (it asks for a row's page ids before it knows the row's position when the whole table fits its
    staging area): rows beyond the bound take the ids of their slice afterwards and are as right."""
    from gibbs_amd import ops
    dtype, nh, nkv, hd, page = torch.bfloat16, 8, 2, 64, 8
    seq_lens = [700, 1, 33, 16, 300]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 180, seed=11)
    positions = [l - 1 for l in seq_lens]
    pos = i32(positions)
    q = rnd(5, nh * hd, dtype=dtype, seed=12)
    scale = 1 / math.sqrt(hd)
    out = ops.attention_decode(q, 5, nh, nkv, hd, kp, vp, table, 5, pos, None, scale, None, max_seq=bound,
                               n_splits=n_splits, waves=4, kind=kind)
    mapped = ops.attention_decode(q, 5, nh, nkv, hd, kp, vp, table, 5, pos, i32([0, 1, 2, 3, 4]), scale, None, max_seq=bound,
                                  n_splits=n_splits, waves=4, kind=kind)
    assert torch.equal(out, mapped)
    for r in range(5):
        want = attention_reference(q[r:r + 1].view(1, nh, hd), ks[r], vs[r], [positions[r]], scale, None)
        close(out[r].view(1, nh, hd), want, dtype, f"decode attention row {r}", bf16=1e-2)


@pytest.mark.parametrize("n_splits", [1, 3, 7])
@pytest.mark.parametrize("nh,nkv,hd,page,window", [(4, 2, 16, 16, None), (6, 1, 48, 8, None), (5, 5, 80, 32, 37),
                                                   (32, 8, 64, 16, None), (4, 2, 128, 16, None), (2, 2, 96, 64, 100),
                                                   (3, 1, 32, 16, 5), (8, 2, 48, 16, None), (12, 2, 32, 8, 90)])
def test_attention_prefill_matrix_cores(nh, nkv, hd, page, window, n_splits):
    """Prompt portions on the matrix cores: a long portion after a cached context that ends off a
    tile edge, a whole short prompt, a 2-token portion, a single decoded row and a 65-row portion
    that starts at position 0, all in one call; with the key tiles whole or cut into slices (more
    slices than the short requests have tiles: slices without keys)."""
    from gibbs_amd import ops
    dtype = torch.bfloat16
    seq_lens = [333, 9, 130, 77, 65]
    q_lens = [150, 9, 2, 1, 65]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 120, seed=11)
    ctx = [s - q for s, q in zip(seq_lens, q_lens)]
    cu = np.concatenate([[0], np.cumsum(q_lens)])
    n = int(cu[-1])
    q = rnd(n, nh * hd, dtype=dtype, seed=9)
    scale = 1 / math.sqrt(hd)
    out = ops.attention_prefill(q, n, nh, nkv, hd, kp, vp, table, 5, i32(cu), i32(ctx), scale, window, n_splits=n_splits)
    pos = i32([c + t for c, ql in zip(ctx, q_lens) for t in range(ql)])
    row_req = i32([r for r, ql in enumerate(q_lens) for _ in range(ql)])
    plain = ops.attention_plain(q, n, nh, nkv, hd, kp, vp, table, 5, pos, row_req, scale, window)
    for r in range(5):
        rows = slice(int(cu[r]), int(cu[r + 1]))
        want = attention_reference(q[rows].view(-1, nh, hd), ks[r], vs[r], list(range(ctx[r], seq_lens[r])), scale, window)
        close(out[rows].view(-1, nh, hd), want, dtype, f"prefill attention request {r}", bf16=1e-2)
    close(out, plain, dtype, "prefill vs plain kernel", bf16=1e-2)
    # only the requests from the third on: the rows before them stay as they were
    first_req, first_row = 2, int(cu[2])
    part = torch.full_like(out, 7.0)
    ops.attention_prefill(q, n, nh, nkv, hd, kp, vp, table, 5, i32(cu), i32(ctx), scale, window, out=part,
                          n_splits=n_splits, first_req=first_req, first_row=first_row)
    assert torch.equal(part[first_row:], out[first_row:]) and (part[:first_row] == 7.0).all()
    # several query heads of a kv head's group in one workgroup (one K and V tile for all of them): every row of
    # every head goes through the same operations in the same order, so the result is the same to the bit
    for heads in (2, 4):
        if (nh // nkv) % heads == 0 and hd <= 64:
            many = ops.attention_prefill(q, n, nh, nkv, hd, kp, vp, table, 5, i32(cu), i32(ctx), scale, window,
                                         n_splits=n_splits, heads_per_wg=heads)
            assert torch.equal(many, out), f"{heads} heads a workgroup"
    with pytest.raises(ops.KernelError, match="heads a workgroup"):
        ops.attention_prefill(q, n, nh, nkv, hd, kp, vp, table, 5, i32(cu), i32(ctx), scale, window, heads_per_wg=3)


def test_prefill_splits_choice():
    from gibbs_amd.ops import prefill_splits
    assert prefill_splits(32, 32, 2048) == 1                 # a whole 2,048-token prompt fills the chip
    assert prefill_splits(8, 32, 8192) == 8                  # a portion of 512 late in a long prompt does not
    assert prefill_splits(1, 4, 300) == 1 and prefill_splits(1, 4, 100000) == 16
    assert prefill_splits(8, 32, 8192, window=128) == 1      # a window bounds the keys


@pytest.mark.parametrize("dtype", DT)
def test_attention_far_key_stands_out(dtype):
    """One key far back among hundreds gets a large score: its value must dominate the output."""
    from gibbs_amd import ops
    nh = nkv = 1; hd = 32; L = 700
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, 16, [L], 64, seed=3)
    q = rnd(1, hd, dtype=dtype, seed=1)
    far = 5
    page, off = table[0, far // 16].item(), far % 16
    kp[page, 0, off] = (q[0].float() * 8).to(dtype)
    ks[0][far, 0] = kp[page, 0, off]
    out = ops.attention_plain(q, 1, nh, nkv, hd, kp, vp, table, 1, i32([L - 1]), i32([0]), 1 / math.sqrt(hd))
    want = attention_reference(q.view(1, 1, hd), ks[0], vs[0], [L - 1], 1 / math.sqrt(hd), None)
    close(out.view(1, 1, hd), want, dtype, "far key", f32=2e-5, bf16=1e-2)
    assert (out.float() - vs[0][far, 0].float()).abs().max() < 0.05 * vs[0][far, 0].float().abs().max() + 0.05
    if dtype == torch.bfloat16:
        # the same through the fast kernels: split keys (the far key lies in the first slice), and
        # the matrix-core kernel with the row as the last of a 2-row portion
        split = ops.attention_decode(q, 1, nh, nkv, hd, kp, vp, table, 1, i32([L - 1]), i32([0]), 1 / math.sqrt(hd), n_splits=8)
        close(split.view(1, 1, hd), want, dtype, "far key, split keys", bf16=1e-2)
        q2 = torch.cat([rnd(1, hd, dtype=dtype, seed=2), q])
        pre = ops.attention_prefill(q2, 2, nh, nkv, hd, kp, vp, table, 1, i32([0, 2]), i32([L - 2]), 1 / math.sqrt(hd))
        close(pre[1].view(1, 1, hd), want, dtype, "far key, matrix cores", bf16=1e-2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("variant", ["half_split", "interleaved"])
@pytest.mark.parametrize("table_len", [0, 6, 64])       # no table; positions 9 and 17 beyond it; all from it
@pytest.mark.parametrize("nh,nkv,hd,rot", [(4, 2, 16, 16), (3, 1, 48, 32), (2, 2, 128, 128), (2, 1, 24, 12)])
def test_qk_rope_kv(dtype, variant, nh, nkv, hd, rot, table_len):
    from gibbs_amd import ops
    from gibbs_amd.parts.rope import rope_inv_freq
    n, page, num_pages = 6, 8, 10
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype)
    qkv0 = qkv.clone()
    qg, kg = rnd(hd, seed=1) + 1, rnd(hd, seed=2) + 1
    inv = torch.from_numpy(rope_inv_freq(rot, 10000.0, "f32")).to(DEV)
    positions = [3, 4, 5, 0, 17, 9]
    row_req = [0, 0, 0, 1, 1, 2]
    table = i32([[4, 7, -1], [2, 9, 0], [5, 1, -1]])
    kp = torch.zeros(num_pages, nkv, page, hd, dtype=dtype, device=DEV)
    vp = torch.zeros_like(kp)
    cos_sin = ops.rope_table(inv, table_len) if table_len else None
    ops.qk_rope_kv(qkv, n, nh, nkv, hd, q_gain=qg, k_gain=kg, eps=1e-6, inv_freq=inv, rotary_dim=rot, variant=variant,
                   pos=i32(positions), row_req=i32(row_req), kpages=kp, vpages=vp, table=table, n_req=3, cos_sin=cos_sin)
    if table_len:   # a table changes nothing, to the bit: it holds what the kernel computes
        qkv1, kp1, vp1 = qkv0.clone(), torch.zeros_like(kp), torch.zeros_like(vp)
        ops.qk_rope_kv(qkv1, n, nh, nkv, hd, q_gain=qg, k_gain=kg, eps=1e-6, inv_freq=inv, rotary_dim=rot,
                       variant=variant, pos=i32(positions), row_req=i32(row_req), kpages=kp1, vpages=vp1, table=table,
                       n_req=3)
        assert torch.equal(qkv1, qkv) and torch.equal(kp1, kp) and torch.equal(vp1, vp)

    def ref(x, gain):                                     # x: [n, heads, hd] float64
        x = F.rms_norm(x, (hd,), gain.double(), eps=1e-6)
        ang = torch.tensor(positions, dtype=torch.float32, device=DEV)[:, None] * inv[None, :]
        c, s = ang.double().cos()[:, None, :], ang.double().sin()[:, None, :]
        out = x.clone()
        half = rot // 2
        i0 = torch.arange(half) if variant == "half_split" else torch.arange(half) * 2
        i1 = i0 + half if variant == "half_split" else i0 + 1
        out[..., i0] = x[..., i0] * c - x[..., i1] * s
        out[..., i1] = x[..., i0] * s + x[..., i1] * c
        return out
    q0 = qkv0[:, :nh * hd].double().view(n, nh, hd)
    k0 = qkv0[:, nh * hd:(nh + nkv) * hd].double().view(n, nkv, hd)
    v0 = qkv0[:, (nh + nkv) * hd:].view(n, nkv, hd)
    close(qkv[:, :nh * hd].view(n, nh, hd), ref(q0, qg), dtype, "q", bf16=8e-3)
    kr = ref(k0, kg)
    for i, (p, r) in enumerate(zip(positions, row_req)):
        pg = table[r, p // page].item()
        close(kp[pg, :, p % page], kr[i], dtype, "k page", bf16=8e-3)
        assert torch.equal(vp[pg, :, p % page], v0[i])
    assert kp.float().abs().sum(dim=(1, 3)).count_nonzero().item() == n, "exactly one page slot per row was written"


def plain_qk(x, gain, positions, inv, eps):
    """Per-head RMSNorm then the half-split rotation of x [n, heads, hd], by the plain implementation
    (float32 angle = float32(pos) * inv_freq, src/graph/cpu.rs:673)."""
    from tests.plain import lfm2_plain as P
    return torch.tensor(P.rope_half_split(P.rms_norm(x.double().cpu().numpy(), gain.double().cpu().numpy(), eps), positions, inv))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("table_len", [0, 4096])
def test_qk_rope_kv_at_far_positions(dtype, table_len):
    """theta 1e6, heads of 64, rows at positions 32,767 and 99,999 (and beside them, and near the start):
    there the float32 product float32(pos) * inv_freq has lost its low bits, and an angle computed any
    other way (in float64, from a recurrence, as pos * a rounded inverse) is off by up to 4e-3 rad.  Against
    the plain implementation's rotation, which takes the reference's float32 steps."""
    from gibbs_amd import ops
    from tests.plain import lfm2_plain as P
    nh, nkv, hd, page = 4, 2, 64, 16
    positions = [99999, 32767, 99998, 5, 65536, 32768]
    n = len(positions)
    inv_np = P.rope_inv_freq(hd, 1e6)
    inv = torch.from_numpy(inv_np).to(DEV)
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=3)
    qkv0 = qkv.clone()
    qg, kg = rnd(hd, seed=1) * 0.1 + 1, rnd(hd, seed=2) * 0.1 + 1
    width = 100000 // page
    table = np.full((n, width), -1, dtype=np.int32)
    for r, p in enumerate(positions):                       # one request per row, one real page each
        table[r, p // page] = n - 1 - r
    kp = torch.zeros(n, nkv, page, hd, dtype=dtype, device=DEV)
    vp = torch.zeros_like(kp)
    ops.qk_rope_kv(qkv, n, nh, nkv, hd, q_gain=qg, k_gain=kg, eps=1e-5, inv_freq=inv, rotary_dim=hd, variant="half_split",
                   pos=i32(positions), row_req=i32(list(range(n))), kpages=kp, vpages=vp, table=i32(table), n_req=n,
                   cos_sin=ops.rope_table(inv, table_len) if table_len else None)
    q0 = qkv0[:, :nh * hd].view(n, nh, hd)
    k0 = qkv0[:, nh * hd:(nh + nkv) * hd].view(n, nkv, hd)
    close(qkv[:, :nh * hd].view(n, nh, hd), plain_qk(q0, qg, positions, inv_np, 1e-5), dtype, "q at far positions", f32=2e-6, bf16=8e-3)
    kr = plain_qk(k0, kg, positions, inv_np, 1e-5)
    for r, p in enumerate(positions):
        close(kp[n - 1 - r, :, p % page], kr[r], dtype, f"k at position {p}", f32=2e-6, bf16=8e-3)
    # the same angles in float64 would fail this bound: the test can tell the difference
    ang32 = (np.float32(99999) * inv_np).astype(np.float64)
    ang64 = 99999.0 * inv_np.astype(np.float64)
    assert np.abs(np.cos(ang32) - np.cos(ang64)).max() > 1e-4


@pytest.mark.parametrize("kind", ["valu", "mfma"])
@pytest.mark.parametrize("window", [None, 48])
def test_attention_decode_fused_at_far_positions(kind, window):
    """Decoded tokens at positions 99,999 and 32,767 (theta 1e6, pages of 16: 6,250 page ids, so the
    matrix-core walk must cut the cache into slices whatever the batch) beside a short request: q/k norm and
    rotation against the plain implementation's, attention against float64 over all 100,000 keys.  The
    query gain is large, so that the softmax stands on a few hundred keys spread over the whole cache (a
    slice or a page lost shows), and with a window of 48 keys every score depends on the rotation."""
    from gibbs_amd import ops
    from tests.plain import lfm2_plain as P
    dtype, nh, nkv, hd, page = torch.bfloat16, 8, 2, 64, 16
    seq_lens = [100000, 32768, 40]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, sum(-(-l // page) for l in seq_lens) + 3, seed=11)
    n = len(seq_lens)
    positions = [l - 1 for l in seq_lens]
    pos, row_req = i32(positions), i32(list(range(n)))
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=9)
    qg, kg = rnd(hd, seed=1) * 0.1 + 3.0, rnd(hd, seed=2) * 0.1 + 1
    inv_np = P.rope_inv_freq(hd, 1e6)
    inv = torch.from_numpy(inv_np).to(DEV)
    scale = 1 / math.sqrt(hd)
    got = ops.attention_decode_fused(qkv, n, nh, nkv, hd, kp, vp, table, n, pos, row_req, scale, q_gain=qg, k_gain=kg,
                                     eps=1e-5, inv_freq=inv, rotary_dim=hd, variant="half_split", window=window,
                                     max_seq=max(seq_lens), kind=kind, cos_sin=ops.rope_table(inv, 4096))
    # (the kernel rounds the prepared q and the new key to bfloat16, as the separate kernels store them; with
    # scores this large that rounding alone moves the output by 1 %, so the reference takes the same values)
    q = plain_qk(qkv[:, :nh * hd].view(n, nh, hd), qg, positions, inv_np, 1e-5).to(DEV).to(dtype).double()
    k_new = plain_qk(qkv[:, nh * hd:(nh + nkv) * hd].view(n, nkv, hd), kg, positions, inv_np, 1e-5).to(DEV).to(dtype).double()
    v_new = qkv[:, (nh + nkv) * hd:].view(n, nkv, hd)
    for r, p in enumerate(positions):
        pg = table[r, p // page].item()
        close(kp[pg, :, p % page], k_new[r], dtype, f"new key at position {p}", bf16=8e-3)
        assert torch.equal(vp[pg, :, p % page], v_new[r])
        k_all = torch.cat([ks[r][:p].double(), k_new[r:r + 1]])
        v_all = torch.cat([vs[r][:p].double(), v_new[r:r + 1].double()])
        want = attention_reference(q[r:r + 1], k_all, v_all, [p], scale, window)
        close(got[r].view(1, nh, hd), want, dtype, f"row at position {p}", bf16=1e-2)


def test_rope_table():
    from gibbs_amd import ops
    from gibbs_amd.parts.rope import rope_inv_freq
    inv = torch.from_numpy(rope_inv_freq(48, 1e6, "f32")).to(DEV)
    t = ops.rope_table(inv, 5000)
    ang = (torch.arange(5000, dtype=torch.float32, device=DEV)[:, None] * inv[None, :]).double()   # float32 products
    assert t.shape == (5000, 24, 2)
    assert (t[..., 0].double() - ang.cos()).abs().max().item() < 2e-7
    assert (t[..., 1].double() - ang.sin()).abs().max().item() < 2e-7


def test_argmax_rules():
    from gibbs_amd import ops
    nan, inf = float("nan"), float("inf")
    rows = torch.tensor([[1.0, 3.0, 3.0, 2.0, 0.0], [nan, 1.0, nan, 1.0, 0.0], [-inf] * 5, [nan] * 5,
                         [0.0, -1.0, -2.0, -3.0, 5.0]], device=DEV)
    assert ops.argmax(rows).tolist() == [1, 1, 0, 0, 4]
    big = rnd(3, 65536 + 37)
    big[1, 40000] = big[1, 70] = 99.0
    assert ops.argmax(big).tolist() == [big[0].argmax().item(), 70, big[2].argmax().item()]


def test_sample_against_plain():
    from gibbs_amd import ops
    from tests.plain import lfm2_plain as P
    V, M = 1000, 12
    logits = rnd(M, V, scale=3.0, seed=5)
    rng = np.random.default_rng(0)
    temp = np.array([0.8, 1.0, 0.3, 1.5] * 3, dtype=np.float32)
    top_p = np.array([0.9, 0.5, 1.0, 0.95] * 3, dtype=np.float32)
    top_k = np.array([50, 64, 5, 1] * 3, dtype=np.int32)
    u = rng.random(M).astype(np.float32)
    got = ops.sample(logits, torch.tensor(temp, device=DEV), torch.tensor(top_p, device=DEV), i32(top_k),
                     torch.tensor(u, device=DEV)).tolist()
    for m in range(M):
        cand, probs = P.nucleus(logits[m].cpu().numpy(), float(temp[m]), int(top_k[m]), float(top_p[m]))
        assert got[m] == P.draw(cand, probs, float(u[m])), f"row {m}"
    # temperature <= 1e-4 is greedy
    g = ops.sample(logits, torch.zeros(M, device=DEV), torch.tensor(top_p, device=DEV), i32(top_k), torch.tensor(u, device=DEV))
    assert g.tolist() == logits.argmax(-1).tolist()


@pytest.mark.parametrize("V,R", [(700, 64), (65536 + 37, 64), (97, 5)])
def test_repetition_penalty(V, R):
    """The kernel against the plain rule, row by row: greedy and sampled rows, tokens seen once and
    several times, positive and negative logits, ids outside the vocabulary and empty places in the
    list, rows without a penalty (left alone bit for bit)."""
    from gibbs_amd import ops
    from tests.plain import lfm2_plain as P
    rng = np.random.default_rng(V + R)
    M = 7
    logits = rnd(M, V, scale=3.0, seed=V)
    recent = rng.integers(0, min(V, 12), size=(M, R)).astype(np.int32)       # few distinct ids: many repeats
    recent[1, R // 2:] = -1                                                      # a short history
    recent[2, 0] = V + 5                                                         # an id outside the vocabulary
    recent[3] = rng.integers(0, V, size=R)
    recent[6] = -1                                                               # nothing recent
    penalty = np.array([1.3, 2.0, 1.1, 1.5, 1.0, 0.7, 1.8], dtype=np.float32)  # 1.0 and below: none
    temp = np.array([0.0, 0.8, 1e-4, 1.2, 0.0, 0.9, 0.7], dtype=np.float32)
    before = logits.clone()
    got = ops.repetition_penalty(logits, i32(recent), torch.tensor(penalty, device=DEV), torch.tensor(temp, device=DEV))
    assert got.data_ptr() == logits.data_ptr()
    got = got.cpu().numpy()
    for m in range(M):
        want = P.repetition_penalty(before[m].cpu().numpy(), [t for t in recent[m] if t >= 0], float(penalty[m]),
                                    greedy=bool(temp[m] <= 1e-4))
        assert np.array_equal(got[m], want), f"row {m}: {np.abs(got[m] - want).max()}"
    assert np.array_equal(got[4], before[4].cpu().numpy()) and np.array_equal(got[6], before[6].cpu().numpy())
    assert not np.array_equal(got[0], before[0].cpu().numpy())


@pytest.mark.parametrize("V", [65536, 50001, 700])
def test_sample_large_vocabulary_ties_and_specials(V):
    """Top-k by two walks over the row: vocabularies beyond one element per thread, a thousand values tied
    at the top (the smaller ids win), a row of equal logits (more ties than the candidate list holds),
    NaN (never a candidate) and -inf among the values, and -0 beside +0 at the top (equal values)."""
    from gibbs_amd import ops
    from tests.plain import lfm2_plain as P
    rng = np.random.default_rng(V)
    rows = [rng.standard_normal(V).astype(np.float32) * 3 for _ in range(6)]
    top = rows[1].max() + 1
    rows[1][rng.choice(V, size=min(1000, V // 2), replace=False)] = top          # many ties at the top
    rows[2][:] = 0.25                                                          # everything ties
    rows[3][rng.choice(V, size=V // 3, replace=False)] = np.nan
    rows[3][rng.choice(V, size=V // 4, replace=False)] = -np.inf
    rows[4] = -np.abs(rows[4]) - 1
    zeros = rng.choice(V, size=40, replace=False)
    rows[4][zeros[:20]] = 0.0
    rows[4][zeros[20:]] = -0.0
    rows[5][:] = -np.inf                                                       # nothing above -inf: still candidates
    rows[5][V // 2] = 1.0
    logits = torch.tensor(np.stack(rows), device=DEV)
    M = len(rows)
    for temp, p, k in [(0.8, 0.9, 50), (1.3, 1.0, 64), (0.5, 0.97, 7)]:
        u = rng.random(M).astype(np.float32)
        got = ops.sample(logits, torch.full((M,), temp, device=DEV), torch.full((M,), p, device=DEV),
                         i32([k] * M), torch.tensor(u, device=DEV)).tolist()
        for m in range(M):
            cand, probs = P.nucleus(rows[m], temp, k, p)
            assert got[m] == P.draw(cand, probs, float(u[m])), f"row {m}, k {k}"
    greedy = ops.sample(logits, torch.zeros(M, device=DEV), torch.ones(M, device=DEV), i32([50] * M), torch.zeros(M, device=DEV))
    assert greedy.tolist() == [P.argmax_first(r) for r in rows] == ops.argmax(logits).tolist()


# --------------------------------------------------------------------------- fused decode kernels
def rms_scale(x, eps):
    return 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)


@pytest.mark.parametrize("n,o,i", [(1, 64, 128), (8, 3072, 2048), (16, 331 * 8, 1000), (17, 200, 512), (64, 96, 4096), (5, 40, 72),
                                   (48, 8200, 512), (64, 3072, 2048),      # two tiles a workgroup; many rows, one tile
                                   (3, 20, 104), (8, 1001, 1000), (7, 4100, 104), (8, 4099, 2048), (9, 4100, 72),
                                   (12, 36, 200),                           # paired operands with ragged ends, both layouts
                                   (13, 2100, 264), (10, 40, 520)])         # 9 to 16 rows: two tiles of 8 rows in pairs; few features: staged
def test_skinny_store_with_rms_prologue(n, o, i):
    from gibbs_amd import ops
    x, w = rnd(n, i, dtype=torch.bfloat16, scale=3.0), rnd(o, i, dtype=torch.bfloat16, seed=1)
    plain = x.double() @ w.double().t()
    close(ops.skinny_store(x, w), plain, torch.bfloat16, "skinny_store", bf16=4e-3)
    got = ops.skinny_store(x, w, rms_eps=1e-5)
    close(got, plain * rms_scale(x, 1e-5), torch.bfloat16, "skinny_store rms", bf16=4e-3)
    assert torch.equal(ops.skinny_store(x, ops.PackedWeight(w), rms_eps=1e-5), got), "tile-ordered weights: same sums"


@pytest.mark.parametrize("n,o,i", [(1, 2048, 2048), (8, 2048, 8192), (33, 200, 512), (64, 72, 96), (64, 2048, 2048),
                                   (40, 1000, 4096),                        # many rows: partial sums over k, then the add
                                   (7, 36, 200), (8, 4100, 136), (2, 12, 8),
                                   (12, 2056, 200), (15, 4100, 136), (10, 36, 200)])   # 9 to 16 rows: pairs (8 and 16 features), staged
def test_skinny_residual(n, o, i):
    from gibbs_amd import ops
    y, w = rnd(n, i, dtype=torch.bfloat16), rnd(o, i, dtype=torch.bfloat16, seed=1)
    x = rnd(n, o, scale=2.0, seed=2)
    want = x.double() + y.double() @ w.double().t()
    mirror = torch.zeros(n, o, dtype=torch.bfloat16, device=DEV)
    x0 = x.clone()
    ops.skinny_residual(y, w, x, mirror)
    close(x, want, torch.float32, "skinny_residual", f32=2e-5)
    assert torch.equal(mirror, x.to(torch.bfloat16))
    ops.skinny_residual(y, ops.PackedWeight(w), x0, mirror)
    assert torch.equal(x0, x), "tile-ordered weights: same sums"


@pytest.mark.parametrize("n,f,i", [(1, 8192, 2048), (8, 200, 512), (40, 128, 72), (64, 256, 1024), (64, 6200, 256),
                                   (36, 8192, 2048),                        # two tiles a workgroup
                                   (5, 4100, 104), (8, 52, 40), (11, 4090, 72), (14, 2200, 104), (9, 60, 136)])
def test_skinny_glu(n, f, i):
    from gibbs_amd import ops
    x, w = rnd(n, i, dtype=torch.bfloat16, scale=2.0), rnd(2 * f, i, dtype=torch.bfloat16, scale=0.05, seed=1)
    gu = (x.double() @ w.double().t()) * rms_scale(x, 1e-6)
    want = F.silu(gu[:, :f]) * gu[:, f:]
    got = ops.skinny_glu(x, w, rms_eps=1e-6)
    close(got, want, torch.bfloat16, "skinny_glu", bf16=6e-3)
    assert torch.equal(ops.skinny_glu(x, ops.PackedWeight(w, groups=2), rms_eps=1e-6), got), "tile-ordered weights: same sums"
    with pytest.raises(ops.KernelError, match="row groups"):
        ops.skinny_glu(x, ops.PackedWeight(w), rms_eps=1e-6)


@pytest.mark.parametrize("n,c,i,k,bias", [(1, 2048, 2048, 3, False), (8, 72, 96, 4, True), (20, 40, 64, 2, True), (64, 96, 128, 3, False),
                                          (13, 2056, 96, 3, True), (16, 2104, 64, 4, False), (11, 40, 64, 2, True),   # 9 to 16 rows
                                          (31, 1, 512, 3, False), (2, 1, 520, 4, True)])   # one channel: sums that cancel
def test_skinny_conv(n, c, i, k, bias):
    """In-projection + convolution of decoded tokens against the unfused kernels and the reference."""
    from gibbs_amd import ops
    x = rnd(n, i, dtype=torch.bfloat16, scale=2.0)
    w = rnd(3 * c, i, dtype=torch.bfloat16, scale=0.1, seed=1)
    taps, b = rnd(c, k, seed=4), (rnd(c, seed=5) if bias else None)
    slots = torch.randperm(n + 3)[:n].to(torch.int32).to(DEV)
    ctx = i32([j % (k + 1) for j in range(n)])             # 0 (fresh), shorter than the history, longer
    state = rnd(n + 3, k - 1, c, seed=6)
    state2, state3 = state.clone(), state.clone()
    y = ops.skinny_conv(x, w, taps, b, state, slots, ctx, rms_eps=1e-5)
    y3 = ops.skinny_conv(x, ops.PackedWeight(w, groups=3), taps, b, state3, slots, ctx, rms_eps=1e-5)
    assert torch.equal(y3, y) and torch.equal(state3, state), "tile-ordered weights: same sums"
    bcx = (x.double() @ w.double().t()) * rms_scale(x, 1e-5)
    B, C, X = bcx[:, :c], bcx[:, c:2 * c], bcx[:, 2 * c:]
    bx = B * X
    want_state = state2.double().clone()
    for r in range(n):
        hist = state2[slots[r]].double().clone()
        for j in range(k - 1):
            if int(ctx[r]) - (k - 1) + j < 0:
                hist[j] = 0
        window = torch.cat([hist, bx[r:r + 1]])
        cv = (window * taps.double().t()).sum(0) + (b.double() if bias else 0)
        close(y[r], C[r] * cv, torch.bfloat16, f"skinny_conv row {r}", bf16=8e-3)
        want_state[slots[r]] = window[1:]
    # All rows' states against one scale.  The new entry B * x is a product of two float32 sums over k, whose
    # rounding error follows the size of their terms, not of the sums: with one channel, a row whose B or x
    # cancels to almost nothing has a tiny state of its own and misses a bound taken from that row alone
    # (random shapes found such rows), though every value is as exact as float32 sums get.
    close(state, want_state, torch.float32, "state", f32=2e-5)
    untouched = [s for s in range(n + 3) if s not in slots.tolist()]
    assert torch.equal(state[untouched], state2[untouched])


def test_embed_and_residual_mirror():
    from gibbs_amd import ops
    table = rnd(50, 72, dtype=torch.bfloat16)
    mirror = torch.zeros(4, 72, dtype=torch.bfloat16, device=DEV)
    x = ops.embed(table, i32([3, 49, 0, 3]), 4, mirror=mirror)
    assert torch.equal(mirror.float(), x)
    d = rnd(4, 72, dtype=torch.bfloat16, seed=3)
    x0 = x.clone()
    ops.residual_add(x, d, mirror)
    assert torch.equal(x, x0 + d.float()) and torch.equal(mirror, x.to(torch.bfloat16))
    parts = rnd(3, 4, 72, seed=4)                                      # float32 partial sums, added in order
    x1 = x.clone()
    ops.residual_add(x, parts, mirror)
    assert torch.equal(x, ((x1 + parts[0]) + parts[1]) + parts[2]) and torch.equal(mirror, x.to(torch.bfloat16))
    out = ops.add_rmsnorm(x, None, None, 1e-5, torch.bfloat16)       # no gain
    close(out, F.rms_norm(x.double(), (72,), None, 1e-5), torch.bfloat16, "gain-free norm")


@pytest.mark.parametrize("kind", ["valu", "mfma", "mfma-merge-pass"])
@pytest.mark.parametrize("n_splits,table_len,waves", [(1, 0, 8), (4, 20, 4), (None, 1024, None)])   # rows at 699 and 32 beyond a table of 20
@pytest.mark.parametrize("variant", ["half_split", "interleaved"])
@pytest.mark.parametrize("nh,nkv,hd,rot,page,window", [(4, 2, 16, 16, 16, None), (32, 8, 64, 64, 16, None), (6, 1, 48, 32, 8, None),
                                                       (5, 5, 80, 80, 32, 37), (16, 2, 128, 128, 16, None), (24, 2, 32, 32, 16, None)])
def test_attention_decode_fused(nh, nkv, hd, rot, page, window, variant, n_splits, table_len, waves, kind):
    """The fused decode attention against the separate kernels: same pages afterwards, same output,
    for rows at a page's first slot, its last slot, position 0 and far into the cache."""
    from gibbs_amd import ops
    from gibbs_amd.parts.rope import rope_inv_freq
    dtype = torch.bfloat16
    seq_lens = [700, 1, 33, 16, 17]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 120, seed=7)
    n = len(seq_lens)
    pos, row_req = i32([l - 1 for l in seq_lens]), i32(list(range(n)))
    qkv = rnd(n, (nh + 2 * nkv) * hd, dtype=dtype, seed=9)
    qg, kg = rnd(hd, seed=1) * 0.1 + 1, rnd(hd, seed=2) * 0.1 + 1
    inv = torch.from_numpy(rope_inv_freq(rot, 10000.0, "f32")).to(DEV)
    scale = 1 / math.sqrt(hd)
    kp2, vp2, qkv2 = kp.clone(), vp.clone(), qkv.clone()
    ops.qk_rope_kv(qkv2, n, nh, nkv, hd, q_gain=qg, k_gain=kg, eps=1e-6, inv_freq=inv, rotary_dim=rot, variant=variant,
                   pos=pos, row_req=row_req, kpages=kp2, vpages=vp2, table=table, n_req=n)
    want = ops.attention_decode(qkv2, n, nh, nkv, hd, kp2, vp2, table, n, pos, row_req, scale, window, max_seq=700, n_splits=3)
    kp1, vp1 = kp.clone(), vp.clone()
    got = ops.attention_decode_fused(qkv, n, nh, nkv, hd, kp1, vp1, table, n, pos, row_req, scale, q_gain=qg,
                                     k_gain=kg, eps=1e-6, inv_freq=inv, rotary_dim=rot, variant=variant,
                                     window=window, max_seq=700, n_splits=n_splits, waves=waves, kind=kind,
                                     cos_sin=ops.rope_table(inv, table_len) if table_len else None)
    close(kp1, kp2, dtype, "new keys in the pages", bf16=8e-3)
    assert torch.equal(vp1, vp2)
    close(got, want, dtype, "fused decode attention", bf16=8e-3)


@pytest.mark.parametrize("n_rows,nh,nkv,hd,n_splits", [(64, 32, 8, 64, 8), (3, 6, 2, 48, 5), (2, 4, 1, 128, 40),
                                                       (4200, 8, 8, 16, 2)])
def test_slices_merged_by_the_last_to_finish_or_by_a_second_kernel(n_rows, nh, nkv, hd, n_splits):
    """The key slices of a row are merged by the workgroup that finishes last, through memory that the other
    workgroups wrote in the same kernel; a second kernel does the same arithmetic where it is asked for, or where
    rows x groups of heads exceed the counters (4,200 x 8).  Up to 8 slices both add in the same order: the results
    are equal bit for bit, call after call (the counters are left at zero, no partial result is read before it has
    arrived); beyond 8 they differ by rounding."""
    from gibbs_amd import ops
    dtype, page = torch.bfloat16, 16
    long_rows = n_rows <= 64
    seq_lens = [(900 + 37 * r) if long_rows else 20 + r % 13 for r in range(n_rows)]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, sum(-(-l // page) for l in seq_lens) + 8, seed=3)
    pos = i32([l - 1 for l in seq_lens])
    scale = 1 / math.sqrt(hd)
    # (other queries in every call: a partial result left over from the call before would show)
    for call in range(12 if long_rows else 2):
        qc = rnd(n_rows, nh * hd, dtype=dtype, seed=4 + call) * (1 + call % 3)
        got = ops.attention_decode(qc, n_rows, nh, nkv, hd, kp, vp, table, n_rows, pos, None, scale, None,
                                   max_seq=max(seq_lens), n_splits=n_splits, waves=4, kind="mfma")
        want = ops.attention_decode(qc, n_rows, nh, nkv, hd, kp, vp, table, n_rows, pos, None, scale, None,
                                    max_seq=max(seq_lens), n_splits=n_splits, waves=4, kind="mfma-merge-pass")
        if n_splits <= 8:
            assert torch.equal(got, want), f"call {call}"
        else:
            close(got, want, dtype, f"merged in the kernel, call {call}", bf16=4e-3)
        for r in range(min(n_rows, 3)):
            ref = attention_reference(qc[r:r + 1].view(1, nh, hd), ks[r], vs[r], [seq_lens[r] - 1], scale, None)
            close(got[r].view(1, nh, hd), ref, dtype, f"row {r}, call {call}", bf16=1e-2)


def test_attention_block_table_segments():
    """Requests with more pages than the kernels keep in LDS at a time (pages of 2 tokens, 2,300
    keys): the fast kernels cross from one segment of the block table to the next."""
    from gibbs_amd import ops
    from gibbs_amd.parts.rope import rope_inv_freq
    dtype, nh, nkv, hd, page = torch.bfloat16, 2, 1, 32, 2
    seq_lens = [2300, 1100]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 1800, seed=5)
    scale = 1 / math.sqrt(hd)
    # prompt portions ending at the last key of each request
    q_lens = [130, 70]
    ctx = [s - q for s, q in zip(seq_lens, q_lens)]
    cu = np.concatenate([[0], np.cumsum(q_lens)])
    n = int(cu[-1])
    q = rnd(n, nh * hd, dtype=dtype, seed=9)
    out = ops.attention_prefill(q, n, nh, nkv, hd, kp, vp, table, 2, i32(cu), i32(ctx), scale)
    for r in range(2):
        rows = slice(int(cu[r]), int(cu[r + 1]))
        want = attention_reference(q[rows].view(-1, nh, hd), ks[r], vs[r], list(range(ctx[r], seq_lens[r])), scale, None)
        close(out[rows].view(-1, nh, hd), want, dtype, f"prefill over segments, request {r}", bf16=1e-2)
    # decoded rows at the last positions, one key slice and several
    pos, row_req = i32([l - 1 for l in seq_lens]), i32([0, 1])
    qd = rnd(2, nh * hd, dtype=dtype, seed=3)
    want = ops.attention_plain(qd, 2, nh, nkv, hd, kp, vp, table, 2, pos, row_req, scale)
    for ns in (1, 3):
        close(ops.attention_decode(qd, 2, nh, nkv, hd, kp, vp, table, 2, pos, row_req, scale, n_splits=ns), want, dtype,
              f"decode over segments, {ns} slices", bf16=1e-2)
        qkv = torch.cat([qd, rnd(2, 2 * nkv * hd, dtype=dtype, seed=4)], dim=1).contiguous()
        kp1, vp1, kp2, vp2, qkv2 = kp.clone(), vp.clone(), kp.clone(), vp.clone(), qkv.clone()
        ops.qk_rope_kv(qkv2, 2, nh, nkv, hd, q_gain=None, k_gain=None, eps=0.0, inv_freq=None, rotary_dim=0,
                       variant="half_split", pos=pos, row_req=row_req, kpages=kp2, vpages=vp2, table=table, n_req=2)
        ref = ops.attention_plain(qkv2, 2, nh, nkv, hd, kp2, vp2, table, 2, pos, row_req, scale)
        got = ops.attention_decode_fused(qkv, 2, nh, nkv, hd, kp1, vp1, table, 2, pos, row_req, scale, q_gain=None,
                                         k_gain=None, eps=0.0, inv_freq=None, rotary_dim=0, variant="half_split",
                                         n_splits=ns)
        close(got, ref, dtype, f"fused decode over segments, {ns} slices", bf16=1e-2)


def test_decode_tail_one_kernel():
    """The end of a captured decode step: next tokens (first largest logit, NaN never wins), the log, positions,
    cached lengths, draws and per-row step counts, and the tokens' embeddings as the next step's rows."""
    from gibbs_amd import ops
    n, V, hidden, cap = 5, 1001, 72, 4
    logits = rnd(n, V, seed=3)
    logits[1, 7] = logits[1, 900] = 50.0           # a tie: the first wins
    logits[2, 3] = float("nan")
    table = rnd(V, hidden, dtype=torch.bfloat16, seed=4)
    ids, pos, ctx = i32([9] * n), i32([10, 20, 30, 40, 50]), i32([10, 20, 30, 40, 50])
    log, steps = torch.full((cap, n), -1, dtype=torch.int32, device=DEV), i32([0, 1, 2, 3, 4])
    u, u_all = torch.zeros(n, device=DEV), rnd(cap, n, seed=5)
    x, mirror = torch.zeros(n, hidden, device=DEV), torch.zeros(n, hidden, dtype=torch.bfloat16, device=DEV)
    ops.decode_tail(logits, ids, pos, ctx, log, steps, u, u_all, n, table, x, mirror)
    want = torch.nan_to_num(logits, nan=-float("inf")).argmax(-1).int()
    want[1] = 7
    assert torch.equal(ids, want) and pos.tolist() == [11, 21, 31, 41, 51] and ctx.tolist() == pos.tolist()
    assert steps.tolist() == [1, 2, 3, 4, 5]
    for r in range(n):
        assert [int(log[s, r]) for s in range(cap)] == [int(want[r]) if s == r else -1 for s in range(cap)]   # row 4: beyond the log
        assert float(u[r]) == (float(u_all[r + 1, r]) if r + 1 < cap else 0.0)
    assert torch.equal(x, table[want.long()].float()) and torch.equal(mirror, table[want.long()])
    # tokens that a sampling kernel has put into ids; no embedding asked for
    ids2, steps2 = i32([4, 3, 2, 1, 0]), i32([0] * n)
    ops.decode_tail(None, ids2, pos, ctx, log, steps2, None, None, n)
    assert log[0].tolist() == [4, 3, 2, 1, 0] and pos.tolist() == [12, 22, 32, 42, 52] and ids2.tolist() == [4, 3, 2, 1, 0]


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh", "gelu", "relu"])
def test_activations_of_the_gated_kernels(dtype, activation):
    """The activation table in the stand-alone kernel (both precisions, vector and scalar variants) and in the
    epilogue of the fused decode product."""
    from gibbs_amd import ops
    act = {"silu": F.silu, "gelu_tanh": lambda g: F.gelu(g, approximate="tanh"), "gelu": F.gelu, "relu": F.relu}[activation]
    for f in (200, 203):
        gu = rnd(7, 2 * f, dtype=dtype, scale=2.0, seed=f)
        close(ops.glu(gu, activation), act(gu[:, :f].double()) * gu[:, f:].double(), dtype, f"glu {activation} {f}")
    if dtype == torch.bfloat16:
        x = rnd(5, 96, dtype=dtype, seed=1)
        w = rnd(2 * 48, 96, dtype=dtype, scale=0.2, seed=2)
        want = act(x.double() @ w[:48].double().T) * (x.double() @ w[48:].double().T)
        close(ops.skinny_glu(x, w, activation=activation), want, dtype, f"skinny_glu {activation}")
    with pytest.raises(ops.KernelError, match="not implemented"):
        ops.glu(rnd(2, 8, dtype=dtype), "softsign")


@pytest.mark.parametrize("dtype", DT)
def test_attention_plain_with_score_slopes(dtype):
    """A linear bias on the scores by distance: slope[h] * (key position - query position)."""
    from gibbs_amd import ops
    nh, nkv, hd, page = 6, 2, 32, 8
    seq_lens = [70, 9]
    kp, vp, table, ks, vs = paged_setup(dtype, nkv, hd, page, seq_lens, 24, seed=3)
    rows = [(0, list(range(60, 70))), (1, [8])]
    pos, row_req = i32([p for _, ps in rows for p in ps]), i32([r for r, ps in rows for _ in ps])
    n = pos.numel()
    q = rnd(n, nh * hd, dtype=dtype, seed=9)
    slopes = torch.tensor([0.5 ** (h + 1) for h in range(nh)], dtype=torch.float32, device=DEV)
    out = ops.attention_plain(q, n, nh, nkv, hd, kp, vp, table, 2, pos, row_req, hd ** -0.5, slopes=slopes)
    at = 0
    for r, ps in rows:
        kk, vv = ks[r].double().repeat_interleave(nh // nkv, 1), vs[r].double().repeat_interleave(nh // nkv, 1)
        for i, p in enumerate(ps):
            s = torch.einsum("hd,lhd->hl", q[at + i].double().view(nh, hd), kk[:p + 1]) * hd ** -0.5
            s = s + slopes.double()[:, None] * (torch.arange(p + 1, device=DEV) - p)[None, :]
            want = torch.einsum("hl,lhd->hd", s.softmax(-1), vv[:p + 1])
            close(out[at + i].view(nh, hd), want, dtype, f"slopes request {r} position {p}", f32=2e-5, bf16=1e-2)
        at += len(ps)

"""The decode attention's entry point that allocates nothing (`gibbs_attention_decode_static`: the
key slices' partial results go to an array the library holds on the GPU), called through ctypes as
a caller without an allocator would, against the existing entry point with a workspace of the
caller's: two calls in a row, the second with a smaller input, whose slices then fill only the
head of the array that the first call left full."""
import ctypes
import math
from ctypes import c_float, c_int, c_long, c_void_p

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
NH, NKV, HD, PAGE = 8, 2, 64, 16


def _library():
    from gibbs_amd import build
    lib = ctypes.CDLL(build.ensure_built())
    common = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_long, c_long, c_float,
              c_int, c_int, c_int, c_int, c_int, c_void_p]
    lib.gibbs_attention_decode.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + common
    lib.gibbs_attention_decode_static.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p] + common
    for fn in (lib.gibbs_attention_decode, lib.gibbs_attention_decode_static):
        fn.restype = c_int
    lib.gibbs_attention_decode_workspace.argtypes = [c_int, c_int, c_int, c_int]
    lib.gibbs_attention_decode_workspace.restype = c_long
    lib.gibbs_attention_decode_static_capacity.restype = c_long
    lib.gibbs_last_error.restype = ctypes.c_char_p
    return lib


def _case(seq_lens, seed):
    """Keys and values of `seq_lens` requests on shuffled pages, one query row at the end of each."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    rng = np.random.default_rng(seed)
    pages_of = [-(-n // PAGE) for n in seq_lens]
    num_pages = sum(pages_of) + 3
    kp = torch.randn((num_pages, NKV, PAGE, HD), generator=g).to(torch.bfloat16).to(DEV)
    vp = torch.randn((num_pages, NKV, PAGE, HD), generator=g).to(torch.bfloat16).to(DEV)
    order = rng.permutation(num_pages).tolist()
    table = np.zeros((len(seq_lens), max(pages_of)), dtype=np.int32)
    for r, n in enumerate(pages_of):
        table[r, :n] = [order.pop() for _ in range(n)]
    q = torch.randn((len(seq_lens), NH * HD), generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([n - 1 for n in seq_lens], dtype=torch.int32, device=DEV)
    row_req = torch.arange(len(seq_lens), dtype=torch.int32, device=DEV)
    return q, kp, vp, torch.from_numpy(table).to(DEV), pos, row_req, num_pages


def _reference(q, kp, vp, table, pos):
    """Plain float64 attention of every row over its pages."""
    out = torch.zeros((q.shape[0], NH, HD), dtype=torch.float64)
    kp, vp, table = kp.double().cpu(), vp.double().cpu(), table.cpu()
    for r in range(q.shape[0]):
        n = int(pos[r]) + 1
        pages = table[r, :-(-n // PAGE)].long()
        k = kp[pages].permute(0, 2, 1, 3).reshape(-1, NKV, HD)[:n].repeat_interleave(NH // NKV, 1)
        v = vp[pages].permute(0, 2, 1, 3).reshape(-1, NKV, HD)[:n].repeat_interleave(NH // NKV, 1)
        s = torch.einsum("hd,lhd->hl", q[r].double().cpu().view(NH, HD), k) / math.sqrt(HD)
        out[r] = torch.einsum("hl,lhd->hd", s.softmax(-1), v)
    return out.view(q.shape[0], NH * HD)


def test_static_scratch_entry_point_twice_in_a_row():
    lib = _library()
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    capacity = lib.gibbs_attention_decode_static_capacity()
    assert capacity > 0
    # the first call's slices fill 6 rows x 8 heads x 8 slices; the second call's 2 x 8 x 3
    for seq_lens, n_splits, seed in (([700, 1, 33, 16, 500, 129], 8, 1), ([300, 40], 3, 2)):
        q, kp, vp, table, pos, row_req, num_pages = _case(seq_lens, seed)
        n = len(seq_lens)
        need = lib.gibbs_attention_decode_workspace(n, NH, HD, n_splits)
        assert 0 < need <= capacity
        common = (pos.data_ptr(), row_req.data_ptr(), table.data_ptr(), table.shape[1], PAGE, num_pages, n, NH, NKV, HD,
                  NH * HD, NH * HD, 1 / math.sqrt(HD), 0, n_splits, 4, 0, max(seq_lens), stream)
        partial = torch.full((need,), float("nan"), dtype=torch.float32, device=DEV)
        want = torch.zeros((n, NH * HD), dtype=torch.bfloat16, device=DEV)
        got = torch.zeros_like(want)
        assert lib.gibbs_attention_decode(q.data_ptr(), kp.data_ptr(), vp.data_ptr(), want.data_ptr(),
                                          partial.data_ptr(), *common) == 0, lib.gibbs_last_error()
        assert lib.gibbs_attention_decode_static(q.data_ptr(), kp.data_ptr(), vp.data_ptr(), got.data_ptr(),
                                                 *common) == 0, lib.gibbs_last_error()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"static scratch and caller's workspace differ for {seq_lens}"
        ref = _reference(q, kp, vp, table, pos)
        err = (got.double().cpu() - ref).abs().max().item()
        assert err <= 1e-2 * ref.abs().max().item(), f"attention differs from the float64 reference: {err}"


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    lib = _library()
    q, kp, vp, table, pos, row_req, num_pages = _case([64, 64], 3)
    capacity = lib.gibbs_attention_decode_static_capacity()
    n_splits = capacity // (2 * NH * (HD + 2)) + 1           # one slice more than the array holds
    assert n_splits <= 65535
    out = torch.zeros((2, NH * HD), dtype=torch.bfloat16, device=DEV)
    status = lib.gibbs_attention_decode_static(
        q.data_ptr(), kp.data_ptr(), vp.data_ptr(), out.data_ptr(), pos.data_ptr(), row_req.data_ptr(), table.data_ptr(),
        table.shape[1], PAGE, num_pages, 2, NH, NKV, HD, NH * HD, NH * HD, 1 / math.sqrt(HD), 0, int(n_splits), 4, 0, 64,
        c_void_p(torch.cuda.current_stream().cuda_stream))
    assert status != 0 and b"floats of scratch" in lib.gibbs_last_error()
    torch.cuda.synchronize()
    assert not out.any(), "a refused call must not run"

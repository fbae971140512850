"""lsattn_decode_attention_static (the decode call whose split-K partials live in the library's per-GPU static array)
against lsattn_decode_attention with caller-allocated partials: same kernels, so the outputs must agree bit for bit.
Two calls in a row, the second on a smaller input, so that rows left in the array by the first call would show."""
import ctypes as C

import pytest
import torch

from tests.helpers import assert_lse_close, assert_o_close, decode_case

pytestmark = pytest.mark.gpu


def _both(lsa, seed, B, Hq, Hkv, lens, BS, dtype=torch.float16, spare_rows=0):
    ck = lsa.longserve_cuda_kernels
    dev = "cuda:0"
    D = 128
    q, kv, table, b_req, b_len = decode_case(seed, B, Hq, Hkv, D, lens, sum(lens) + 257, dtype)
    q, kv, table, b_req, b_len = (t.to(dev) for t in (q, kv, table, b_req, b_len))
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    max_len = max(lens)
    nblk = (max_len + BS - 1) // BS + spare_rows  # (the caller's buffers may be taller than the longest request needs)
    mid_o = torch.full((nblk, B, Hq, D), float("nan"), device=dev)
    mid_l = torch.full((nblk, B, Hq), float("nan"), device=dev)
    o_ref = torch.full((B, Hq, D), float("nan"), device=dev)
    l_ref = torch.full((B, Hq), float("nan"), device=dev)
    ck.flash_decoding(mid_o, mid_l, q, k, v, table, b_req, b_len, max_len, o_ref, l_ref, BS)
    o = torch.full((B, Hq, D), float("nan"), device=dev)
    l = torch.full((B, Hq), float("nan"), device=dev)
    ck.flash_decoding_static(q, k, v, table, b_req, b_len, max_len, o, l, BS)
    torch.cuda.synchronize()
    return (o, l), (o_ref, l_ref), (q, kv, table, b_req, b_len)


def test_static_scratch_decode_matches_caller_scratch_twice(lsa):
    from oracle import attn_oracle as orc
    # first call: ragged batch with an empty request, GQA 32/8, many partial rows
    lens1 = [4000, 0, 1, 2049, 777, 3100]
    (o, l), (o_ref, l_ref), inp = _both(lsa, 41, len(lens1), 32, 8, lens1, 256)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    q, kv, table, b_req, b_len = (t.cpu() for t in inp)
    oo, ll = orc.decode_full(q, kv[:, :8], kv[:, 8:], table, b_req, b_len)
    assert_o_close(o, oo, "static decode O")
    assert_lse_close(l, ll, "static decode LSE")
    # second call, smaller in every dimension (fewer requests, heads, rows, shorter blocks): the array still holds
    # the first call's partials
    lens2 = [300, 65, 129]
    (o, l), (o_ref, l_ref), inp = _both(lsa, 42, len(lens2), 8, 2, lens2, 64, torch.bfloat16)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    q, kv, table, b_req, b_len = (t.cpu() for t in inp)
    oo, ll = orc.decode_full(q, kv[:, :2], kv[:, 2:], table, b_req, b_len)
    assert_o_close(o, oo, "static decode O (second call)")
    assert_lse_close(l, ll, "static decode LSE (second call)")


def test_static_scratch_matches_a_caller_whose_buffers_are_taller_than_the_batch_needs(lsa):
    """The caller-scratch call on buffers of 70 rows for a batch that reaches 5: the merge's shape follows the rows the
    longest request can reach in both entry points, so the bits agree whatever the buffer's height."""
    lens = [1200, 37, 640]
    (o, l), (o_ref, l_ref), _ = _both(lsa, 43, len(lens), 32, 8, lens, 256, spare_rows=65)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
    # and a long request at small batch, where both take the wide merge (80 rows)
    lens = [20480, 5000]
    (o, l), (o_ref, l_ref), _ = _both(lsa, 44, len(lens), 8, 2, lens, 256, spare_rows=3)
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref)


def test_static_scratch_call_replays_from_a_hip_graph(lsa):
    """The use the entry point names: recorded into a HIP graph (after one eager call, which looks the array's address
    up) and replayed on new inputs written into the same buffers; every replay against the eager caller-scratch call."""
    ck = lsa.longserve_cuda_kernels
    dev = "cuda:0"
    B, Hq, Hkv, D, BS = 3, 16, 4, 128, 128
    lens = [900, 130, 513]
    max_len = max(lens)
    cases = [decode_case(50 + i, B, Hq, Hkv, D, lens, sum(lens) + 100) for i in range(3)]
    q, kv, table, b_req, b_len = (t.to(dev).clone() for t in cases[0])
    o = torch.empty((B, Hq, D), device=dev)
    l = torch.empty((B, Hq), device=dev)
    ck.flash_decoding_static(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len, max_len, o, l, BS)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        ck.flash_decoding_static(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len, max_len, o, l, BS)
    nblk = (max_len + BS - 1) // BS
    for case in cases[1:] + cases[:1]:
        # new queries and new pool contents under the same request table (a case's table goes with its own b_req_idx:
        # rows of the table that belong to no request hold the out-of-range padding value)
        q.copy_(case[0].to(dev))
        kv.copy_(case[1].to(dev))
        o.fill_(float("nan")); l.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        mid_o = torch.empty((nblk, B, Hq, D), device=dev)
        mid_l = torch.empty((nblk, B, Hq), device=dev)
        o_ref = torch.empty((B, Hq, D), device=dev)
        l_ref = torch.empty((B, Hq), device=dev)
        ck.flash_decoding(mid_o, mid_l, q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len, max_len, o_ref, l_ref, BS)
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(l, l_ref)


def test_static_scratch_rejects_oversize_and_caller_buffers(lsa):
    from loongserve_amd import _lib
    ck = lsa.longserve_cuda_kernels
    dev = "cuda:0"
    B, Hq, Hkv, D, BS = 64, 32, 8, 128, 16
    max_len = 32768  # 2048 rows x 64 x 32 x 129 x 4 B = 2.2 GB of partials: beyond the array
    q = torch.zeros((B, Hq, D), dtype=torch.float16, device=dev)
    kv = torch.zeros((8, 2 * Hkv, D), dtype=torch.float16, device=dev)
    table = torch.zeros((B, max_len), dtype=torch.int32, device=dev)
    b_req = torch.arange(B, dtype=torch.int32, device=dev)
    b_len = torch.ones(B, dtype=torch.int32, device=dev)
    o = torch.zeros((B, Hq, D), device=dev)
    l = torch.zeros((B, Hq), device=dev)
    with pytest.raises(RuntimeError, match="workspace"):
        ck.flash_decoding_static(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len, max_len, o, l, BS)
    # a block that names partial buffers is refused: the entry point owns them
    mid_o = torch.zeros((1, B, Hq, D), device=dev)
    mid_l = torch.zeros((1, B, Hq), device=dev)
    a1 = ck._stage1_args(mid_o, mid_l, q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len, 1, 256)
    a2 = ck._stage2_args(o, l, b_len, mid_o, mid_l, 256)
    assert _lib.load().lsattn_decode_attention_static(C.byref(a1), C.byref(a2), None) == -1
    torch.cuda.synchronize()

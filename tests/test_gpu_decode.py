"""GPU parity of token-indexed flash decoding against the CPU oracle (through the C ABI)."""
import math

import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import assert_lse_close, assert_o_close, decode_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,BS", [(32, 8, 256), (4, 4, 64), (16, 8, 16), (10, 5, 128), (12, 4, 256), (8, 1, 32), (14, 2, 256),
                                       (5, 1, 64), (12, 2, 128), (3, 1, 16), (8, 1, 256), (16, 2, 64), (9, 1, 128), (32, 2, 256), (8, 2, 100), (4, 4, 7)])
def test_stage1_stage2_vs_oracle(lsa, dtype, Hq, Hkv, BS):
    _check_stage1_stage2(lsa, dtype, Hq, Hkv, BS)


def _check_stage1_stage2(lsa, dtype, Hq, Hkv, BS):
    print("case", dtype, Hq, Hkv, BS, flush=True)
    B, D = 5, 128
    lens = [700, 1, 256, 33, 1025]
    q, kv, table, b_req, b_len = decode_case(100, B, Hq, Hkv, D, lens, 3000, dtype)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    nblk = (max(lens) + BS - 1) // BS
    mid_o = torch.full((nblk, B, Hq, D), float("nan"))
    mid_l = torch.full((nblk, B, Hq), float("nan"))
    orc.decode_stage1(q, k, v, table, b_req, b_len, max(lens), mid_o, mid_l, BS)
    kvd = kv.to(DEV)
    from loongserve_amd import decoding
    # opt-in layout first: groups of blocks merged into one partial; the rows of a group's other blocks are marked empty,
    # rows past the request stay untouched, and the merge gives the same result
    assert not decoding.STAGE1_MERGES_BLOCKS  # the default is the reference's one partial per block
    decoding.STAGE1_MERGES_BLOCKS = True
    try:
        mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
        ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
        lsa.longserve_flash_decode_stage1(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV),
                                          b_len.to(DEV), max(lens), mo_d, ml_d, BS)
    finally:
        decoding.STAGE1_MERGES_BLOCKS = False
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
    torch.cuda.synchronize()
    assert torch.equal(torch.isnan(ml_d.cpu()), torch.isnan(mid_l))                 # the same rows are written
    merge = min(16, decoding._fused_block_seq(BS, B, max(lens), Hkv) // BS)
    first = (torch.arange(nblk) % merge == 0)[:, None, None]
    assert bool((torch.isinf(ml_d.cpu()) == (~first & ~torch.isnan(mid_l))).all())   # -inf exactly on a group's other rows
    o_ref, l_ref = orc.decode_full(q, k, v, table, b_req, b_len)
    assert_o_close(o_d, o_ref, "o from merged groups")
    assert_lse_close(l_d, l_ref, "lse from merged groups")
    # then the default: one partial per block, the reference's buffers
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    lsa.longserve_flash_decode_stage1(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV),
                                      b_len.to(DEV), max(lens), mo_d, ml_d, BS)
    torch.cuda.synchronize()
    # blocks past a request's length are left untouched, like the reference
    written = ~torch.isnan(mid_l)
    assert torch.equal(torch.isnan(ml_d.cpu()), ~written)
    mo_c, ml_c = mo_d.cpu(), ml_d.cpu()
    assert_o_close(torch.where(written[..., None], mo_c, torch.zeros(())), torch.where(written[..., None], mid_o, torch.zeros(())),
                   "mid_o")
    assert_lse_close(ml_c[written], mid_l[written], "mid_lse")
    for odt in (torch.float32, dtype):
        o_d = torch.empty(B, Hq, D, dtype=odt, device=DEV)
        l_d = torch.empty(B, Hq, device=DEV)
        lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
        torch.cuda.synchronize()
        o_ref, l_ref = orc.decode_full(q, k, v, table, b_req, b_len)
        if odt == torch.bfloat16:
            assert_o_close(o_d, o_ref, "o bf16 out", max_abs=4e-3, rel=4e-3)  # 8-bit mantissa output
        else:
            assert_o_close(o_d, o_ref, "o")
        assert_lse_close(l_d, l_ref, "lse")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("merge", [2, 8, 16])
@pytest.mark.parametrize("Hq,Hkv,BS,lens", [
    (32, 8, 16, [700, 1, 256, 33, 1025]),      # group 4, many short blocks
    (8, 1, 128, [5000]),                       # group 8 (two rounds of four heads), one request: the waves split a block
    (16, 1, 256, [3000, 9000]),                # group 16 (two tasks per KV head), few workgroups: split path
    (16, 4, 32, [100, 2049, 17, 640, 1, 999]),  # group 4, ragged
    (4, 4, 128, [4097, 130]),                  # one query head per KV head
])
def test_stage1_forced_merge_blocks(lsa, dtype, merge, Hq, Hkv, BS, lens):
    _check_merge_blocks(lsa, dtype, merge, Hq, Hkv, BS, lens)


def _check_merge_blocks(lsa, dtype, merge, Hq, Hkv, BS, lens):
    """merge_blocks = m of flash_decoding_stage1: the partial of blocks [m j, m j + m) of a request in row m j, the other
    rows the request reaches marked empty, rows past it untouched; checked row by row against the oracle's stage 1 at
    block size m * BS, and through stage 2 at the caller's block size."""
    print("case", dtype, merge, Hq, Hkv, BS, lens, flush=True)
    B, D = len(lens), 128
    q, kv, table, b_req, b_len = decode_case(500 + merge, B, Hq, Hkv, D, lens, sum(lens) + 300, dtype)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    nblk = (max(lens) + BS - 1) // BS
    ngrp = (nblk + merge - 1) // merge
    ref_o = torch.full((ngrp, B, Hq, D), float("nan"))
    ref_l = torch.full((ngrp, B, Hq), float("nan"))
    orc.decode_stage1(q, k, v, table, b_req, b_len, max(lens), ref_o, ref_l, BS * merge)
    kvd = kv.to(DEV)
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    lsa.longserve_cuda_kernels.flash_decoding_stage1(mo_d, ml_d, q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV),
                                                     b_len.to(DEV), max(lens), BS, merge)
    torch.cuda.synchronize()
    mo_c, ml_c = mo_d.cpu(), ml_d.cpu()
    for b in range(B):
        reach = (lens[b] + BS - 1) // BS
        for i in range(nblk):
            if i >= reach:
                assert torch.isnan(ml_c[i, b]).all() and torch.isnan(mo_c[i, b]).all(), (b, i)   # untouched
            elif i % merge:
                assert (ml_c[i, b] == float("-inf")).all() and torch.isnan(mo_c[i, b]).all(), (b, i)  # empty, mid_o left alone
            else:
                assert_o_close(mo_c[i, b], ref_o[i // merge, b], "mid_o row %d request %d" % (i, b))
                assert_lse_close(ml_c[i, b], ref_l[i // merge, b], "mid_lse row %d request %d" % (i, b))
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
    torch.cuda.synchronize()
    o_ref, l_ref = orc.decode_full(q, k, v, table, b_req, b_len)
    assert_o_close(o_d, o_ref, "o")
    assert_lse_close(l_d, l_ref, "lse")


@pytest.fixture(params=["mfma", "split", "mfma listed"], ids=["plain", "split", "listed"])
def matrix_pipe(tuning, request):
    """Stage 1 through the matrix-pipe kernel wherever its conditions hold, whatever the launch's size: its plain shape
    (a wave per 256 tokens; blocks a multiple of 32 tokens; by itself the library takes it for large launches), the
    shape whose four waves split a block (blocks a multiple of 128 tokens; small launches of groups of four and more),
    and the plain shape over a list of the units that exist (by itself: launches of very many workgroups)."""
    tuning(decode_stage1=request.param.split()[0], decode_listed="on" if "listed" in request.param else "off")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,BS", [(32, 8, 256), (4, 4, 64), (10, 5, 128), (8, 1, 32), (5, 1, 64), (9, 1, 128), (16, 2, 64), (32, 2, 256),
                                       (17, 1, 96), (66, 2, 32), (7, 7, 160)])
def test_matrix_pipe_stage1_stage2_vs_oracle(lsa, matrix_pipe, dtype, Hq, Hkv, BS):
    """Groups of 1 to 33 query heads (padded to 16-row operands, 17 and 33: a second / third task with one live row),
    blocks of one to eight 32-token batches, requests of 1 token, of a partial batch and of a partial block."""
    _check_stage1_stage2(lsa, dtype, Hq, Hkv, BS)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("merge", [2, 16])
@pytest.mark.parametrize("Hq,Hkv,BS,lens", [
    (8, 1, 128, [5000]),
    (16, 1, 256, [3000, 9000]),
    (16, 4, 32, [100, 2049, 17, 640, 1, 999]),
    (40, 8, 64, [4097, 130]),
])
def test_matrix_pipe_stage1_forced_merge_blocks(lsa, matrix_pipe, dtype, merge, Hq, Hkv, BS, lens):
    _check_merge_blocks(lsa, dtype, merge, Hq, Hkv, BS, lens)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_large_group_launch_that_takes_the_matrix_pipe_by_itself(lsa, dtype):
    """64 query heads over 8 KV heads, 2 requests of about 17000 tokens: 2 x 8 x 67 waves of the matrix-pipe kernel, the
    library's own choice (nothing forced), through the fused call and through the two stages."""
    lsa.set_tuning()
    B, Hq, Hkv, D, BS = 2, 64, 8, 128, 256
    lens = [17000, 16411]
    q, kv, table, b_req, b_len = decode_case(77, B, Hq, Hkv, D, lens, sum(lens) + 1000, dtype)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    o_ref, l_ref = orc.decode_full(q, k, v, table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_token_decode_attention_flash_decoding(q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV), mo_d, ml_d, B, max(lens),
                                                        Hq, D, kvd[:, :Hkv], kvd[:, Hkv:], BS, o_d, l_d)
    torch.cuda.synchronize()
    assert_o_close(o_d, o_ref, "o, fused call")
    assert_lse_close(l_d, l_ref, "lse, fused call")
    mo_d.fill_(float("nan"))
    ml_d.fill_(float("nan"))
    lsa.longserve_flash_decode_stage1(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV), b_len.to(DEV), max(lens),
                                      mo_d, ml_d, BS)
    lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
    torch.cuda.synchronize()
    reach = torch.tensor([(n + BS - 1) // BS for n in lens])
    assert torch.equal(torch.isnan(ml_d.cpu()), (torch.arange(nblk)[:, None] >= reach[None, :])[:, :, None].expand(nblk, B, Hq))
    assert_o_close(o_d, o_ref, "o, two stages")
    assert_lse_close(l_d, l_ref, "lse, two stages")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_skewed_batch_that_walks_the_unit_list_by_itself(lsa, dtype):
    """One request of 40000 tokens among 127 of 1 to 300 (and two of none), 64 tokens per partial: the plain grid would
    be 157 x 2 x 130 = 40820 workgroups, nearly all of them without work, so the library walks the list of the units
    that exist (its own choice: nothing forced).  Two stages, per-block partials; rows no request reaches stay
    untouched."""
    lsa.set_tuning()
    import random
    rng = random.Random(5)
    B, Hq, Hkv, D, BS = 130, 32, 8, 128, 64
    lens = [rng.randint(1, 300) for _ in range(B)]
    lens[37] = 40000
    lens[0] = lens[129] = lens[64] = 0
    lens[1] = 64
    q, kv, table, b_req, b_len = decode_case(78, B, Hq, Hkv, D, lens, sum(lens) + 1000, dtype)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    live = [b for b in range(B) if lens[b] > 0]
    o_ref, l_ref = orc.decode_full(q[live], k, v, table, b_req[live], b_len[live])
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_flash_decode_stage1(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV), b_len.to(DEV), max(lens),
                                      mo_d, ml_d, BS)
    lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
    torch.cuda.synchronize()
    reach = torch.tensor([(n + BS - 1) // BS for n in lens])
    assert torch.equal(torch.isnan(ml_d.cpu()), (torch.arange(nblk)[:, None] >= reach[None, :])[:, :, None].expand(nblk, B, Hq))
    assert_o_close(o_d[live], o_ref, "o, two stages")
    assert_lse_close(l_d[live], l_ref, "lse, two stages")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_call_gives_the_same_bits_with_either_layout_of_its_partials(lsa, monkeypatch, dtype):
    """The fused call keeps the partials of a request side by side in mid_o; with the reference's layout (a block of all
    requests after the other, what the two stage functions use) it must return the same bits."""
    B, Hq, Hkv, D, BS = 5, 16, 4, 128, 64
    lens = [700, 1, 64, 2049, 333]
    q, kv, table, b_req, b_len = decode_case(91, B, Hq, Hkv, D, lens, sum(lens) + 100, dtype)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    res = []
    for by_request in (True, False):
        monkeypatch.setattr(lsa.longserve_cuda_kernels, "FUSED_PARTIALS_BY_REQUEST", by_request)
        mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
        ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
        o_d = torch.empty(B, Hq, D, device=DEV)
        l_d = torch.empty(B, Hq, device=DEV)
        lsa.longserve_cuda_kernels.flash_decoding(mo_d, ml_d, q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV),
                                                  b_len.to(DEV), max(lens), o_d, l_d, BS)
        torch.cuda.synchronize()
        assert_o_close(o_d, o_ref, "o, partials by request %s" % by_request)
        assert_lse_close(l_d, l_ref, "lse, partials by request %s" % by_request)
        res.append((o_d.cpu(), l_d.cpu(), ml_d.cpu()))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    # the same partials, in the other order: request b's block i is row (b, i) of the one and row (i, b) of the other
    by_req = res[0][2].reshape(B, nblk, Hq)
    for b, n in enumerate(lens):
        for i in range((n + BS - 1) // BS):
            assert torch.equal(by_req[b, i], res[1][2][i, b]), (b, i)


@pytest.mark.parametrize("B", [1024, 1025])
def test_unit_list_at_its_largest_batch_and_past_it(lsa, tuning, B):
    """The list of units is numbered in LDS for up to 1024 requests; a larger batch takes the plain grid whatever the
    tuning block asks for.  Requests of 0 to 120 tokens and one of 9000, 64 tokens per partial."""
    import random
    tuning(decode_stage1="mfma", decode_listed="on")
    rng = random.Random(B)
    Hq, Hkv, D, BS = 8, 2, 128, 64
    lens = [rng.randint(0, 120) for _ in range(B)]
    lens[B // 3] = 9000
    q, kv, table, b_req, b_len = decode_case(500 + B, B, Hq, Hkv, D, lens, sum(lens) + 300)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    lsa.longserve_flash_decode_stage1(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV), b_len.to(DEV), max(lens),
                                      mo_d, ml_d, BS)
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_flash_decode_stage2(mo_d, ml_d, b_len.to(DEV), o_d, l_d, BS)
    torch.cuda.synchronize()
    live = [b for b in range(B) if lens[b] > 0]
    reach = torch.tensor([(n + BS - 1) // BS for n in lens])
    assert torch.equal(torch.isnan(ml_d.cpu()), (torch.arange(nblk)[:, None] >= reach[None, :])[:, :, None].expand(nblk, B, Hq))
    assert_o_close(o_d[live], o_ref[live], "o")
    assert_lse_close(l_d[live], l_ref[live], "lse")


def test_gather_indices_bit_exact(lsa):
    # q = 0 and V[slot] = ordinal code of the slot: the set of gathered slots is read back from O*len
    B, H, D = 3, 2, 128
    lens = [37, 300, 1000]
    q, kv, table, b_req, b_len = decode_case(200, B, H, H, D, lens, 1500)
    q.zero_()
    kv[:, H:, :] = (torch.arange(1500, dtype=torch.float32) % 2048)[:, None, None].to(torch.float16)
    kv[:, H:, 1] = 1.0
    kvd = kv.to(DEV)
    BS = 256
    nblk = (max(lens) + BS - 1) // BS
    mo = torch.zeros(nblk, B, H, D, device=DEV)
    ml = torch.zeros(nblk, B, H, device=DEV)
    o, lse = lsa.longserve_token_decode_attention_flash_decoding(q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV),
                                                                 mo, ml, B, max(lens), H, D, kvd[:, :H], kvd[:, H:], BS)
    torch.cuda.synchronize()
    assert o.dtype == torch.float32
    for b in range(B):
        slots = table[int(b_req[b]), :lens[b]].long()
        want = float(kv[slots, H, 0].float().sum())
        got = float(o[b, 0, 0]) * lens[b]
        assert abs(got - want) <= 1e-4 * max(want, 1.0) + 0.5, (got, want)
        assert abs(float(o[b, 1, 1]) - 1.0) < 1e-6
        assert abs(float(lse[b, 0]) - math.log(lens[b])) < 1e-5


def test_multi_instance_decode_with_empty_peer(lsa):
    # each request's KV split over 3 instances; one peer holds nothing for one request
    from loongserve_amd.simulate import DecodeInstance, multi_instance_decode
    B, Hq, Hkv, D = 4, 8, 2, 128
    lens = [900, 64, 333, 2000]
    q, kv, table, b_req, b_len = decode_case(300, B, Hq, Hkv, D, lens, 4000)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    cuts = [[300, 600], [0, 64], [111, 111], [700, 1300]]  # ranges: master [0,c0), peer1 [c0,c1), peer2 [c1,len)
    kvd = kv.to(DEV)
    insts = []
    for r in range(3):
        t = torch.full_like(table, orc.INT32_PAD)
        ln = []
        for b in range(B):
            lo = [0, cuts[b][0], cuts[b][1]][r]
            hi = [cuts[b][0], cuts[b][1], lens[b]][r]
            t[int(b_req[b]), :hi - lo] = table[int(b_req[b]), lo:hi]
            ln.append(hi - lo)
        insts.append(DecodeInstance(kvd, t.to(DEV), b_req.to(DEV), torch.tensor(ln, dtype=torch.int32, device=DEV), max(ln)))
    o, lse = multi_instance_decode(q.to(DEV), insts, Hkv)
    torch.cuda.synchronize()
    assert o.dtype == torch.float16
    assert_o_close(o, o_ref, "multi-instance o")
    assert_lse_close(lse, l_ref, "multi-instance lse")


def test_stage2_empty_request_defined(lsa):
    B, H, D = 2, 4, 128
    mo = torch.randn(3, B, H, D, device=DEV)
    ml = torch.randn(3, B, H, device=DEV)
    o = torch.full((B, H, D), 7.0, device=DEV)
    l = torch.full((B, H), 7.0, device=DEV)
    lsa.longserve_flash_decode_stage2(mo, ml, torch.tensor([0, 3], dtype=torch.int32, device=DEV), o, l, 1)
    torch.cuda.synchronize()
    assert torch.all(o[0] == 0) and torch.all(torch.isinf(l[0]) & (l[0] < 0))
    o_ref, l_ref = orc.lse_merge([(mo[i, 1].cpu(), ml[i, 1].cpu()) for i in range(3)])
    assert_o_close(o[1], o_ref, "o", max_abs=1e-5, rel=1e-5)
    assert_lse_close(l[1], l_ref, "lse", rel=1e-5)


@pytest.mark.parametrize("nblk", [1, 7, 31, 64, 65, 300, 1029])
def test_stage2_alone_over_few_and_many_partials(lsa, nblk):
    """The merge on its own, on random partials: every count of blocks around the points where the kernel changes its
    walk (rows in flight per slice, the wide launch for many partials of few rows), empty partials in between, requests
    that use fewer blocks than the buffer has, fp32 and fp16 outputs."""
    print("case nblk", nblk, flush=True)
    B, H, D, BS = 3, 5, 128, 16
    g = torch.Generator().manual_seed(nblk)
    mo = torch.randn(nblk, B, H, D, generator=g)
    ml = torch.randn(nblk, B, H, generator=g) * 6
    ml[torch.rand(nblk, B, H, generator=g) < 0.15] = float("-inf")
    lens = torch.tensor([nblk * BS, max(1, (nblk * BS) // 3 + 1), 0], dtype=torch.int32)
    o_ref = torch.empty(B, H, D)
    l_ref = torch.empty(B, H)
    orc.decode_stage2(mo, ml, lens, o_ref, l_ref, BS)
    for odt in (torch.float32, torch.float16):
        o = torch.full((B, H, D), 9.0, dtype=odt, device=DEV)
        l = torch.full((B, H), 9.0, device=DEV)
        lsa.longserve_flash_decode_stage2(mo.to(DEV), ml.to(DEV), lens.to(DEV), o, l, BS)
        torch.cuda.synchronize()
        # a (b, h) whose partials are all empty merges to (0, -inf), like a request without tokens
        dead = torch.isinf(l_ref) & (l_ref < 0)
        assert torch.equal(torch.isinf(l.cpu()) & (l.cpu() < 0), dead)
        assert torch.all(o.cpu()[dead] == 0)
        if odt == torch.float32:
            assert_o_close(o, torch.where(dead[..., None], torch.zeros(()), o_ref), "o", max_abs=2e-5, rel=1e-5)
        else:
            assert_o_close(o, torch.where(dead[..., None], torch.zeros(()), o_ref), "o fp16", max_abs=4e-3, rel=1e-3)
        assert_lse_close(l, l_ref, "lse", rel=1e-5)


@pytest.mark.parametrize("B,H,nblk", [(70, 32, 1030), (300, 8, 520), (9, 5, 1024)])
def test_stage2_of_one_long_request_among_many_short_ones(lsa, B, H, nblk):
    """The merge of a batch in which one request has a thousand partials and the others a few: more (request, head) pairs
    than the narrow launch's bound for the wide one, with enough partials for the wide launch all the same (70 x 32), too
    many pairs for it (300 x 8), and a small batch; the long request in the middle of the batch, so that the heads of a
    request and the requests of a head are both told apart in the grid."""
    print("case", B, H, nblk, flush=True)
    D, BS = 128, 16
    g = torch.Generator().manual_seed(B * 1000 + nblk)
    mo = torch.randn(nblk, B, H, D, generator=g)
    ml = torch.randn(nblk, B, H, generator=g) * 5
    ml[torch.rand(nblk, B, H, generator=g) < 0.1] = float("-inf")
    lens = torch.randint(1, 4 * BS, (B,), generator=g).to(torch.int32)
    lens[B // 2] = nblk * BS - 3
    lens[0] = 0
    o_ref = torch.empty(B, H, D)
    l_ref = torch.empty(B, H)
    orc.decode_stage2(mo, ml, lens, o_ref, l_ref, BS)
    o = torch.full((B, H, D), 9.0, device=DEV)
    l = torch.full((B, H), 9.0, device=DEV)
    lsa.longserve_flash_decode_stage2(mo.to(DEV), ml.to(DEV), lens.to(DEV), o, l, BS)
    torch.cuda.synchronize()
    dead = torch.isinf(l_ref) & (l_ref < 0)
    assert torch.equal(torch.isinf(l.cpu()) & (l.cpu() < 0), dead)
    assert_o_close(o, torch.where(dead[..., None], torch.zeros(()), o_ref), "o", max_abs=2e-5, rel=1e-5)
    assert_lse_close(l, l_ref, "lse", rel=1e-5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_peaked_softmax_keeps_the_bars(lsa, dtype):
    """Scores of magnitude up to ~64: a few tokens carry each request."""
    B, Hq, Hkv, D, BS = 3, 4, 2, 128, 256
    lens = [3000, 700, 64]
    q, kv, table, b_req, b_len = decode_case(5, B, Hq, Hkv, D, lens, 5000, dtype)
    g = torch.Generator().manual_seed(9)
    q = (torch.randn(q.shape, generator=g) * 4).to(dtype)
    kv[:, :Hkv] = (torch.randn((5000, Hkv, D), generator=g) * 4).to(dtype)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    mo = torch.empty(nblk, B, Hq, D, device=DEV)
    ml = torch.empty(nblk, B, Hq, device=DEV)
    o, l = lsa.longserve_token_decode_attention_flash_decoding(q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV), mo, ml, B,
                                                               max(lens), Hq, D, kvd[:, :Hkv], kvd[:, Hkv:], BS)
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "o")
    assert_lse_close(l, l_ref, "lse")


def test_one_request_of_a_million_tokens(lsa):
    """The longest context the serving configs name (1M tokens) in one request: the fused call's coarsest split, the wide
    merge, 32-bit positions near 2^20 and slot numbers above 2^20.  Checked through closed forms rather than a CPU pass
    over 1 GB of rows: q = 0 gives O = mean of the request's V rows and LSE = ln(n); a query equal to 40 x one key's
    direction puts almost all weight on that token."""
    n, Hq, Hkv, D, BS = 1_048_576, 4, 2, 128, 256
    pool = n + 4096
    g = torch.Generator(device=DEV).manual_seed(11)
    kv = (torch.randn((pool, 2 * Hkv, D), generator=g, device=DEV) * 0.5).half()
    perm = torch.randperm(pool, generator=g, device=DEV)[:n].to(torch.int32)
    table = torch.full((2, n + 8), 2147483647, dtype=torch.int32, device=DEV)
    table[1, :n] = perm
    b_req = torch.tensor([1], dtype=torch.int32, device=DEV)
    b_len = torch.tensor([n], dtype=torch.int32, device=DEV)
    nblk = (n + BS - 1) // BS
    mo = torch.empty(nblk, 1, Hq, D, device=DEV)
    ml = torch.empty(nblk, 1, Hq, device=DEV)
    q = torch.zeros(1, Hq, D, dtype=torch.float16, device=DEV)
    o, lse = lsa.longserve_token_decode_attention_flash_decoding(q, table, b_req, b_len, mo, ml, 1, n, Hq, D, kv[:, :Hkv], kv[:, Hkv:], BS)
    torch.cuda.synchronize()
    v_mean = kv[perm.long(), Hkv:].double().mean(0)                        # [Hkv, D]
    want = v_mean.repeat_interleave(Hq // Hkv, 0)[None].float()
    assert (o - want).abs().max().item() <= 2e-5
    assert (lse - math.log(n)).abs().max().item() <= 1e-4 * math.log(n)
    # a peaked query: token t of the request (any position, here near the end) dominates
    t = n - 12345
    slot = int(perm[t])
    kdir = kv[slot, :Hkv].float()                                          # [Hkv, D]
    q2 = (kdir * (40.0 / kdir.norm(dim=-1, keepdim=True))).repeat_interleave(Hq // Hkv, 0)[None].half()
    o2, lse2 = lsa.longserve_token_decode_attention_flash_decoding(q2, table, b_req, b_len, mo, ml, 1, n, Hq, D, kv[:, :Hkv], kv[:, Hkv:], BS)
    torch.cuda.synchronize()
    s = torch.einsum("hd,nhd->hn", q2[0].float().view(Hkv, Hq // Hkv, D).reshape(Hq, D)[::Hq // Hkv], kv[perm.long(), :Hkv].float()) / math.sqrt(D)
    lse_ref = torch.logsumexp(s.double(), dim=-1).float().repeat_interleave(Hq // Hkv)
    o_ref = torch.einsum("hn,nhd->hd", torch.softmax(s.double(), dim=-1), kv[perm.long(), Hkv:].double()).float().repeat_interleave(Hq // Hkv, 0)
    assert_lse_close(lse2[0], lse_ref.cpu(), "peaked lse")
    assert_o_close(o2[0], o_ref.cpu(), "peaked o")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,BS,lens", [
    (32, 8, 256, [5000, 1, 256, 257, 0, 9000, 300]),          # two task groups of four KV heads
    (8, 1, 256, [3000, 700, 12000, 256]),                     # one KV head: the four waves of a workgroup hold four shares
    (16, 2, 512, [100, 5000, 2049, 17, 1024, 1, 999]),        # two KV heads: two waves on tasks, two shares per workgroup
    (40, 5, 256, [4097, 130, 0, 0, 6000]),                    # five KV heads: the second task group half empty
    (17, 1, 1024, [40000, 3, 2048]),                          # a second task with one live row; a split of 1024 dealt in blocks of 256
])
def test_fused_call_in_equal_shares(lsa, tuning, dtype, Hq, Hkv, BS, lens):
    """The fused call with stage 1 dealt in equal shares of blocks (forced: these launches are far smaller than the ones
    the library deals that way by itself): shares that end inside a request, requests inside a share, requests without
    tokens, more workers than blocks; the partials' buffers start as NaN (every row the merge reads must have been
    written, as a partial or as an empty row) and are as tall as the caller's BLOCK_SEQ of 256 makes them."""
    tuning(decode_listed="shares")
    B, D = len(lens), 128
    q, kv, table, b_req, b_len = decode_case(500 + Hq + len(lens), B, Hq, Hkv, D, lens, sum(lens) + 500, dtype)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + 255) // 256
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    o_d = torch.full((B, Hq, D), float("nan"), device=DEV)
    l_d = torch.full((B, Hq), float("nan"), device=DEV)
    lsa.longserve_cuda_kernels.flash_decoding(mo_d, ml_d, q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV), b_len.to(DEV),
                                              max(lens), o_d, l_d, BS)
    torch.cuda.synchronize()
    assert_o_close(o_d, o_ref, "o")
    assert_lse_close(l_d, l_ref, "lse")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_large_batch_that_is_dealt_in_equal_shares_by_itself(lsa, dtype):
    """48 requests of 1 to 9000 tokens, 32 query heads on 8 KV heads: 48 x 36 blocks of 256 tokens at most, enough for the
    library to deal them in equal shares by itself (nothing forced) in the fused call; the two stages on their own keep
    one partial per block."""
    lsa.set_tuning()
    import random
    rng = random.Random(17)
    B, Hq, Hkv, D, BS = 48, 32, 8, 128, 256
    lens = [rng.randint(1, 9000) for _ in range(B)]
    lens[5] = 9000
    lens[6] = 0
    q, kv, table, b_req, b_len = decode_case(79, B, Hq, Hkv, D, lens, sum(lens) + 1000, dtype)
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
    kvd = kv.to(DEV)
    nblk = (max(lens) + BS - 1) // BS
    mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
    ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
    o_d = torch.empty(B, Hq, D, device=DEV)
    l_d = torch.empty(B, Hq, device=DEV)
    lsa.longserve_token_decode_attention_flash_decoding(q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV), mo_d, ml_d, B, max(lens),
                                                        Hq, D, kvd[:, :Hkv], kvd[:, Hkv:], BS, o_d, l_d)
    torch.cuda.synchronize()
    assert_o_close(o_d, o_ref, "o, fused call")
    assert_lse_close(l_d, l_ref, "lse, fused call")
    # (in equal shares a request has far fewer partials than blocks: most rows of the buffer are never written)
    ml = ml_d.cpu()
    assert int(torch.isnan(ml).sum()) > int(torch.isfinite(ml).sum()) > 0
    # the entry point that brings its own partials takes the same route (its array holds a row per 256 tokens here)
    o_s = torch.full((B, Hq, D), float("nan"), device=DEV)
    l_s = torch.full((B, Hq), float("nan"), device=DEV)
    lsa.longserve_cuda_kernels.flash_decoding_static(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], table.to(DEV), b_req.to(DEV), b_len.to(DEV),
                                                     max(lens), o_s, l_s, 1024)
    torch.cuda.synchronize()
    assert torch.equal(o_s, o_d) and torch.equal(l_s, l_d)
    # recorded in a HIP graph and replayed on new queries: every replay against the eager call
    qd = q.to(DEV).clone()
    td, rd, ld = table.to(DEV), b_req.to(DEV), b_len.to(DEV)
    o_g = torch.empty(B, Hq, D, device=DEV)
    l_g = torch.empty(B, Hq, device=DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lsa.longserve_token_decode_attention_flash_decoding(qd, td, rd, ld, mo_d, ml_d, B, max(lens), Hq, D, kvd[:, :Hkv], kvd[:, Hkv:], BS, o_g, l_g)
    for rep in range(3):
        qd.copy_((torch.randn(q.shape, generator=torch.Generator().manual_seed(900 + rep)) * 0.5).to(dtype))
        o_g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        o_e = torch.empty(B, Hq, D, device=DEV)
        l_e = torch.empty(B, Hq, device=DEV)
        lsa.longserve_token_decode_attention_flash_decoding(qd, td, rd, ld, mo_d, ml_d, B, max(lens), Hq, D, kvd[:, :Hkv], kvd[:, Hkv:], BS, o_e, l_e)
        torch.cuda.synchronize()
        assert torch.equal(o_g, o_e) and torch.equal(l_g, l_e), "replay %d" % rep


@pytest.mark.parametrize("seed", [5, 19, 77])
def test_random_fused_calls_in_equal_shares(lsa, tuning, seed):
    """Seeded random sweep of the fused call with stage 1 forced into equal shares, and of the entry point that brings
    its own partials on the same inputs (bit for bit the same where the caller's buffers are tall enough for blocks of
    256 tokens, which is what that entry point always deals): 1 to 40 requests of 0 to 9000 tokens (several empty,
    of one token, of exactly a block), groups of 1 to 20 query heads on 1 to 8 KV heads, both dtypes, the caller's
    BLOCK_SEQ 256 to 2048, buffers as tall as that makes them."""
    import random
    rng = random.Random(seed)
    tuning(decode_listed="shares")
    for case in range(8):
        dtype = rng.choice([torch.float16, torch.bfloat16])
        Hkv = rng.choice([1, 2, 3, 5, 8])
        Hq = Hkv * rng.choice([1, 2, 4, 5, 8, 16, 17, 20])
        BS = rng.choice([256, 512, 1024, 2048])
        B = rng.choice([1, 2, 3, 9, 17, 40])
        lens = [rng.choice([0, 1, 2, 255, 256, 257, 511, 512, 1000, 2049, 4096, 9000, rng.randint(1, 9000)]) for _ in range(B)]
        if max(lens) == 0:
            lens[0] = 300
        print("case", seed, case, dtype, Hq, Hkv, BS, lens, flush=True)
        D = 128
        q, kv, table, b_req, b_len = decode_case(7000 + 100 * seed + case, B, Hq, Hkv, D, lens, sum(lens) + 300, dtype)
        o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], table, b_req, b_len)
        kvd, qd, td, rd, ld = kv.to(DEV), q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV)
        nblk = (max(lens) + BS - 1) // BS
        mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
        ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
        o_d = torch.full((B, Hq, D), float("nan"), device=DEV)
        l_d = torch.full((B, Hq), float("nan"), device=DEV)
        lsa.longserve_cuda_kernels.flash_decoding(mo_d, ml_d, qd, kvd[:, :Hkv], kvd[:, Hkv:], td, rd, ld, max(lens), o_d, l_d, BS)
        torch.cuda.synchronize()
        what = "seed %d case %d" % (seed, case)
        live = torch.tensor(lens) > 0
        assert_o_close(o_d[live.to(DEV)], o_ref[live], "o, " + what)
        assert_lse_close(l_d, l_ref, "lse, " + what)
        o_s = torch.full((B, Hq, D), float("nan"), device=DEV)
        l_s = torch.full((B, Hq), float("nan"), device=DEV)
        lsa.longserve_cuda_kernels.flash_decoding_static(qd, kvd[:, :Hkv], kvd[:, Hkv:], td, rd, ld, max(lens), o_s, l_s, BS)
        torch.cuda.synchronize()
        assert_o_close(o_s[live.to(DEV)], o_ref[live], "o, own partials, " + what)
        assert_lse_close(l_s, l_ref, "lse, own partials, " + what)
        if nblk >= (max(lens) + 255) // 256:  # (both calls then deal blocks of 256 tokens: the same sums in the same order)
            assert torch.equal(o_s[live.to(DEV)], o_d[live.to(DEV)]) and torch.equal(l_s, l_d), "own partials, " + what


@pytest.mark.parametrize("seed", [3, 11, 42])
def test_random_decode_shapes_on_both_stage1_kernels(lsa, tuning, seed):
    """Seeded random sweep of stage 1 + stage 2 against the oracle, once with the library's own choice of stage-1 kernel
    and once through each shape of the matrix-pipe kernel wherever its conditions hold (plain grid, split waves, listed
    units): ragged batches with requests of a single token,
    of exactly a block, and of a block plus one; groups of 1 to 20 query heads per KV head; blocks of 32 to 512 tokens;
    per-block partials and merged groups of blocks; both dtypes; unused rows and requests in the table."""
    import random
    rng = random.Random(seed)
    for case in range(10):
        dtype = rng.choice([torch.float16, torch.bfloat16])
        Hkv = rng.choice([1, 2, 3, 8])
        group = rng.choice([1, 2, 4, 5, 7, 8, 9, 12, 16, 17, 20])
        Hq = Hkv * group
        BS = rng.choice([32, 64, 96, 128, 256, 384, 512])
        B = rng.choice([1, 2, 5, 9])
        lens = [rng.choice([1, 2, 31, 32, 33, BS - 1, BS, BS + 1, 2 * BS, 3 * BS + 7, 700, 1500, 2600]) for _ in range(B)]
        lens = [max(n, 1) for n in lens]
        merge = rng.choice([1, 1, 2, 4, 16])
        print("case", seed, case, dtype, Hq, Hkv, BS, lens, merge, flush=True)
        D = 128
        q, kv, table, b_req, b_len = decode_case(9000 + 100 * seed + case, B, Hq, Hkv, D, lens, sum(lens) + 200, dtype)
        k, v = kv[:, :Hkv], kv[:, Hkv:]
        o_ref, l_ref = orc.decode_full(q, k, v, table, b_req, b_len)
        kvd, qd, td, rd, ld = kv.to(DEV), q.to(DEV), table.to(DEV), b_req.to(DEV), b_len.to(DEV)
        nblk = (max(lens) + BS - 1) // BS
        for forced in (False, "mfma", "split", "mfma listed"):
            if forced:
                tuning(decode_stage1=forced.split()[0], decode_listed="on" if "listed" in forced else "off")
            else:
                tuning()
            mo_d = torch.full((nblk, B, Hq, D), float("nan"), device=DEV)
            ml_d = torch.full((nblk, B, Hq), float("nan"), device=DEV)
            lsa.longserve_cuda_kernels.flash_decoding_stage1(mo_d, ml_d, qd, kvd[:, :Hkv], kvd[:, Hkv:], td, rd, ld, max(lens), BS, merge)
            o_d = torch.empty(B, Hq, D, device=DEV)
            l_d = torch.empty(B, Hq, device=DEV)
            lsa.longserve_flash_decode_stage2(mo_d, ml_d, ld, o_d, l_d, BS)
            torch.cuda.synchronize()
            what = "seed %d case %d%s" % (seed, case, ", matrix pipe shape " + forced if forced else "")
            reach = torch.tensor([(n + BS - 1) // BS for n in lens])
            untouched = (torch.arange(nblk)[:, None] >= reach[None, :])[:, :, None].expand(nblk, B, Hq)
            assert torch.equal(torch.isnan(ml_d.cpu()), untouched), "rows written, " + what
            assert_o_close(o_d, o_ref, "o, " + what)
            assert_lse_close(l_d, l_ref, "lse, " + what)

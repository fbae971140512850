"""GPU parity of the context-migration KV copy + registration against the oracle (bit-exact, through the C ABI)."""
import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import meta

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _i32(x):
    return torch.tensor(x, dtype=torch.int32)


def test_kv_ranges_match_oracle(lsa):
    g = torch.Generator().manual_seed(3)
    B = 700  # more than one 256-thread block
    first = torch.randint(0, 9, (B,), generator=g, dtype=torch.int32)
    begin = first + torch.randint(-5, 4000, (B,), generator=g, dtype=torch.int32)
    end = begin + torch.randint(0, 5000, (B,), generator=g, dtype=torch.int32)
    for P in (1, 2, 4, 7):
        rb, re, nl = lsa.pre_copy_and_register_kv(begin.to(DEV), end.to(DEV), first.to(DEV), P)
        rb_o, re_o, nl_o = orc.kv_ranges(begin.tolist(), end.tolist(), first.tolist(), P)
        assert torch.equal(rb.cpu(), rb_o) and torch.equal(re.cpu(), re_o) and torch.equal(nl.cpu(), nl_o)
    empty = torch.empty(0, dtype=torch.int32, device=DEV)
    rb, re, nl = lsa.pre_copy_and_register_kv(empty, empty, empty, 4)
    assert rb.numel() == 0


def test_kv_ranges_of_a_window_that_starts_before_the_first_held_token(lsa):
    """The ceil of a negative quotient, in the form the reference documents (Python floor division of x + P - 1,
    copy_and_register_kv.py:42-45), in literal numbers: window [0, 3) or [4, 20) against a chunk whose first held token is
    9, 5 or 8 with 4 peers.  The reference's own windows never start more than P - 1 before the first held token, where
    every reading of the division agrees; for the others a C-style truncating division would give -1 / 0 / 0 here."""
    begin, end, first = _i32([0, 0, 4]).to(DEV), _i32([3, 3, 20]).to(DEV), _i32([9, 5, 8]).to(DEV)
    rb, re, nl = lsa.pre_copy_and_register_kv(begin, end, first, 4)
    assert rb.tolist() == [-2, -1, -1]          # ceil(-9/4), ceil(-5/4), ceil(-4/4)
    assert re.tolist() == [-1, 0, 3]            # ceil(-6/4), ceil(-2/4), ceil(12/4)
    assert nl.tolist() == [1, 1, 4]
    rb_o, re_o, nl_o = orc.kv_ranges([0, 0, 4], [3, 3, 20], [9, 5, 8], 4)
    assert torch.equal(rb.cpu(), rb_o) and torch.equal(re.cpu(), re_o) and torch.equal(nl.cpu(), nl_o)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("register", [True, False])
def test_copy_and_register_matches_oracle(lsa, dtype, register):
    g = torch.Generator().manual_seed(17)
    B, Hkv, D = 6, 8, 128
    lens = [300, 0, 1, 700, 257, 40]          # new_kv_cache_len per request (one empty)
    begin = [0, 5, 3, 10, 0, 2]
    begin[4] = -1                              # negative bound: the reference skips the request
    start_loc, off = [], 0
    for n, b0 in zip(lens, begin):
        start_loc.append(off)
        off += n + max(b0, 0) + 3
    kv = torch.randn(off + 8, 2 * Hkv, D, generator=g).to(dtype)
    pool_n = 4000
    pool = torch.randn(pool_n, 2 * Hkv, D, generator=g).to(dtype)
    table = torch.full((B + 2, 1200), orc.INT32_PAD, dtype=torch.int32)
    new_len, rb = _i32(lens), _i32(begin)
    re = rb + new_len
    len_sum = torch.cumsum(new_len, 0, dtype=torch.int64)
    cur = _i32([7, 0, 100, 0, 5, 1159])
    b_req = _i32([3, 0, 7, 1, 5, 2])
    used = 11
    mem_index = torch.randperm(pool_n, generator=g)[:used + int(len_sum[-1])].to(torch.int32)
    max_len = 600                               # rounds up to 768: request 3 (700 rows) is copied whole
    pool_o, table_o = pool.clone(), table.clone()
    orc.kv_copy_register(B, new_len, rb, re, len_sum, kv, _i32(start_loc), cur, mem_index, pool_o, table_o, b_req, used, max_len, register)
    pool_d, table_d = pool.to(DEV), table.to(DEV)
    lsa.destindex_copy_and_register_kv(B, new_len.to(DEV), rb.to(DEV), re.to(DEV), len_sum.to(DEV), kv.to(DEV), _i32(start_loc).to(DEV),
                                       cur.to(DEV), mem_index.to(DEV), pool_d, table_d, b_req.to(DEV), used, max_len, register)
    torch.cuda.synchronize()
    assert torch.equal(pool_d.cpu().view(torch.int16), pool_o.view(torch.int16))
    assert torch.equal(table_d.cpu(), table_o)
    if not register:
        assert torch.equal(table_o, table)
    # the grid bound of the reference: with max_len_in_batch = 256 only the first 256 rows of a request are copied
    pool_o2, table_o2 = pool.clone(), table.clone()
    orc.kv_copy_register(B, new_len, rb, re, len_sum, kv, _i32(start_loc), cur, mem_index, pool_o2, table_o2, b_req, used, 256, register)
    pool_d2, table_d2 = pool.to(DEV), table.to(DEV)
    lsa.destindex_copy_and_register_kv(B, new_len.to(DEV), rb.to(DEV), re.to(DEV), len_sum.to(DEV), kv.to(DEV), _i32(start_loc).to(DEV),
                                       cur.to(DEV), mem_index.to(DEV), pool_d2, table_d2, b_req.to(DEV), used, 256, register)
    torch.cuda.synchronize()
    assert torch.equal(pool_d2.cpu().view(torch.int16), pool_o2.view(torch.int16))
    assert torch.equal(table_d2.cpu(), table_o2)
    assert not torch.equal(pool_o2, pool_o)


def test_migration_round_trip_feeds_decode(lsa):
    """Rows copied by the migration kernel are found again by token-indexed decode through the registered table."""
    g = torch.Generator().manual_seed(23)
    Hq, Hkv, D, n = 8, 2, 128, 500
    kv = (torch.randn(n, 2 * Hkv, D, generator=g) * 0.5).to(torch.float16)
    q = (torch.randn(1, Hq, D, generator=g) * 0.5).to(torch.float16)
    pool = torch.zeros(3000, 2 * Hkv, D, dtype=torch.float16, device=DEV)
    table = torch.full((2, 600), orc.INT32_PAD, dtype=torch.int32, device=DEV)
    mem_index = torch.randperm(3000, generator=g)[:n].to(torch.int32)
    z = lambda v: _i32([v]).to(DEV)
    lsa.destindex_copy_and_register_kv(1, z(n), z(0), z(n), torch.tensor([n], device=DEV), kv.to(DEV), z(0), z(0), mem_index.to(DEV),
                                       pool, table, z(1), 0, n, True)
    nblk = (n + 255) // 256
    mo = torch.empty(nblk, 1, Hq, D, device=DEV)
    ml = torch.empty(nblk, 1, Hq, device=DEV)
    o, lse = lsa.longserve_token_decode_attention_flash_decoding(q.to(DEV), table, z(1), z(n), mo, ml, 1, n, Hq, D, pool[:, :Hkv], pool[:, Hkv:], 256)
    torch.cuda.synchronize()
    t_cpu = torch.arange(n, dtype=torch.int32)[None]
    o_ref, l_ref = orc.decode_full(q, kv[:, :Hkv], kv[:, Hkv:], t_cpu, _i32([0]), _i32([n]))
    assert (o.cpu() - o_ref).abs().max().item() <= 2e-3
    assert torch.allclose(lse.cpu(), l_ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decoding_stage_migration_matches_oracle(lsa, dtype):
    g = torch.Generator().manual_seed(41)
    L, slots, Hkv, D, B = 4, 3000, 4, 128, 5
    kv = torch.randn(L, slots, 2 * Hkv, D, generator=g).to(dtype)
    table = torch.full((8, 1400), orc.INT32_PAD, dtype=torch.int32)
    lens = [1300, 40, 600, 1, 257]
    req = _i32([3, 7, 0, 5, 1])
    perm = torch.randperm(slots, generator=g).to(torch.int32)
    off = 0
    for b, n in enumerate(lens):
        table[int(req[b]), :n] = perm[off:off + n]
        off += n
    num = _i32([700, 0, 600, 1, 33])
    b_len = _i32(lens)
    total = int(num.sum())
    mem_state = torch.ones(slots, dtype=torch.int32)
    # sender
    buf_o, ms_o = torch.zeros(L, total, 2 * Hkv, D, dtype=dtype), mem_state.clone()
    orc.decoding_stage_migration_sender(buf_o, table, ms_o, kv, req, num, b_len)
    buf_d, ms_d = torch.zeros(L, total, 2 * Hkv, D, dtype=dtype, device=DEV), mem_state.to(DEV)
    lsa.decoding_stage_migration_sender_kernel(buf_d, table.to(DEV), ms_d, kv.to(DEV), req.to(DEV), num.to(DEV), b_len.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(buf_d.cpu().view(torch.int16), buf_o.view(torch.int16))
    assert torch.equal(ms_d.cpu(), ms_o)
    # receiver (another instance: holds len - num tokens of each request, kv_cache is a strided view with spare slots)
    pool_o = torch.randn(L, 2500, 2 * Hkv, D, generator=g).to(dtype)
    table_o = torch.full((8, 1400), orc.INT32_PAD, dtype=torch.int32)
    alloc = torch.randperm(2500, generator=g)[:total].to(torch.int32)
    held = b_len - num
    pool_d, table_d = pool_o.to(DEV), table_o.to(DEV)
    orc.decoding_stage_migration_receiver(buf_o, table_o, pool_o, alloc, req, num, held)
    lsa.decoding_stage_migration_receiver_kernel(buf_d, table_d, pool_d, alloc.to(DEV), req.to(DEV), num.to(DEV), held.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(pool_d.cpu().view(torch.int16), pool_o.view(torch.int16))
    assert torch.equal(table_d.cpu(), table_o)


def test_striped_ring_with_scale_down_then_decode(lsa):
    """The elastic flow end to end: a striped prefill over P = 3 logical instances; rank r keeps, while the chunks pass
    by, the rows of its window of global token positions (here rank 0 keeps [0, cut) and rank 1 the rest, rank 2 nothing);
    afterwards a decode token attends to both kept parts through the multi-instance merge.  Prefill rows and the decode
    result are compared with dense attention over the whole sequence."""
    from loongserve_amd.simulate import DecodeInstance, KVChunk, multi_instance_decode, ring_prefill_with_migration
    g = torch.Generator().manual_seed(31)
    P, N, Hq, Hkv, D = 3, 1000, 8, 2, 128
    cut = 617
    q = (torch.randn(N, Hq, D, generator=g) * 0.5).half()
    kv = (torch.randn(N, 2 * Hkv, D, generator=g) * 0.5).half()
    m1 = meta([N])
    o_ref, _ = orc.attn_step(q, kv[:, :Hkv], kv[:, Hkv:], *m1, *m1, 1)
    chunks = []
    for j in range(P):
        kj = kv[j::P].contiguous()
        st, ln, fr = meta([kj.shape[0]], [j])
        chunks.append(KVChunk(kj.to(DEV), st.to(DEV), ln.to(DEV), fr.to(DEV)))
    windows = [(0, cut), (cut, N), (N, N)]
    kept = []
    for r in range(P):
        qi = q[r::P].contiguous().to(DEV)
        qs, ql, qf = [t.to(DEV) for t in meta([qi.shape[0]], [r])]
        order = [(r - i) % P for i in range(P)]
        pool = torch.zeros(2000, 2 * Hkv, D, dtype=torch.float16, device=DEV)
        table = torch.full((2, N + 8), orc.INT32_PAD, dtype=torch.int32, device=DEV)
        mem_index = torch.randperm(2000, generator=g)[:N].to(torch.int32).to(DEV)
        b, e = windows[r]
        o, _, _, n_kept = ring_prefill_with_migration(qi, [chunks[i] for i in order], qs, ql, qf, P, qi.shape[0], Hkv,
                                                      _i32([b]).to(DEV), _i32([e]).to(DEV), mem_index, pool, table,
                                                      _i32([1]).to(DEV))
        torch.cuda.synchronize()
        assert (o.float().cpu() - o_ref[r::P]).abs().max().item() <= 2e-3
        assert int(n_kept[0]) == e - b
        # the kept rows are the window's tokens, stripe by stripe in the order the chunks passed by
        want = torch.cat([torch.arange(j, N, P)[(torch.arange(j, N, P) >= b) & (torch.arange(j, N, P) < e)] for j in order])
        slots = table[1, :e - b].long()
        assert torch.equal(pool[slots].cpu(), kv[want])
        assert bool((table[1, e - b:] == orc.INT32_PAD).all())
        kept.append((pool, table, e - b))
    # one decode token: instance 0 is the master, instance 1 a peer, instance 2 holds nothing
    qd = (torch.randn(1, Hq, D, generator=g) * 0.5).half()
    insts = [DecodeInstance(p, t, _i32([1]).to(DEV), _i32([n]).to(DEV), max(n, 1)) for p, t, n in kept]
    o, lse = multi_instance_decode(qd.to(DEV), insts, Hkv)
    torch.cuda.synchronize()
    t_cpu = torch.arange(N, dtype=torch.int32)[None]
    o_d, l_d = orc.decode_full(qd, kv[:, :Hkv], kv[:, Hkv:], t_cpu, _i32([0]), _i32([N]))
    assert (o.float().cpu() - o_d).abs().max().item() <= 2e-3
    assert torch.allclose(lse.cpu(), l_d, rtol=1e-4, atol=1e-4)


def test_decoding_stage_migration_keeps_the_attention_result(lsa):
    """Scale-out during decoding (longserve_model.py:588-619): instance A hands the last tokens of some requests to
    instance B; attention over A's remaining tokens merged with B's received ones equals attention over what A held
    before, and the slots A gave up are free again."""
    from loongserve_amd.simulate import DecodeInstance, multi_instance_decode
    g = torch.Generator().manual_seed(43)
    Hq, Hkv, D, B = 8, 2, 128, 3
    lens, moved = [900, 300, 64], [400, 0, 64]
    mm_a = lsa.LongServeMemoryManager(3000, torch.float16, Hkv, D, 1)
    mm_b = lsa.LongServeMemoryManager(2000, torch.float16, Hkv, D, 1)
    rm_a, rm_b = lsa.LongServeReqManager(4, 1024, mm_a), lsa.LongServeReqManager(4, 1024, mm_b)
    mm_a.kv_buffer.copy_((torch.randn(mm_a.kv_buffer.shape, generator=g) * 0.5).half())
    rows = _i32([2, 0, 3]).to(DEV)
    b_len = _i32(lens).to(DEV)
    slots_a = mm_a.alloc(sum(lens))
    lsa.init_req_to_token_indexes(rm_a.req_to_token_indexs, rows, b_len, slots_a)
    q = (torch.randn(B, Hq, D, generator=g) * 0.5).half().to(DEV)
    before, lse_before = multi_instance_decode(q, [DecodeInstance(mm_a.kv_buffer[0], rm_a.req_to_token_indexs, rows, b_len, max(lens))], Hkv)
    before, lse_before = before.clone(), lse_before.clone()
    # A sends, B receives into freshly allocated slots of its own pool
    num = _i32(moved).to(DEV)
    total = sum(moved)
    buf = torch.empty(1, total, 2 * Hkv, D, dtype=torch.float16, device=DEV)
    free_before = mm_a.can_use_mem_size
    lsa.decoding_stage_migration_sender_kernel(buf, rm_a.req_to_token_indexs, mm_a.mem_state, mm_a.kv_buffer, rows, num, b_len)
    mm_a.can_use_mem_size += total                         # the sender kernel cleared the reference counts of what it sent
    assert int((mm_a.mem_state == 0).sum()) == mm_a.can_use_mem_size == free_before + total
    slots_b = mm_b.alloc(total)
    held_b = torch.zeros(B, dtype=torch.int32, device=DEV)
    lsa.decoding_stage_migration_receiver_kernel(buf, rm_b.req_to_token_indexs, mm_b.kv_buffer, slots_b, rows, num, held_b)  # int64 slots, as alloc returns them
    len_a, len_b = b_len - num, num
    after, lse_after = multi_instance_decode(q, [
        DecodeInstance(mm_a.kv_buffer[0], rm_a.req_to_token_indexs, rows, len_a, max(lens)),
        DecodeInstance(mm_b.kv_buffer[0], rm_b.req_to_token_indexs, rows, len_b, max(max(moved), 1))], Hkv)
    torch.cuda.synchronize()
    assert (after.float() - before.float()).abs().max().item() <= 2e-3
    assert torch.allclose(lse_after, lse_before, rtol=1e-4, atol=1e-4)

"""Pins for the CPU oracle (oracle/attn_oracle.py).

The reference holds no golden vectors for this path and its only prefill self-test is
stale, so every oracle function is checked here against something it was NOT written
from: a library routine, a brute-force float64 loop, a closed-form special case or an
algebraic invariant.  A dropped term, a wrong sign, a transposed operand or an off-by-one
in the mask fails at least one of these.
"""
import math

import pytest
import torch

from oracle import attn_oracle as orc


def _meta(lens, firsts=None):
    lens = torch.tensor(lens, dtype=torch.int32)
    start = (torch.cumsum(lens, 0) - lens).to(torch.int32)
    firsts = torch.zeros_like(lens) if firsts is None else torch.tensor(firsts, dtype=torch.int32)
    return start, lens, firsts


def _rand(shape, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 0.5).to(dtype)


def brute_force_step(q, k, v, qs, ql, qf, ks, kl, kf, P):
    """float64 loops, written from the definition: key n visible to row m iff
    kf + n*P <= qf + m*P; softmax over visible keys of q.k/sqrt(D)."""
    Tq, Hq, D = q.shape
    Hkv = k.shape[1]
    O = [[[0.0] * D for _ in range(Hq)] for _ in range(Tq)]
    LSE = [[-math.inf] * Hq for _ in range(Tq)]
    for b in range(len(ql)):
        for m in range(int(ql[b])):
            for h in range(Hq):
                hk = h // (Hq // Hkv)
                sc = []
                for n in range(int(kl[b])):
                    if int(kf[b]) + n * P <= int(qf[b]) + m * P:
                        dot = sum(float(q[int(qs[b]) + m, h, d]) * float(k[int(ks[b]) + n, hk, d]) for d in range(D))
                        sc.append((n, dot / math.sqrt(D)))
                if not sc:
                    continue
                mx = max(s for _, s in sc)
                den = sum(math.exp(s - mx) for _, s in sc)
                LSE[int(qs[b]) + m][h] = mx + math.log(den)
                for n, s in sc:
                    w = math.exp(s - mx) / den
                    for d in range(D):
                        O[int(qs[b]) + m][h][d] += w * float(v[int(ks[b]) + n, hk, d])
    return torch.tensor(O, dtype=torch.float64), torch.tensor(LSE, dtype=torch.float64)


@pytest.mark.parametrize("P,qf,kf", [(1, [0, 0], [0, 0]), (1, [7, 3], [2, 0]), (3, [1, 2], [2, 0]), (4, [0, 3], [3, 1])])
def test_attn_step_vs_brute_force(P, qf, kf):
    Hq, Hkv, D = 4, 2, 8
    qs, ql, qf_t = _meta([5, 3], qf)
    ks, kl, kf_t = _meta([7, 4], kf)
    q, k, v = _rand((8, Hq, D), 1), _rand((11, Hkv, D), 2), _rand((11, Hkv, D), 3)
    O, LSE = orc.attn_step(q, k, v, qs, ql, qf_t, ks, kl, kf_t, P, dtype=torch.float64)
    Ob, Lb = brute_force_step(q, k, v, qs, ql, qf_t, ks, kl, kf_t, P)
    assert torch.allclose(O, Ob, atol=1e-12)
    assert torch.equal(torch.isinf(LSE), torch.isinf(Lb))
    fin = ~torch.isinf(Lb)
    assert torch.allclose(LSE[fin], Lb[fin], atol=1e-12)
    # rows that see nothing: O = 0, LSE = -inf
    assert torch.all(O[~fin] == 0)


def test_attn_step_vs_library_sdpa_causal():
    T, H, D = 193, 6, 64
    q, k, v = _rand((T, H, D), 4), _rand((T, 2, D), 5), _rand((T, 2, D), 6)
    s, l, f = _meta([T])
    O, LSE = orc.attn_step(q, k, v, s, l, f, s, l, f, 1)
    kk = k.float().repeat_interleave(3, dim=1).permute(1, 0, 2)
    vv = v.float().repeat_interleave(3, dim=1).permute(1, 0, 2)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float().permute(1, 0, 2)[None], kk[None], vv[None],
                                                           is_causal=True)[0].permute(1, 0, 2)
    assert torch.allclose(O, ref, atol=2e-6, rtol=1e-5)
    sc = torch.einsum("thd,shd->hts", q.float(), kk.permute(1, 0, 2)) / math.sqrt(D)
    sc = sc.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(LSE, torch.logsumexp(sc, -1).permute(1, 0), atol=1e-5)


def test_special_cases_single_key_zero_q_constant_v():
    H, D = 2, 16
    s1, l1, f1 = _meta([1])
    q, k, v = _rand((1, H, D), 7), _rand((1, H, D), 8), _rand((1, H, D), 9)
    O, LSE = orc.attn_step(q, k, v, s1, l1, f1, s1, l1, f1, 1)
    assert torch.allclose(O, v.float(), atol=1e-7)                      # single visible key: O = V
    assert torch.allclose(LSE[0], (q.float() * k.float()).sum(-1)[0] / math.sqrt(D), atol=1e-6)
    T = 9
    s, l, f = _meta([T])
    k, v = _rand((T, H, D), 10), _rand((T, H, D), 11)
    O, LSE = orc.attn_step(torch.zeros(T, H, D, dtype=torch.float16), k, v, s, l, f, s, l, f, 1)
    cm = torch.cumsum(v.float(), 0) / torch.arange(1, T + 1)[:, None, None]
    assert torch.allclose(O, cm, atol=1e-6)                             # q = 0: running mean of V
    assert torch.allclose(LSE, torch.log(torch.arange(1, T + 1).float())[:, None].expand(T, H), atol=1e-6)
    vc = torch.full((T, H, D), 0.25, dtype=torch.float16)
    O, _ = orc.attn_step(_rand((T, H, D), 12), k, vc, s, l, f, s, l, f, 1)
    assert torch.allclose(O, vc.float(), atol=1e-6)                     # constant V: O = V


def _shard_contiguous(k, v, lens, nshard, rng):
    """Random contiguous partition of each sequence over nshard nodes (the recipe of the
    reference's own self-test, ring_context_flashattention_nopad.py:354-371)."""
    B = len(lens)
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    cuts = []
    for b in range(B):
        c = sorted(int(x) for x in torch.randint(0, lens[b] + 1, (nshard - 1,), generator=rng))
        cuts.append([0] + c + [lens[b]])
    shards = []
    for j in range(nshard):
        ks, vs, sl, fi = [], [], [], []
        for b in range(B):
            a, e = cuts[b][j], cuts[b][j + 1]
            ks.append(k[starts[b] + a:starts[b] + e])
            vs.append(v[starts[b] + a:starts[b] + e])
            sl.append(e - a)
            fi.append(a)
        st, ln, fr = _meta(sl, fi)
        shards.append((torch.cat(ks), torch.cat(vs), st, ln, fr))
    return shards


def test_ring_equals_monolithic_reference_recipe():
    # B=2, Hq=40, Hkv=4, D=128, KV contiguously partitioned over 8 nodes: RING:324-371
    g = torch.Generator().manual_seed(0)
    lens = [int(x) for x in torch.randint(1, 300, (2,), generator=g)]
    T, Hq, Hkv, D = sum(lens), 40, 4, 128
    q, k, v = _rand((T, Hq, D), 20), _rand((T, Hkv, D), 21), _rand((T, Hkv, D), 22)
    s, l, f = _meta(lens)
    O_full, LSE_full = orc.attn_step(q, k, v, s, l, f, s, l, f, 1)
    shards = _shard_contiguous(k, v, lens, 8, g)
    parts = [orc.attn_step(q, ks, vs, s, l, f, st, ln, fr, 1) for ks, vs, st, ln, fr in shards]
    O, LSE = orc.lse_merge(parts)
    assert torch.allclose(O, O_full, atol=2e-6)
    assert torch.allclose(LSE, LSE_full, atol=2e-6)
    # step order does not matter (commutativity / associativity of the LSE merge)
    O2, LSE2 = orc.lse_merge(parts[::-1])
    assert torch.allclose(O2, O, atol=2e-6) and torch.allclose(LSE2, LSE, atol=2e-6)
    # in-place (o, m, l) state of the reference operator gives the same answer
    o = torch.zeros(T, Hq, D, dtype=torch.float32)
    m = torch.full((T, Hq), float("-inf"))
    ll = torch.zeros(T, Hq)
    for ks, vs, st, ln, fr in shards:
        orc.context_attention_fwd(q, ks, vs, o, s, l, f, st, ln, fr, 1, max(lens), m, ll)
    assert torch.allclose(o, O_full, atol=3e-6)
    assert torch.allclose(orc.state_lse(m, ll).float(), LSE_full, atol=1e-5)


def test_striped_equals_contiguous():
    T, H, D, P = 37, 2, 16, 4
    q, k, v = _rand((T, H, D), 30), _rand((T, H, D), 31), _rand((T, H, D), 32)
    s, l, f = _meta([T])
    O_full, LSE_full = orc.attn_step(q, k, v, s, l, f, s, l, f, 1)
    O = torch.zeros_like(O_full)
    LSE = torch.zeros_like(LSE_full)
    for r in range(P):  # rank r owns tokens r, r+P, ... (loongserve/longserve_server/io_struct.py:78-81)
        qi = q[r::P]
        qs_, ql_, qf_ = _meta([qi.shape[0]], [r])
        parts = []
        for j in range(P):
            kj, vj = k[j::P], v[j::P]
            ks_, kl_, kf_ = _meta([kj.shape[0]], [j])
            parts.append(orc.attn_step(qi, kj, vj, qs_, ql_, qf_, ks_, kl_, kf_, P))
        o_r, l_r = orc.lse_merge(parts)
        O[r::P], LSE[r::P] = o_r, l_r
    assert torch.allclose(O, O_full, atol=2e-6)
    assert torch.allclose(LSE, LSE_full, atol=2e-6)


def test_merge_with_empty_partial_is_identity():
    O = _rand((5, 2, 8), 40, torch.float32)
    L = _rand((5, 2), 41, torch.float32)
    e = (torch.zeros_like(O), torch.full_like(L, float("-inf")))
    O2, L2 = orc.lse_merge([(O, L), e])
    assert torch.allclose(O2, O) and torch.allclose(L2, L)
    O3, L3 = orc.lse_merge([e, e])
    assert torch.all(O3 == 0) and torch.all(torch.isinf(L3))


def _decode_case(seed, B, Hq, Hkv, D, lens, pool):
    g = torch.Generator().manual_seed(seed)
    q = _rand((B, Hq, D), seed + 1)
    kv = _rand((pool, 2 * Hkv, D), seed + 2)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    max_seq = max(max(lens), 1) + 3
    table = torch.full((B + 2, max_seq), orc.INT32_PAD, dtype=torch.int32)
    b_req = torch.randperm(B + 2, generator=g)[:B].to(torch.int32)
    off = 0
    for b in range(B):
        table[int(b_req[b]), :lens[b]] = perm[off:off + lens[b]]
        off += lens[b]
    return q, kv, table, b_req, torch.tensor(lens, dtype=torch.int32)


@pytest.mark.parametrize("BS", [1, 16, 64, 256])
def test_decode_stage1_stage2_vs_dense(BS):
    B, Hq, Hkv, D = 3, 8, 2, 128
    lens = [300, 1, 77]
    q, kv, table, b_req, b_len = _decode_case(50, B, Hq, Hkv, D, lens, 500)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    nblk = (max(lens) + BS - 1) // BS
    mid_o = torch.full((nblk, B, Hq, D), float("nan"))
    mid_l = torch.full((nblk, B, Hq), float("nan"))
    o = torch.empty(B, Hq, D)
    lse = torch.empty(B, Hq)
    orc.decode_stage1(q, k, v, table, b_req, b_len, max(lens), mid_o, mid_l, BS)
    orc.decode_stage2(mid_o, mid_l, b_len, o, lse, BS)
    # independent dense computation with torch.softmax on explicitly gathered rows
    for b in range(B):
        rows = table[int(b_req[b]), :lens[b]].long()
        kk = k[rows].float().repeat_interleave(Hq // Hkv, 1)
        vv = v[rows].float().repeat_interleave(Hq // Hkv, 1)
        s = torch.einsum("hd,nhd->hn", q[b].float(), kk) / math.sqrt(D)
        ref = torch.einsum("hn,nhd->hd", torch.softmax(s, -1), vv)
        assert torch.allclose(o[b], ref, atol=2e-6)
        assert torch.allclose(lse[b], torch.logsumexp(s, -1), atol=1e-5)
    of, lf = orc.decode_full(q, k, v, table, b_req, b_len)
    assert torch.allclose(of, o, atol=2e-6) and torch.allclose(lf, lse, atol=1e-5)


def test_decode_gather_is_bit_exact_identity_code():
    # q = 0 and V rows that encode their own slot number: O * len is the sum of the
    # gathered slot ids, and the gathered rows themselves compare bit-for-bit
    B, H, D = 2, 1, 128
    lens = [5, 9]
    q, kv, table, b_req, b_len = _decode_case(60, B, H, H, D, lens, 64)
    q.zero_()
    kv[:, H:, :] = torch.arange(64, dtype=torch.float16)[:, None, None]
    k, v = kv[:, :H], kv[:, H:]
    o, lse = orc.decode_full(q, k, v, table, b_req, b_len)
    for b in range(B):
        slots = table[int(b_req[b]), :lens[b]].long()
        assert torch.equal(orc.gather_rows(v, table, int(b_req[b]), 0, lens[b]), v[slots])
        assert abs(float(o[b, 0, 0]) * lens[b] - float(slots.sum())) < 1e-3
        assert abs(float(lse[b, 0]) - math.log(lens[b])) < 1e-6


def test_decode_empty_request_and_merge_trick():
    # a peer that holds nothing for a request contributes (0, -inf); block_seq=1 stage 2 merges
    # instance partials and split-K blocks alike (longserve_model.py:514-516, stage2.cu:30)
    B, Hq, Hkv, D = 2, 4, 4, 128
    lens = [40, 25]
    q, kv, table, b_req, b_len = _decode_case(70, B, Hq, Hkv, D, lens, 100)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    full_o, full_l = orc.decode_full(q, k, v, table, b_req, b_len)
    # split each request: peer holds the first part (request 1: nothing), master the rest
    cut = [13, 0]
    t_peer = torch.full_like(table, orc.INT32_PAD)
    t_master = torch.full_like(table, orc.INT32_PAD)
    for b in range(B):
        r = int(b_req[b])
        t_peer[r, :cut[b]] = table[r, :cut[b]]
        t_master[r, :lens[b] - cut[b]] = table[r, cut[b]:lens[b]]
    peer_len = torch.tensor(cut, dtype=torch.int32)
    master_len = torch.tensor([lens[b] - cut[b] for b in range(B)], dtype=torch.int32)
    BS, P = 16, 2
    nblk = (int(master_len.max()) + BS - 1) // BS
    gm = torch.full((P - 1 + nblk, B, Hq, D), float("nan"))
    gl = torch.full((P - 1 + nblk, B, Hq), float("nan"))
    pm = torch.empty(int(peer_len.max()) // BS + 1, B, Hq, D)
    pl = torch.empty(int(peer_len.max()) // BS + 1, B, Hq)
    po, plse = orc.token_decode_attention_flash_decoding(q, t_peer, b_req, peer_len, pm, pl, B, int(peer_len.max()),
                                                         Hq, D, k, v, BS)
    assert torch.all(po[1] == 0) and torch.all(torch.isinf(plse[1]))
    gm[0], gl[0] = po, plse
    orc.decode_stage1(q, k, v, t_master, b_req, master_len, int(master_len.max()), gm[P - 1:], gl[P - 1:], BS)
    merge_len = ((P - 1) + (master_len + BS - 1) // BS).to(torch.int32)
    o = torch.empty(B, Hq, D)
    lse = torch.empty(B, Hq)
    orc.decode_stage2(gm, gl, merge_len, o, lse, 1)
    assert torch.allclose(o, full_o, atol=2e-6) and torch.allclose(lse, full_l, atol=1e-5)


def test_kv_scatter_and_register():
    src = _rand((6, 4, 8), 80)
    pool = torch.zeros(10, 4, 8, dtype=torch.float16)
    dest = torch.tensor([7, 2, 9, 0, 4, 5], dtype=torch.int32)
    orc.kv_scatter(src, dest, pool)
    for i in range(6):
        assert torch.equal(pool[int(dest[i])], src[i])
    assert torch.all(pool[[1, 3, 6, 8]] == 0)
    table = torch.full((4, 5), orc.INT32_PAD, dtype=torch.int32)
    orc.register_tokens(table, torch.tensor([2, 0]), torch.tensor([0, 4]), torch.tensor([4, 2]), dest)
    assert table[2].tolist() == [7, 2, 9, 0, orc.INT32_PAD]
    assert table[0].tolist() == [4, 5] + [orc.INT32_PAD] * 3
    assert torch.all(table[[1, 3]] == orc.INT32_PAD)
    # the decode-stage registration: known answer, and the same as a numpy fancy-index assignment
    orc.copy_kv_index_to_req(table, torch.tensor([0, 3]), torch.tensor([3, 1]), torch.tensor([11, 12]))
    assert table[0].tolist() == [4, 5, 11] + [orc.INT32_PAD] * 2 and table[3].tolist() == [12] + [orc.INT32_PAD] * 4
    import numpy as np
    rng = np.random.default_rng(3)
    t1 = torch.full((9, 20), orc.INT32_PAD, dtype=torch.int32)
    t2 = t1.numpy().copy()
    req, ln, mem = rng.permutation(9)[:6], rng.integers(1, 21, 6), rng.integers(0, 1000, 6)
    orc.copy_kv_index_to_req(t1, torch.from_numpy(req), torch.from_numpy(ln), torch.from_numpy(mem))
    t2[req, ln - 1] = mem
    assert (t1.numpy() == t2).all()


def test_kv_ranges_count_the_locally_held_tokens_of_the_window():
    """Pin by brute force: local row n holds global token first + n * P, so [range_begin, range_end) must be exactly
    the rows whose global index falls in [index_begin, index_end) (for windows that start at or after `first`)."""
    import random
    rnd = random.Random(5)
    for _ in range(300):
        P = rnd.randint(1, 6)
        first = rnd.randint(0, 7)
        n_rows = rnd.randint(0, 40)
        begin = first + rnd.randint(0, 60)
        end = begin + rnd.randint(0, 80)
        rb, re, nl = orc.kv_ranges([begin], [end], [first], P)
        rows = [n for n in range(0, 400) if begin <= first + n * P < end]
        assert int(nl[0]) == len(rows)
        if rows:
            assert (int(rb[0]), int(re[0])) == (rows[0], rows[-1] + 1)
    # a window that starts before the first held token: the Python floor form goes negative and the copy skips the request
    rb, re, nl = orc.kv_ranges([0], [3], [9], 4)
    assert int(rb[0]) == -2 and int(re[0]) == -1 and int(nl[0]) == 1


def test_kv_copy_register_against_index_copy():
    g = torch.Generator().manual_seed(11)
    B, rows, pool_n, W = 4, 60, 200, 24
    kv = torch.randn(rows, 3, 8, generator=g).to(torch.float16)
    pool = torch.zeros(pool_n, 3, 8, dtype=torch.float16)
    table = torch.full((6, 50), orc.INT32_PAD, dtype=torch.int32)
    new_len = torch.tensor([5, 0, 7, 3], dtype=torch.int32)
    begin = torch.tensor([2, 4, 0, 1], dtype=torch.int32)
    end = begin + new_len
    len_sum = torch.cumsum(new_len, 0, dtype=torch.int64)
    start_loc = torch.tensor([0, 10, 20, 40], dtype=torch.int32)
    cur = torch.tensor([3, 0, 9, 1], dtype=torch.int32)
    b_req = torch.tensor([5, 1, 0, 2], dtype=torch.int32)
    used = 4
    mem_index = torch.randperm(pool_n, generator=g)[:used + int(len_sum[-1])].to(torch.int32)
    orc.kv_copy_register(B, new_len, begin, end, len_sum, kv, start_loc, cur, mem_index, pool, table, b_req, used, 16, True)
    # the same through index_copy_ on explicitly built row / slot lists
    src_rows, slots = [], []
    for b in range(B):
        off = used + (int(len_sum[b - 1]) if b else 0)
        for n in range(int(new_len[b])):
            src_rows.append(int(start_loc[b]) + int(begin[b]) + n)
            slots.append(int(mem_index[off + n]))
            assert int(table[int(b_req[b]), int(cur[b]) + n]) == slots[-1]
    want = torch.zeros_like(pool).index_copy_(0, torch.tensor(slots), kv[src_rows])
    assert torch.equal(pool, want)
    assert int((table != orc.INT32_PAD).sum()) == len(slots)
    # negative bound: request skipped; row limit: rows past ceil(max_len/256)*256 are not copied
    pool2 = torch.zeros_like(pool)
    orc.kv_copy_register(1, torch.tensor([3], dtype=torch.int32), torch.tensor([-1], dtype=torch.int32), torch.tensor([2], dtype=torch.int32),
                         torch.tensor([3]), kv, torch.tensor([5], dtype=torch.int32), cur, mem_index, pool2, table.clone(), b_req, 0, 16, False)
    assert int(pool2.abs().sum()) == 0


def _ulp_diff_f16(a, b):
    """Distance in fp16 representable steps between two float16 arrays (monotone integer mapping)."""
    import numpy as np
    def key(v):
        i = v.view(np.int16).astype(np.int32)
        return np.where(i < 0, -32768 - i, i)
    return np.abs(key(a) - key(b))


def test_elementwise_oracle_against_float64_formulas():
    import numpy as np
    from oracle import elementwise_oracle as ew
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((7, 512)) * 2).astype(np.float16)
    w = (1 + 0.1 * rng.standard_normal(512)).astype(np.float16)
    want = torch.from_numpy(x.astype(np.float64)) * torch.from_numpy(w.astype(np.float64)) / torch.sqrt(
        (torch.from_numpy(x.astype(np.float64)) ** 2).mean(dim=1, keepdim=True) + 1e-5)
    got = ew.rms_norm(x, w, 1e-5)
    assert _ulp_diff_f16(got, want.numpy().astype(np.float16)).max() <= 1  # fp32 product order vs float64
    io = (rng.standard_normal((5, 256)) * 3).astype(np.float16)
    ref = io.copy()
    ew.silu_and_mul_inplace(io)
    g, u = torch.from_numpy(ref[:, :128].astype(np.float64)), torch.from_numpy(ref[:, 128:].astype(np.float64))
    want = (g * torch.sigmoid(g) * u).numpy()
    assert np.array_equal(io[:, 128:], ref[:, 128:])                      # second half untouched
    assert np.abs(io[:, :128].astype(np.float64) - want).max() <= 2 ** -10 * np.abs(want).max() * 2  # two half roundings
    assert _ulp_diff_f16(io[:, :128], want.astype(np.float16)).max() <= 1


def test_rotary_oracle_is_a_rotation_and_rounds_once():
    import numpy as np
    from fractions import Fraction
    from oracle import elementwise_oracle as ew
    rng = np.random.default_rng(4)
    T, H, D = 6, 3, 32
    x = rng.standard_normal((T, H, D)).astype(np.float16)
    ang = rng.uniform(0, 6.28, (T, D // 2))
    cos, sin = np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)
    y = x.copy()
    ew.rotary_emb(y, cos, sin)
    # complex multiplication (x1 + i x2)(cos + i sin) in float64, within the half roundings
    z = (x[..., :D // 2].astype(np.float64) + 1j * x[..., D // 2:].astype(np.float64)) * (cos + 1j * sin.astype(np.float64))[:, None, :]
    assert np.abs(y[..., :D // 2] - z.real).max() <= 4e-3 and np.abs(y[..., D // 2:] - z.imag).max() <= 4e-3
    # norm preservation (cos^2 + sin^2 = 1 up to the rounding of the tables)
    n0 = (x.astype(np.float64) ** 2).sum(-1); n1 = (y.astype(np.float64) ** 2).sum(-1)
    assert np.abs(n1 / n0 - 1).max() < 5e-3
    # exact rational arithmetic: t = round_half(x2*sin); x1' = round_half(x1*cos - t), each rounded exactly once
    def rh(fr):  # nearest-even rounding of a Fraction to float16 through exact comparison
        f = np.float16(float(fr))
        cands = [f, np.nextafter(f, np.float16(np.inf)), np.nextafter(f, np.float16(-np.inf))]
        best = min(cands, key=lambda c: (abs(Fraction(float(c)) - fr), int(np.float16(c).view(np.int16)) & 1))
        return np.float16(best)
    for (t, h, i) in [(0, 0, 0), (1, 2, 5), (5, 1, 15), (3, 0, 9)]:
        x1, x2 = Fraction(float(x[t, h, i])), Fraction(float(x[t, h, D // 2 + i]))
        c, s = Fraction(float(cos[t, i])), Fraction(float(sin[t, i]))
        assert y[t, h, i] == rh(x1 * c - Fraction(float(rh(x2 * s))))
        assert y[t, h, D // 2 + i] == rh(x1 * s + Fraction(float(rh(x2 * c))))


def test_decoding_stage_migration_oracle_round_trip():
    """Pin by invariant: send then receive on another instance reproduces, slot for slot, the tail of every request
    (torch.index_select is the independent routine), the sender frees exactly those slots and the receiver's table is
    extended by exactly the new slots."""
    g = torch.Generator().manual_seed(8)
    L, slots, W, B = 3, 90, 6, 4
    kv_a = torch.randn(L, slots, 2, W, generator=g).to(torch.float16)
    table_a = torch.full((6, 40), orc.INT32_PAD, dtype=torch.int32)
    lens = [20, 7, 33, 1]
    req = torch.tensor([4, 0, 2, 5], dtype=torch.int32)
    perm = torch.randperm(slots, generator=g).to(torch.int32)
    off = 0
    for b, n in enumerate(lens):
        table_a[int(req[b]), :n] = perm[off:off + n]
        off += n
    mem_state = torch.ones(slots, dtype=torch.int32)
    num = torch.tensor([5, 0, 33, 1], dtype=torch.int32)
    b_len = torch.tensor(lens, dtype=torch.int32)
    buf = torch.zeros(L, int(num.sum()), 2, W, dtype=torch.float16)
    orc.decoding_stage_migration_sender(buf, table_a, mem_state, kv_a, req, num, b_len)
    want_slots = torch.cat([table_a[int(req[b]), lens[b] - int(num[b]):lens[b]] for b in range(B)]).long()
    assert torch.equal(buf, kv_a.index_select(1, want_slots))
    freed = torch.zeros(slots, dtype=torch.bool); freed[want_slots] = True
    assert torch.equal(mem_state == 0, freed)
    # receiver on an instance that holds the first (len - num) tokens of each request
    kv_b = torch.zeros(L, 70, 2, W, dtype=torch.float16)
    table_b = torch.full((6, 40), orc.INT32_PAD, dtype=torch.int32)
    alloc = torch.randperm(70, generator=g)[:int(num.sum())].to(torch.int32)
    held = b_len - num
    orc.decoding_stage_migration_receiver(buf, table_b, kv_b, alloc, req, num, held)
    assert torch.equal(kv_b.index_select(1, alloc.long()), buf)
    o = 0
    for b in range(B):
        n = int(num[b])
        assert torch.equal(table_b[int(req[b]), int(held[b]):int(held[b]) + n], alloc[o:o + n])
        o += n
    assert int((table_b != orc.INT32_PAD).sum()) == int(num.sum())


# --------------------------------------------------------------------------------------------------------------
# KV-pool slot allocator oracle: pinned by slot-by-slot scans written without nonzero / slicing
# --------------------------------------------------------------------------------------------------------------
def _scan_first_free(state, need):
    out = []
    for p, s in enumerate(state):
        if len(out) == need:
            break
        if s == 0:
            out.append(p)
    return out


def _scan_first_fit(state, need):
    run = 0
    for p, s in enumerate(state):
        run = run + 1 if s == 0 else 0
        if run == need:
            return p - need + 1
    return None


def test_pool_oracle_searches_against_slot_scans():
    import numpy as np
    from oracle.pool_oracle import MemoryManagerOracle
    rng = np.random.default_rng(5)
    for trial in range(60):
        size = int(rng.integers(1, 300))
        m = MemoryManagerOracle(size)
        busy = rng.random(size) < rng.choice([0.05, 0.3, 0.7])
        m.add_refs(np.nonzero(busy)[0])
        assert m.can_use_mem_size == int((m.mem_state == 0).sum())
        before = m.mem_state.copy()
        need = int(rng.integers(1, 12))
        want = _scan_first_fit(before, need)
        got = m.alloc_contiguous(need)
        if want is None:
            assert got is None and (m.mem_state == before).all()
        else:
            idx, start, end = got
            assert (start, end) == (want, want + need) and idx.tolist() == list(range(want, want + need))
            assert (m.mem_state[start:end] == 1).all()
        assert m.can_use_mem_size == int((m.mem_state == 0).sum())
        before = m.mem_state.copy()
        need = int(rng.integers(0, m.can_use_mem_size + 1))
        got = m.alloc(need)
        assert got.tolist() == _scan_first_free(before, need)
        assert (m.mem_state[got] == 1).all() and m.can_use_mem_size == int((m.mem_state == 0).sum())
    # a run that ends exactly at the last slot, and one slot short of fitting
    m = MemoryManagerOracle(10)
    m.add_refs(np.array([0, 1, 2, 3, 4, 5]))
    assert m.alloc_contiguous(5) is None
    assert m.alloc_contiguous(4)[1:] == (6, 10)
    with pytest.raises(AssertionError):
        MemoryManagerOracle(4).alloc(5)


def test_pool_oracle_reference_counts_and_duplicates():
    import numpy as np
    from oracle.pool_oracle import MemoryManagerOracle
    m = MemoryManagerOracle(8)
    m.add_refs(np.array([1, 1, 3]))           # slot 1 listed twice: gains one reference, but both entries count as new
    assert m.mem_state.tolist() == [0, 1, 0, 1, 0, 0, 0, 0] and m.can_use_mem_size == 8 - 3
    m.add_refs(np.array([1, 2]))              # slot 1 is shared now
    assert m.mem_state.tolist() == [0, 2, 1, 1, 0, 0, 0, 0] and m.can_use_mem_size == 8 - 3 - 1
    m.free(np.array([1, 2], dtype=np.int32))  # slot 1 keeps one reference, slot 2 becomes free
    assert m.mem_state.tolist() == [0, 1, 0, 1, 0, 0, 0, 0] and m.can_use_mem_size == 8 - 3
    m.free_all()
    assert m.can_use_mem_size == 8 and not m.mem_state.any()
    # a random trace without duplicates keeps the conservation law
    rng = np.random.default_rng(11)
    m = MemoryManagerOracle(200)
    held = []
    for step in range(200):
        if held and rng.random() < 0.45:
            m.free(held.pop(int(rng.integers(len(held)))))
        else:
            need = int(rng.integers(1, 20))
            if need <= m.can_use_mem_size:
                got = m.alloc_contiguous(need) if rng.random() < 0.5 else None
                held.append(got[0].copy() if got is not None else m.alloc(need).copy())
        assert m.can_use_mem_size == int((m.mem_state == 0).sum())
        assert sum(len(h) for h in held) == int(m.mem_state.sum())


def test_oracle_against_the_committed_known_answers():
    """tests/golden/attention_known_answers.npz: answers computed once by float64 loops over the definition
    (tests/golden/make_fixtures.py, no oracle code); the oracle must reproduce them."""
    import os
    import numpy as np
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_known_answers.npz"))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    cum = lambda ln: torch.cumsum(t(ln), 0).to(torch.int32) - t(ln)
    o, lse = orc.attn_step(t(z["pf_q"]), t(z["pf_k"]), t(z["pf_v"]), cum(z["pf_q_len"]), t(z["pf_q_len"]), t(z["pf_q_first"]),
                           cum(z["pf_kv_len"]), t(z["pf_kv_len"]), t(z["pf_kv_first"]), int(z["pf_peers"]), dtype=torch.float64)
    assert torch.allclose(o, t(z["pf_o"]), atol=1e-12) and torch.allclose(lse, t(z["pf_lse"]), atol=1e-12)
    assert torch.equal(torch.isinf(lse), torch.isinf(t(z["pf_lse"])))
    Hkv = z["dc_pool"].shape[1] // 2
    pool = t(z["dc_pool"])
    o, lse = orc.decode_full(t(z["dc_q"]), pool[:, :Hkv], pool[:, Hkv:], t(z["dc_table"]), t(z["dc_b_req"]), t(z["dc_b_len"]),
                             dtype=torch.float64)
    assert torch.allclose(o, t(z["dc_o"]), atol=1e-12) and torch.allclose(lse, t(z["dc_lse"]), atol=1e-12)

"""GPU parity of the prefill step against the CPU oracle (through the C ABI)."""
import math

import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import assert_inplace_o_close, assert_lse_close, assert_o_close, meta, rand_t

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("prefill_geometry")]
DEV = "cuda:0"


def _dev(*ts):
    return [t.to(DEV) for t in ts]


def _run_step(lsa, q, k, v, qm, km, P, max_q):
    qd, kd, vd = _dev(q, k, v)
    qs, ql, qf = _dev(*qm)
    ks, kl, kf = _dev(*km)
    o, lse = lsa.prefill_attention_step(qd, kd, vd, qs, ql, qf, ks, kl, kf, P, max_q)
    torch.cuda.synchronize()
    return o, lse


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("lens,Hq,Hkv", [([256], 2, 2), ([1000], 4, 1), ([1, 77, 513, 300], 8, 2), ([640, 129], 10, 5)])
def test_causal_step_vs_oracle(lsa, dtype, lens, Hq, Hkv):
    print("case", dtype, lens, Hq, Hkv, flush=True)
    T, D = sum(lens), 128
    q, k, v = rand_t((T, Hq, D), 1, dtype), rand_t((T, Hkv, D), 2, dtype), rand_t((T, Hkv, D), 3, dtype)
    m = meta(lens)
    o, lse = _run_step(lsa, q, k, v, m, m, 1, max(lens))
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")


@pytest.mark.parametrize("Hq,Hkv", [(16, 16), (32, 8)])
def test_batch_of_short_prompts(lsa, Hq, Hkv):
    """24 requests of 1 to 1000 tokens: a launch of more than three workgroups per CU whose chunks are short, the kind the
    library gives the four-wave shape (two workgroups per CU) by itself; with grouped heads, four of them per workgroup."""
    lens = [300, 17, 512, 1000, 64, 700, 129, 1] * 3
    T, D = sum(lens), 128
    q, k, v = rand_t((T, Hq, D), 41), rand_t((T, Hkv, D), 42), rand_t((T, Hkv, D), 43)
    m = meta(lens)
    o, lse = _run_step(lsa, q, k, v, m, m, 1, max(lens))
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")


def test_cfg1_single_causal_2048(lsa):
    # baseline configuration 1: 1 x 2048 tokens, 32/32 heads, D=128, fp16, one step
    T, H, D = 2048, 32, 128
    q, k, v = rand_t((T, H, D), 1001), rand_t((T, H, D), 1002), rand_t((T, H, D), 1003)
    m = meta([T])
    o, lse = _run_step(lsa, q, k, v, m, m, 1, T)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "cfg1 O")
    assert_lse_close(lse, lse_ref, "cfg1 LSE")


@pytest.mark.parametrize("P,qf,kf", [(1, [300, 0], [0, 0]), (1, [100, 0], [250, 40]), (4, [1, 2], [2, 0]), (3, [0, 1], [2, 2])])
def test_offdiagonal_and_striped_steps(lsa, P, qf, kf):
    print("case", P, qf, kf, flush=True)
    Hq, Hkv, D = 4, 2, 128
    qlens, klens = [300, 131], [280, 200]
    q = rand_t((sum(qlens), Hq, D), 11)
    k, v = rand_t((sum(klens), Hkv, D), 12), rand_t((sum(klens), Hkv, D), 13)
    qm, km = meta(qlens, qf), meta(klens, kf)
    o, lse = _run_step(lsa, q, k, v, qm, km, P, max(qlens))
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")
    # rows that see nothing: exactly (0, -inf)
    empty = torch.isinf(lse_ref)
    assert torch.all(o.cpu()[empty] == 0)


def test_strided_interleaved_kv_views(lsa):
    # k and v are the two halves of one [T, 2*Hkv, D] buffer, as the layer passes them
    T, Hq, Hkv, D = 400, 8, 2, 128
    q = rand_t((T, Hq, D), 21)
    kv = rand_t((T, 2 * Hkv, D), 22)
    m = meta([T])
    kvd = kv.to(DEV)
    qs, ql, qf = _dev(*m)
    o, lse = lsa.prefill_attention_step(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], qs, ql, qf, qs, ql, qf, 1, T)
    o_ref, lse_ref = orc.attn_step(q, kv[:, :Hkv], kv[:, Hkv:], *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")


def _ring_chunks(k, v, lens, nshard, seed, Hkv):
    from loongserve_amd.simulate import KVChunk
    from tests.test_oracle_pins import _shard_contiguous
    g = torch.Generator().manual_seed(seed)
    shards = _shard_contiguous(k, v, lens, nshard, g)
    chunks = [KVChunk(torch.cat([ks, vs], 1).to(DEV), st.to(DEV), ln.to(DEV), fr.to(DEV)) for ks, vs, st, ln, fr in shards]
    return shards, chunks


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_ring_inplace_state_matches_monolithic(lsa, dtype):
    # the reference's own self-test recipe (RING:324-427): B=2, Hq=40, Hkv=4, D=128, KV split
    # contiguously over 8 nodes, result compared with dense causal attention
    from loongserve_amd.simulate import ring_prefill, ring_prefill_partials
    g = torch.Generator().manual_seed(0)
    lens = [int(x) for x in torch.randint(1, 1024, (2,), generator=g)]
    T, Hq, Hkv, D = sum(lens), 40, 4, 128
    q, k, v = rand_t((T, Hq, D), 31, dtype), rand_t((T, Hkv, D), 32, dtype), rand_t((T, Hkv, D), 33, dtype)
    m = meta(lens)
    shards, chunks = _ring_chunks(k, v, lens, 8, 5, Hkv)
    # node order starting from a chunk that is not the first one, as a ring would
    order = [3, 2, 1, 0, 7, 6, 5, 4]
    qs, ql, qf = _dev(*m)
    o, ms, ls = ring_prefill(q.to(DEV), [chunks[i] for i in order], qs, ql, qf, 1, max(lens), Hkv)
    torch.cuda.synchronize()
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    # the oracle's in-place state over the same eight steps, o stored in the same dtype after every step
    o_st = torch.zeros((T, Hq, D), dtype=dtype)
    m_st, l_st = torch.full((T, Hq), float("-inf")), torch.zeros(T, Hq)
    for i in order:
        ks, vs, st, ln, fr = shards[i]
        orc.context_attention_fwd(q, ks, vs, o_st, *m, st, ln, fr, 1, max(lens), m_st, l_st)
    assert_inplace_o_close(o.cpu(), o_st, o_ref, "ring o")
    assert_lse_close(orc.state_lse(ms.cpu(), ls.cpu()).float(), lse_ref, "state LSE")
    # the fp32-partial route meets the fp32 bars for both dtypes
    o2, lse2 = ring_prefill_partials(q.to(DEV), [chunks[i] for i in order], qs, ql, qf, 1, max(lens), Hkv)
    torch.cuda.synchronize()
    assert_o_close(o2, o_ref, "partials O")
    assert_lse_close(lse2, lse_ref, "partials LSE")
    # and the in-place update agrees with the oracle's restatement of the same recurrence
    o_c = torch.zeros(T, Hq, D, dtype=dtype)
    m_c = torch.full((T, Hq), float("-inf"))
    l_c = torch.zeros(T, Hq)
    for i in order:
        ks, vs, st, ln, fr = shards[i]
        orc.context_attention_fwd(q, ks, vs, o_c, *m, st, ln, fr, 1, max(lens), m_c, l_c)
    assert_lse_close(orc.state_lse(ms.cpu(), ls.cpu()).float(), orc.state_lse(m_c, l_c).float(), "state vs oracle state")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (4, 4)])
def test_inplace_step_over_rows_in_their_start_state_beside_rows_that_carry_one(lsa, dtype, Hq, Hkv):
    # The in-place operator reads a row's old o only if the row carries an earlier step's result (m > -inf, l > 0); rows
    # in their start state may hold anything there.  Both kinds side by side in the blocks of sixteen rows the kernel
    # works in, in whole blocks of either kind, in a whole sequence of either kind; o of the start-state rows is NaN on
    # the device and zero for the oracle.
    lens = [700, 333, 64]
    T, D = sum(lens), 128
    q, k, v = rand_t((T, Hq, D), 61, dtype), rand_t((T, Hkv, D), 62, dtype), rand_t((T, Hkv, D), 63, dtype)
    qm = meta(lens, [5000, 5000, 5000])
    # an earlier step over other keys (positions below every query's) gives every row a state ...
    k0, v0 = rand_t((T, Hkv, D), 64, dtype), rand_t((T, Hkv, D), 65, dtype)
    o_ref = torch.zeros((T, Hq, D), dtype=dtype)
    m_ref, l_ref = torch.full((T, Hq), float("-inf")), torch.zeros(T, Hq)
    km0 = meta(lens)
    orc.context_attention_fwd(q, k0, v0, o_ref, *qm, *km0, 1, max(lens), m_ref, l_ref)
    assert torch.isfinite(m_ref).all()
    # ... which these rows lose again: a ragged stretch, whole blocks, single rows, all of the last sequence
    fresh = torch.zeros(T, dtype=torch.bool)
    fresh[5:23] = True
    fresh[64:192] = True
    fresh[300:700:7] = True
    fresh[700 + 100:700 + 333] = True
    fresh[700 + 333:] = True
    o_ref[fresh] = 0
    m_ref[fresh] = float("-inf")
    l_ref[fresh] = 0
    o_d, m_d, l_d = _dev(o_ref.clone(), m_ref.clone(), l_ref.clone())
    o_d[fresh.to(DEV)] = float("nan")
    qd, kd, vd = _dev(q, k, v)
    qs, ql, qf = _dev(*qm)
    lsa.context_attention_fwd(qd, kd, vd, o_d, qs, ql, qf, qs, ql, qf, 1, max(lens), m_d, l_d)
    torch.cuda.synchronize()
    o_exact, lse_now = orc.attn_step(q, k, v, *qm, *qm, 1)
    o_prev, lse_prev = orc.attn_step(q, k0, v0, *qm, *km0, 1)
    orc.context_attention_fwd(q, k, v, o_ref, *qm, *qm, 1, max(lens), m_ref, l_ref)
    assert torch.isfinite(o_d.float()).all()
    # the exact answer: this step alone for the fresh rows, both steps merged for the others
    both_o, both_lse = orc.lse_merge([(o_prev, lse_prev), (o_exact, lse_now)])
    exact = torch.where(fresh[:, None, None], o_exact, both_o)
    assert_inplace_o_close(o_d.cpu(), o_ref, exact, "o")
    assert_lse_close(orc.state_lse(m_d.cpu(), l_d.cpu()).float(), torch.where(fresh[:, None], lse_now, both_lse), "state LSE")


def test_striped_ring_equals_full_sequence(lsa):
    from loongserve_amd.simulate import KVChunk, ring_prefill_partials
    T, Hq, Hkv, D, P = 1531, 4, 2, 128, 4
    q, k, v = rand_t((T, Hq, D), 41), rand_t((T, Hkv, D), 42), rand_t((T, Hkv, D), 43)
    m = meta([T])
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    chunks = []
    for j in range(P):
        kj = torch.cat([k[j::P], v[j::P]], 1)
        st, ln, fr = meta([kj.shape[0]], [j])
        chunks.append(KVChunk(kj.to(DEV), st.to(DEV), ln.to(DEV), fr.to(DEV)))
    for r in range(P):
        qi = q[r::P].contiguous()
        qs, ql, qf = _dev(*meta([qi.shape[0]], [r]))
        order = [(r - i) % P for i in range(P)]  # local chunk first, then what the ring delivers
        o, lse = ring_prefill_partials(qi.to(DEV), [chunks[i] for i in order], qs, ql, qf, P, qi.shape[0], Hkv)
        torch.cuda.synchronize()
        assert_o_close(o, o_ref[r::P], "striped O rank %d" % r)
        assert_lse_close(lse, lse_ref[r::P], "striped LSE rank %d" % r)


def test_lse_merge_kernel_and_empty_partials(lsa):
    R, H, D = 70, 3, 128
    parts = [(rand_t((R, H, D), 50 + i, torch.float32), rand_t((R, H), 60 + i, torch.float32) * 8) for i in range(5)]
    parts[1][1][:10] = float("-inf")
    parts[1][0][:10] = 0
    for p in parts:
        p[1][20:25] = float("-inf")
        p[0][20:25] = 0
    o_ref, l_ref = orc.lse_merge(parts)
    o, l = lsa.lse_merge([(a.to(DEV), b.to(DEV)) for a, b in parts])
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "merge O", max_abs=1e-5, rel=1e-5)
    assert_lse_close(l, l_ref, "merge LSE", rel=1e-5)
    assert torch.all(o[20:25] == 0)


def test_kv_scatter_and_register_bit_exact(lsa):
    T, Hkv, D, pool_n = 777, 2, 128, 2000
    g = torch.Generator().manual_seed(7)
    src = rand_t((T, 2 * Hkv, D), 70, torch.bfloat16)
    dest = torch.randperm(pool_n, generator=g)[:T].to(torch.int32)
    pool = torch.zeros(pool_n, 2 * Hkv, D, dtype=torch.bfloat16)
    pool_d = pool.to(DEV)
    lsa.kv_scatter(src.to(DEV), dest.to(DEV), pool_d)
    orc.kv_scatter(src, dest, pool)
    assert torch.equal(pool_d.cpu().view(torch.int16), pool.view(torch.int16))
    lens = [500, 0, 277]
    st, ln, _ = meta(lens)
    b_req = torch.tensor([4, 1, 2], dtype=torch.int32)
    table = torch.full((6, 600), orc.INT32_PAD, dtype=torch.int32)
    table_d = table.to(DEV)
    lsa.init_req_to_token_indexes(table_d, b_req.to(DEV), ln.to(DEV), dest.to(DEV), st.to(DEV), max(lens))
    orc.register_tokens(table, b_req, st, ln, dest)
    assert torch.equal(table_d.cpu(), table)
    # the operator names the reference's layer and model call: row scatter, one new slot per request in decode
    pool2 = torch.zeros(pool_n, 2 * Hkv, D, dtype=torch.bfloat16, device=DEV)
    lsa.destindex_copy_kv(src.to(DEV), dest.to(DEV).long(), pool2)
    assert torch.equal(pool2, pool_d)
    for dt in (torch.int32, torch.int64):
        B = 1000
        req = torch.randperm(1200, generator=g)[:B].to(torch.int32)
        ln1 = torch.randint(1, 601, (B,), generator=g, dtype=torch.int32)
        mem = torch.randint(0, 2_000_000, (B,), generator=g).to(dt)
        t_ref = torch.full((1200, 600), orc.INT32_PAD, dtype=torch.int32)
        t_dev = t_ref.to(DEV)
        lsa.copy_kv_index_to_req(t_dev, req.to(DEV), ln1.to(DEV), mem.to(DEV))
        orc.copy_kv_index_to_req(t_ref, req, ln1, mem)
        assert torch.equal(t_dev.cpu(), t_ref)
    # a length of 0 or beyond the row is skipped, nothing else is touched
    t_dev = torch.full((3, 8), 5, dtype=torch.int32, device=DEV)
    lsa.copy_kv_index_to_req(t_dev, torch.tensor([0, 1, 2], dtype=torch.int32, device=DEV),
                             torch.tensor([0, 9, 8], dtype=torch.int32, device=DEV), torch.tensor([7, 7, 7], device=DEV))
    want = torch.full((3, 8), 5, dtype=torch.int32)
    want[2, 7] = 7
    assert torch.equal(t_dev.cpu(), want)


def test_bf16_v_converted_inside_the_kernel_or_before_it(lsa):
    """Both routes for a bfloat16 V (fp16 copy made before the launch, the default; conversion while the tile is
    staged) against the oracle, on lengths that take the main loop and the masked steps, V as a strided view."""
    from loongserve_amd import ops
    lens, Hq, Hkv, D = [700, 1500], 8, 2, 128
    T = sum(lens)
    q = rand_t((T, Hq, D), 11, torch.bfloat16)
    kv = rand_t((T, 2 * Hkv, D), 12, torch.bfloat16)
    k, v = kv[:, :Hkv], kv[:, Hkv:]
    m = meta(lens)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    kvd = kv.to(DEV)
    try:
        for pre in (True, False):
            ops.PRECONVERT_BF16_V = pre
            qs, ql, qf = _dev(*m)
            o, lse = lsa.prefill_attention_step(q.to(DEV), kvd[:, :Hkv], kvd[:, Hkv:], qs, ql, qf, qs, ql, qf, 1, max(lens))
            assert_o_close(o, o_ref, "O (pre-converted V: %s)" % pre)
            assert_lse_close(lse, lse_ref, "LSE (pre-converted V: %s)" % pre)
            # the same in two steps, the second folded into the first in the epilogue: keys [0, 400) of each request,
            # then the rest (rows before position 400 see nothing of the second chunk and must keep their values)
            cut = 400
            idx = torch.cat([torch.arange(int(s0), int(s0) + n) for s0, n in zip(m[0], lens)])
            first = torch.cat([torch.arange(int(s0), int(s0) + cut) for s0 in m[0]])
            rest = torch.cat([torch.arange(int(s0) + cut, int(s0) + n) for s0, n in zip(m[0], lens)])
            assert len(first) + len(rest) == len(idx)
            out = lse = None
            for rows, km in ((first, meta([cut] * len(lens))), (rest, meta([n - cut for n in lens], [cut] * len(lens)))):
                part = kvd[rows.to(DEV)]
                out, lse = lsa.prefill_attention_step(q.to(DEV), part[:, :Hkv], part[:, Hkv:], qs, ql, qf, *_dev(*km), 1,
                                                      max(lens), out, lse, accumulate=out is not None)
            assert_o_close(out, o_ref, "accumulated O (pre-converted V: %s)" % pre)
            assert_lse_close(lse, lse_ref, "accumulated LSE (pre-converted V: %s)" % pre)
    finally:
        ops.PRECONVERT_BF16_V = True


def test_bf16_step_whose_v_leaves_fp16s_range(lsa):
    """A bfloat16 V with magnitudes beyond fp16's largest finite value and below its smallest normal one: the P V product
    runs in fp16, so the step's result is that of the same step on V rewritten as fp16 toward zero (65504 for anything
    larger, fp16's subnormal grid below 2^-14, zero below 2^-24), on both routes (V rewritten before the launch, and
    inside the kernel).  The expected rewriting is spelled out value by value; the oracle runs on the rewritten V.
    O reaches the hundreds here, so its max-abs bar is scaled by the largest |O| of the oracle."""
    from loongserve_amd import ops
    lens, Hq, Hkv, D = [900, 333], 8, 2, 128
    T = sum(lens)
    q = rand_t((T, Hq, D), 21, torch.bfloat16)
    kv = rand_t((T, 2 * Hkv, D), 22, torch.bfloat16)
    special = [(70000.0, 65504.0), (-70000.0, -65504.0), (1e38, 65504.0), (-3e20, -65504.0), (65504.0, 65504.0),
               (2.0 ** -15, 2.0 ** -15), (3 * 2.0 ** -17, 3 * 2.0 ** -17), (-2.0 ** -20, -2.0 ** -20),
               (2.0 ** -26, 0.0), (1.5 * 2.0 ** -25, 0.0), (-1.75 * 2.0 ** -24, -2.0 ** -24)]
    g = torch.Generator().manual_seed(23)
    v_expect = kv[:, Hkv:].float().clone()     # every other value of N(0, 1) * 0.5 in bfloat16 is exact in fp16 down to 2^-24
    tiny = v_expect.abs() < 2.0 ** -14
    v_expect[tiny] = torch.trunc(v_expect[tiny] * 2.0 ** 24) / 2.0 ** 24
    for i in range(400):
        t, h, d = int(torch.randint(0, T, (1,), generator=g)), int(torch.randint(0, Hkv, (1,), generator=g)), int(torch.randint(0, D, (1,), generator=g))
        src, want = special[i % len(special)]
        kv[t, Hkv + h, d] = src
        assert float(kv[t, Hkv + h, d]) == float(torch.tensor(src).to(torch.bfloat16))
        v_expect[t, h, d] = want
    assert float(torch.tensor(1.5 * 2.0 ** -25).to(torch.bfloat16)) == 1.5 * 2.0 ** -25     # (the sources are exact in bfloat16)
    m = meta(lens)
    o_ref, lse_ref = orc.attn_step(q.float(), kv[:, :Hkv].float(), v_expect, *m, *m, 1)
    scale = max(1.0, float(o_ref.abs().max()))
    assert scale > 50
    kvd, qd = kv.to(DEV), q.to(DEV)
    qs, ql, qf = _dev(*m)
    try:
        for pre in (True, False):
            ops.PRECONVERT_BF16_V = pre
            o, lse = lsa.prefill_attention_step(qd, kvd[:, :Hkv], kvd[:, Hkv:], qs, ql, qf, qs, ql, qf, 1, max(lens))
            torch.cuda.synchronize()
            assert_o_close(o, o_ref, "O (pre-converted V: %s)" % pre, max_abs=2e-3 * scale)
            assert_lse_close(lse, lse_ref, "LSE (pre-converted V: %s)" % pre)
    finally:
        ops.PRECONVERT_BF16_V = True


def test_bf16_to_f16_rows_is_exact_in_range_and_saturates(lsa):
    from loongserve_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    src = (torch.randn(300, 3 * 128, generator=g) * 4).to(torch.bfloat16)
    src[0, :6] = torch.tensor([70000.0, -70000.0, 65504.0, 1e-3, 0.0, -0.0]).to(torch.bfloat16)
    src[1, 0] = float("inf")
    sd = src.to(DEV)
    view = sd[:, 128:256]                                  # a strided window: rows of 128 with stride 384
    dst = torch.zeros(300, 128, dtype=torch.float16, device=DEV)
    rc = lib.lsattn_bf16_to_f16_rows(view.data_ptr(), view.stride(0), dst.data_ptr(), dst.stride(0), 300, 128,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(dst.cpu(), src[:, 128:256].to(torch.float16))   # |values| here are far inside fp16's range
    full = torch.zeros(300, 384, dtype=torch.float16, device=DEV)
    assert lib.lsattn_bf16_to_f16_rows(sd.data_ptr(), 384, full.data_ptr(), 384, 300, 384, torch.cuda.current_stream().cuda_stream) == 0
    got = full.cpu()
    assert got[0, :6].tolist() == [65504.0, -65504.0, 65504.0, float(torch.tensor(1e-3).to(torch.bfloat16)), 0.0, -0.0]
    assert got[1, 0].item() == 65504.0 or math.isinf(got[1, 0].item())
    assert lib.lsattn_bf16_to_f16_rows(sd.data_ptr(), 384, full.data_ptr(), 384, 300, 380, None) == -1   # row_elems % 8


@pytest.mark.parametrize("D", [16, 32, 64])
def test_head_sizes_below_128(lsa, D):
    """RING:250 admits head sizes 16, 32 and 64; they have a kernel of their own.  One partial step, and two in-place
    steps whose second one folds into the first one's o."""
    print("case D", D, flush=True)
    lens, Hq, Hkv = [300, 77], 4, 2
    T = sum(lens)
    q, k, v = rand_t((T, Hq, D), 41), rand_t((T, Hkv, D), 42), rand_t((T, Hkv, D), 43)
    m = meta(lens)
    o, lse = _run_step(lsa, q, k, v, m, m, 1, max(lens))
    assert o.shape == (T, Hq, D)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")
    # an earlier chunk of 150 / 40 keys per request (positions before the queries': visible to all), then the causal one
    klens = [150, 40]
    k0, v0 = rand_t((sum(klens), Hkv, D), 44), rand_t((sum(klens), Hkv, D), 45)
    qm = meta(lens, [150, 40])
    km0 = meta(klens)
    od = torch.full((T, Hq, D), float("nan"), dtype=torch.float16, device=DEV)  # (rows in their start state may hold anything)
    md = torch.full((T, Hq), float("-inf"), device=DEV)
    ld = torch.zeros(T, Hq, device=DEV)
    oc, mc, lc = torch.zeros(T, Hq, D, dtype=torch.float16), torch.full((T, Hq), float("-inf")), torch.zeros(T, Hq)
    for kk, vv, km in ((k, v, qm), (k0, v0, km0)):
        lsa.context_attention_fwd(q.to(DEV), kk.to(DEV), vv.to(DEV), od, *_dev(*qm), *_dev(*km), 1, max(lens), md, ld)
        orc.context_attention_fwd(q, kk, vv, oc, *qm, *km, 1, max(lens), mc, lc)
    torch.cuda.synchronize()
    assert_o_close(od, oc.float(), "in-place o")
    assert_lse_close(orc.state_lse(md.cpu(), ld.cpu()).float(), orc.state_lse(mc, lc).float(), "state")


@pytest.mark.parametrize("D", [16, 32, 64])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_head_sizes_below_128_over_a_striped_ring(lsa, D, dtype):
    """The kernel of the small head sizes through everything the 128-wide one is asked: ragged batches with an empty
    request, grouped heads (7 query heads on 1 KV head, 6 on 3), a ring of P = 3 striped shards taken as separate fp32
    partials, folded into a running partial by the epilogue, and folded in place into (o, m, l); strided K/V views of one
    buffer; for bfloat16 the V converted by the kernel and brought as an fp16 copy."""
    print("case D", D, dtype, flush=True)
    from loongserve_amd.simulate import KVChunk, ring_prefill, ring_prefill_accumulate, ring_prefill_partials
    P = 3
    for lens, Hq, Hkv in (([257, 0, 64, 1], 7, 1), ([130, 333], 6, 3)):
        T = sum(lens)
        q, kv = rand_t((T, Hq, D), 71, dtype), rand_t((T, 2 * Hkv, D), 72, dtype)
        k, v = kv[:, :Hkv], kv[:, Hkv:]
        m = meta(lens)
        o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
        # shard r of the striped ring holds tokens r, r + P, ... of every sequence
        chunks, shards = [], []
        for r in range(P):
            idx, st, ln = [], [], []
            for s0, n in zip(m[0].tolist(), lens):
                ids = list(range(s0 + r, s0 + n, P))
                st.append(len(idx))
                ln.append(len(ids))
                idx += ids
            it = torch.tensor(idx, dtype=torch.long)
            km = (torch.tensor(st, dtype=torch.int32), torch.tensor(ln, dtype=torch.int32), torch.full((len(lens),), r, dtype=torch.int32))
            shards.append((kv[it], km))
            chunks.append(KVChunk(kv[it].to(DEV), *(t.to(DEV) for t in km)))
        # the queries of shard 1: tokens 1, 1 + P, ...
        qi, qst, qln = [], [], []
        for s0, n in zip(m[0].tolist(), lens):
            ids = list(range(s0 + 1, s0 + n, P))
            qst.append(len(qi))
            qln.append(len(ids))
            qi += ids
        qit = torch.tensor(qi, dtype=torch.long)
        qm = (torch.tensor(qst, dtype=torch.int32), torch.tensor(qln, dtype=torch.int32), torch.full((len(lens),), 1, dtype=torch.int32))
        ql_q = q[qit]
        qs_d, qn_d, qf_d = _dev(*qm)
        maxq = max(qln)
        order = [1, 0, 2]
        o1, lse1 = ring_prefill_partials(ql_q.to(DEV), [chunks[i] for i in order], qs_d, qn_d, qf_d, P, maxq, Hkv)
        o2, lse2 = ring_prefill_accumulate(ql_q.to(DEV), [chunks[i] for i in order], qs_d, qn_d, qf_d, P, maxq, Hkv)
        o3, m3, l3 = ring_prefill(ql_q.to(DEV), [chunks[i] for i in order], qs_d, qn_d, qf_d, P, maxq, Hkv)
        torch.cuda.synchronize()
        assert_o_close(o1, o_ref[qit], "partials O")
        assert_lse_close(lse1, lse_ref[qit], "partials LSE")
        assert_o_close(o2, o_ref[qit], "accumulated O")
        assert_lse_close(lse2, lse_ref[qit], "accumulated LSE")
        o_st = torch.zeros((len(qi), Hq, D), dtype=dtype)
        m_st, l_st = torch.full((len(qi), Hq), float("-inf")), torch.zeros(len(qi), Hq)
        for i in order:
            kvs, km = shards[i]
            orc.context_attention_fwd(ql_q, kvs[:, :Hkv], kvs[:, Hkv:], o_st, *qm, *km, P, maxq, m_st, l_st)
        assert_inplace_o_close(o3.cpu(), o_st, o_ref[qit], "ring o")
        assert_lse_close(orc.state_lse(m3.cpu(), l3.cpu()).float(), lse_ref[qit], "state LSE")
        if dtype == torch.bfloat16:
            # the caller's fp16 copy of V instead of the conversion inside the kernel
            c = chunks[0]
            vf = torch.empty((c.kv.shape[0], Hkv, D), dtype=torch.float16, device=DEV)
            o4, lse4 = lsa.prefill_attention_step(ql_q.to(DEV), c.kv[:, :Hkv], c.kv[:, Hkv:], qs_d, qn_d, qf_d, c.b_start_loc, c.b_seq_len, c.first_token_global_idx,
                                                  P, maxq, v_f16=vf)
            o5, lse5 = lsa.prefill_attention_step(ql_q.to(DEV), c.kv[:, :Hkv], c.kv[:, Hkv:], qs_d, qn_d, qf_d, c.b_start_loc, c.b_seq_len, c.first_token_global_idx, P, maxq)
            torch.cuda.synchronize()
            vsrc = c.kv[:, Hkv:].cpu().float()
            normal = vsrc.abs() >= 2.0 ** -14  # (exact in fp16's normal range)
            assert torch.equal(vf.cpu().float()[normal], vsrc[normal])
            assert torch.equal(o4, o5) and torch.equal(lse4, lse5)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_ring_accumulated_in_the_epilogue_matches_monolithic(lsa, dtype):
    """Steps folded into a running fp32 (O, LSE) by the kernel's epilogue: same bars as the separate merge, from a
    chunk order in which early steps leave some rows without any key (they must stay empty until a later step fills
    them), and the same again for a striped ring."""
    from loongserve_amd.simulate import KVChunk, ring_prefill_accumulate
    g = torch.Generator().manual_seed(1)
    lens = [int(x) for x in torch.randint(200, 1500, (3,), generator=g)]
    T, Hq, Hkv, D = sum(lens), 8, 2, 128
    q, k, v = rand_t((T, Hq, D), 91, dtype), rand_t((T, Hkv, D), 92, dtype), rand_t((T, Hkv, D), 93, dtype)
    m = meta(lens)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    qs, ql, qf = _dev(*m)
    for nshard, order in ((4, [3, 1, 0, 2]), (2, [1, 0]), (1, [0])):
        print("case", dtype, nshard, flush=True)
        _, chunks = _ring_chunks(k, v, lens, nshard, 6, Hkv)
        # the running partial starts as garbage: the first step writes every row
        out = torch.full((T, Hq, D), float("nan"), device=DEV)
        lse = torch.full((T, Hq), float("nan"), device=DEV)
        o, l = ring_prefill_accumulate(q.to(DEV), [chunks[i] for i in order], qs, ql, qf, 1, max(lens), Hkv, out, lse)
        torch.cuda.synchronize()
        assert o.data_ptr() == out.data_ptr() and l.data_ptr() == lse.data_ptr()
        assert_o_close(o, o_ref, "accumulated O")
        assert_lse_close(l, lse_ref, "accumulated LSE")
    # from the empty state (lse = -inf, o anything) every step may accumulate
    _, chunks = _ring_chunks(k, v, lens, 3, 7, Hkv)
    out = torch.full((T, Hq, D), float("nan"), device=DEV)
    lse = torch.full((T, Hq), float("-inf"), device=DEV)
    for c in (chunks[2], chunks[0], chunks[1]):
        lsa.prefill_attention_step(q.to(DEV), c.k(Hkv), c.v(Hkv), qs, ql, qf, c.b_start_loc, c.b_seq_len,
                                   c.first_token_global_idx, 1, max(lens), out, lse, accumulate=True)
    torch.cuda.synchronize()
    assert_o_close(out, o_ref, "accumulated from empty O")
    assert_lse_close(lse, lse_ref, "accumulated from empty LSE")
    with pytest.raises(ValueError):
        lsa.prefill_attention_step(q.to(DEV), c.k(Hkv), c.v(Hkv), qs, ql, qf, c.b_start_loc, c.b_seq_len,
                                   c.first_token_global_idx, 1, max(lens), accumulate=True)
    # striped ring, P = 3: rank r holds tokens r, r + P, ...
    P, T1 = 3, 1000
    q1, k1, v1 = q[:T1], k[:T1], v[:T1]
    m1 = meta([T1])
    o1_ref, lse1_ref = orc.attn_step(q1, k1, v1, *m1, *m1, 1)
    chunks = []
    for j in range(P):
        kj = torch.cat([k1[j::P], v1[j::P]], 1)
        st, ln, fr = meta([kj.shape[0]], [j])
        chunks.append(KVChunk(kj.to(DEV), st.to(DEV), ln.to(DEV), fr.to(DEV)))
    for r in range(P):
        qi = q1[r::P].contiguous()
        qs1, ql1, qf1 = _dev(*meta([qi.shape[0]], [r]))
        order = [(r - i) % P for i in range(P)]
        o, l = ring_prefill_accumulate(qi.to(DEV), [chunks[i] for i in order], qs1, ql1, qf1, P, qi.shape[0], Hkv)
        torch.cuda.synchronize()
        assert_o_close(o, o1_ref[r::P], "striped accumulated O rank %d" % r)
        assert_lse_close(l, lse1_ref[r::P], "striped accumulated LSE rank %d" % r)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale", [2.0, 4.0])
def test_peaked_softmax_keeps_the_bars(lsa, dtype, scale):
    """Scores of magnitude up to ~16 and ~64 (a few keys carry each row): the running max moves often and far, so the
    main loop's late-maximum path and the rescaling of the accumulators run many times."""
    print("case", dtype, scale, flush=True)
    lens, Hq, Hkv = [2300, 700], 4, 2
    T = sum(lens)
    g = torch.Generator().manual_seed(int(scale))
    q = (torch.randn((T, Hq, 128), generator=g) * scale).to(dtype)
    k = (torch.randn((T, Hkv, 128), generator=g) * scale).to(dtype)
    v = rand_t((T, Hkv, 128), 3, dtype)
    m = meta(lens)
    o, lse = _run_step(lsa, q, k, v, m, m, 1, max(lens))
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("P", [1, 3])
def test_short_queries_against_long_kv_split_along_the_keys(lsa, dtype, P):
    """kv_splits of prefill_attention_step: three sequences of 1 to 200 query rows against KV chunks of 0 to 20000 keys
    (causal boundary inside the chunk, before it, and past its end), GQA 8/2: the slices' partials merged by the library
    equal the unsplit step and the oracle; the library's own choice of the split; accumulate on top of a running partial;
    the caller's workspace."""
    from loongserve_amd import ops
    Hq, Hkv, D = 8, 2, 128
    qlens, klens = [200, 1, 77], [20000, 0, 9000]
    qf = [19000 * P + 1, 5, 30000 * P]          # boundary inside the chunk / nothing to see / everything visible
    kf = [0, 0, 2]
    q = rand_t((sum(qlens), Hq, D), 4100 + P, dtype)
    k = rand_t((sum(klens), Hkv, D), 4200 + P, dtype)
    v = rand_t((sum(klens), Hkv, D), 4300 + P, dtype)
    qm, km = meta(qlens, qf), meta(klens, kf)
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
    dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    dqm, dkm = [t.to(DEV) for t in qm], [t.to(DEV) for t in km]
    assert ops.kv_split_count(len(qlens), Hq, max(qlens), k.shape[0]) > 1
    o1, l1 = lsa.prefill_attention_step(dq, dk, dv, *dqm, *dkm, P, max(qlens), kv_splits=1)
    for S in (None, 2, 7, 15, 33, 64):
        o, l = lsa.prefill_attention_step(dq, dk, dv, *dqm, *dkm, P, max(qlens), kv_splits=S)
        torch.cuda.synchronize()
        assert_o_close(o, o_ref, "O, %s slices" % S)
        assert_lse_close(l, lse_ref, "LSE, %s slices" % S)
        assert_o_close(o, o1.cpu(), "O against the unsplit step, %s slices" % S, max_abs=5e-4, rel=1e-3)
    # accumulate: a running partial over other keys (here: the same chunk once more, so the merge of the two is the chunk's
    # own result with LSE + ln 2), into the caller's workspace
    S = 5
    ws = (torch.empty((S * q.shape[0], Hq, D), device=DEV), torch.empty((S * q.shape[0], Hq), device=DEV))
    o_run, l_run = o1.clone(), l1.clone()
    lsa.prefill_attention_step(dq, dk, dv, *dqm, *dkm, P, max(qlens), out=o_run, lse=l_run, accumulate=True, kv_splits=S,
                               kv_split_workspace=ws)
    torch.cuda.synchronize()
    assert_o_close(o_run, o_ref, "O, accumulated")
    seen = torch.isfinite(lse_ref)
    assert_lse_close(l_run.cpu()[seen], lse_ref[seen] + math.log(2.0), "LSE, accumulated")
    assert bool((l_run.cpu()[~seen] == float("-inf")).all())


@pytest.mark.parametrize("dtype,Hq,Hkv", [(torch.float16, 32, 8), (torch.bfloat16, 16, 16), (torch.float16, 8, 8)])
def test_skewed_batch_with_a_bound_on_its_rows_walks_the_units_that_exist(lsa, prefill_geometry, dtype, Hq, Hkv):
    """One request of 6000 rows among 69 of 0 to 300 (two of them empty) with total_q_len = the rows of the packed q: the
    grid sized by the longest request would be 70 x 24 query tiles per head group and nearly all of them empty, so the
    launch numbers the tiles that exist (every workgroup finds its request from q_b_seq_len; 70 requests: two steps of 64).
    All three epilogues, against the oracle; a second, shifted KV chunk through the folding ones; every forced
    workgroup shape.  A batch the bound does not shrink by half (all requests alike) takes the ordinary grid."""
    import random
    rng = random.Random(Hq)
    lens = [rng.randint(1, 300) for _ in range(70)]
    lens[0] = lens[33] = 0
    lens[65] = 6000
    T = sum(lens)
    q = rand_t((T, Hq, 128), 4701, dtype)
    k, v = rand_t((T, Hkv, 128), 4702, dtype), rand_t((T, Hkv, 128), 4703, dtype)
    m = meta(lens)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    dm = _dev(*m)
    o, lse = lsa.prefill_attention_step(dq, dk, dv, *dm, *dm, 1, max(lens), total_q_len=T)
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")
    # an earlier chunk of 40 keys per request, all visible (positions before the queries'), folded in by both folding epilogues
    klens = [40 if n else 0 for n in lens]
    k0, v0 = rand_t((sum(klens), Hkv, 128), 4704, dtype), rand_t((sum(klens), Hkv, 128), 4705, dtype)
    qm, km0 = meta(lens, [40] * len(lens)), meta(klens)
    kml = meta(lens, [40] * len(lens))
    p0 = orc.attn_step(q, k0, v0, *qm, *km0, 1)
    p1 = orc.attn_step(q, k, v, *qm, *kml, 1)
    o2_ref, l2_ref = orc.lse_merge([p0, p1])
    dqm = _dev(*qm)
    out, l2 = lsa.prefill_attention_step(dq, k0.to(DEV), v0.to(DEV), *dqm, *_dev(*km0), 1, max(lens), total_q_len=T)
    lsa.prefill_attention_step(dq, dk, dv, *dqm, *_dev(*kml), 1, max(lens), out=out, lse=l2, accumulate=True, total_q_len=T)
    torch.cuda.synchronize()
    seen = torch.isfinite(l2_ref)
    assert_o_close(out.cpu()[seen], o2_ref[seen], "accumulated O")
    assert_lse_close(l2, l2_ref, "accumulated LSE")
    o_st = torch.zeros((T, Hq, 128), dtype=dtype, device=DEV)
    m_st = torch.full((T, Hq), float("-inf"), device=DEV)
    l_st = torch.zeros((T, Hq), device=DEV)
    lsa.context_attention_fwd(dq, k0.to(DEV), v0.to(DEV), o_st, *dqm, *_dev(*km0), 1, max(lens), m_st, l_st, total_q_len=T)
    lsa.context_attention_fwd(dq, dk, dv, o_st, *dqm, *_dev(*kml), 1, max(lens), m_st, l_st, total_q_len=T)
    torch.cuda.synchronize()
    assert_lse_close(orc.state_lse(m_st.cpu(), l_st.cpu()).float(), l2_ref, "state LSE")
    bar = dict(max_abs=2e-3, rel=1.5e-3) if dtype == torch.float16 else dict(max_abs=2e-2, rel=6e-3)
    assert_o_close(o_st.cpu()[seen], o2_ref[seen], "in-place o", **bar)
    # a loose bound (twice the rows) is as good; a uniform batch keeps the ordinary grid and the same answer
    o3, l3 = lsa.prefill_attention_step(dq, dk, dv, *dm, *dm, 1, max(lens), total_q_len=2 * T + 5)
    torch.cuda.synchronize()
    assert torch.equal(o3, o) and torch.equal(l3, lse)


def test_kv_cuts_leave_rows_outside_the_sequences_alone(lsa):
    """Rows of q / out that belong to no sequence (a gap between two sequences and a tail) keep what they hold on the
    route cut along the keys, as on the unsplit one, with and without accumulate; the partials' workspace starts as NaN.
    One tensor as workspace, max_kv_len as the bound the cuts are sized by (the k buffer is much taller than the chunks)."""
    Hq, Hkv, D, P = 8, 2, 128, 1
    qlens, klens = [130, 40], [9000, 12000]
    q = rand_t((200, Hq, D), 4401)                       # rows 130..139 and 180..199 belong to no sequence
    k = rand_t((40000, Hkv, D), 4402)                    # chunks at rows 100 and 20000 of a tall buffer
    v = rand_t((40000, Hkv, D), 4403)
    qm = (torch.tensor([0, 140], dtype=torch.int32), torch.tensor(qlens, dtype=torch.int32), torch.tensor([50000, 11000], dtype=torch.int32))
    km = (torch.tensor([100, 20000], dtype=torch.int32), torch.tensor(klens, dtype=torch.int32), torch.tensor([0, 0], dtype=torch.int32))
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
    covered = torch.zeros(200, dtype=torch.bool)
    covered[0:130] = True
    covered[140:180] = True
    dq, dk, dv = q.to(DEV), k.to(DEV), v.to(DEV)
    dqm, dkm = [t.to(DEV) for t in qm], [t.to(DEV) for t in km]
    from loongserve_amd import ops
    assert ops.kv_split_count(2, Hq, max(qlens), max(klens)) > 1
    S = 6
    ws = torch.full((S * 200 * Hq * (D + 1) + 7,), float("nan"), device=DEV)
    out = torch.full((200, Hq, D), 7.0, device=DEV)
    lse = torch.full((200, Hq), 7.0, device=DEV)
    lsa.prefill_attention_step(dq, dk, dv, *dqm, *dkm, P, max(qlens), out=out, lse=lse, kv_splits=S, kv_split_workspace=ws,
                               max_kv_len=max(klens))
    torch.cuda.synchronize()
    assert_o_close(out.cpu()[covered], o_ref[covered], "O")
    assert_lse_close(lse.cpu()[covered], lse_ref[covered], "LSE")
    assert bool((out.cpu()[~covered] == 7.0).all()) and bool((lse.cpu()[~covered] == 7.0).all())
    # accumulate onto an empty running partial whose rows outside the sequences hold a sentinel
    out2 = torch.full((200, Hq, D), float("nan"), device=DEV)
    lse2 = torch.full((200, Hq), float("-inf"), device=DEV)
    out2[~covered.to(DEV)] = 3.0
    lse2[~covered.to(DEV)] = 3.0
    lsa.prefill_attention_step(dq, dk, dv, *dqm, *dkm, P, max(qlens), out=out2, lse=lse2, accumulate=True, max_kv_len=max(klens))
    torch.cuda.synchronize()
    assert_o_close(out2.cpu()[covered], o_ref[covered], "O, accumulated onto empty rows")
    assert_lse_close(lse2.cpu()[covered], lse_ref[covered], "LSE, accumulated onto empty rows")
    assert bool((out2.cpu()[~covered] == 3.0).all()) and bool((lse2.cpu()[~covered] == 3.0).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("P", [1, 3])
def test_context_attention_fwd_with_a_workspace_cuts_the_kv_chunk(lsa, dtype, P):
    """The reference's operator with workspace=: short query chunks (a chunked-prefill step) against KV chunks of up to
    20000 keys, GQA 8/2.  Three steps into one (o, m, l): from the start state through the cut route, an ordinary step,
    and a cut step on top of the running state; against the oracle's restatement of the same update after every step, and
    the final result against one exact step over all keys.  o, m, l strided views (RING:270-275 pass their strides)."""
    Hq, Hkv, D = 8, 2, 128
    qlens = [100, 7, 64]
    Tq = sum(qlens)
    q = rand_t((Tq, Hq, D), 4500 + P, dtype)
    chunks = []
    for j, klens in enumerate(([20000, 3000, 0], [500, 200, 300], [9000, 11000, 8200])):
        k = rand_t((sum(klens), Hkv, D), 4510 + 10 * j + P, dtype)
        v = rand_t((sum(klens), Hkv, D), 4511 + 10 * j + P, dtype)
        kf = [j, 100000 * P + j, 40000 * P + j] if P > 1 else [30000 * j, 300000 + 20000 * j, 100000 + 20000 * j]
        chunks.append((k, v, meta(klens, kf), klens))
    qf = [59990 * P + 1, 390000 * P, 150000 * P]  # sequence 0 ends inside chunk 2's first KV range when P = 1
    qm = meta(qlens, qf)
    o_big = torch.zeros((Tq, Hq + 2, D), dtype=dtype, device=DEV)
    ml_big = torch.zeros((2, Tq, Hq + 1), device=DEV)
    o, m, l = o_big[:, 1:Hq + 1], ml_big[0, :, :Hq], ml_big[1, :, :Hq]
    m.fill_(float("-inf"))
    o_st = torch.zeros((Tq, Hq, D), dtype=dtype)
    m_st, l_st = torch.full((Tq, Hq), float("-inf")), torch.zeros(Tq, Hq)
    ws = torch.full((6 * Tq * Hq * (D + 1),), float("nan"), device=DEV)
    dq, dqm = q.to(DEV), [t.to(DEV) for t in qm]
    parts = []
    for j, (k, v, km, klens) in enumerate(chunks):
        dkm = [t.to(DEV) for t in km]
        kw = dict(workspace=ws, max_kv_len=max(klens), kv_splits=None if j == 0 else 5) if j != 1 else {}
        lsa.context_attention_fwd(dq, k.to(DEV), v.to(DEV), o, *dqm, *dkm, P, max(qlens), m, l, **kw)
        torch.cuda.synchronize()
        orc.context_attention_fwd(q, k, v, o_st, *qm, *km, P, max(qlens), m_st, l_st)
        parts.append(orc.attn_step(q, k, v, *qm, *km, P))
        o_exact, lse_exact = orc.lse_merge(parts)
        seen = torch.isfinite(lse_exact)
        assert_inplace_o_close(o.cpu()[seen], o_st[seen], o_exact[seen], "o after step %d" % j)
        assert_lse_close(orc.state_lse(m.cpu(), l.cpu()).float(), lse_exact, "state LSE after step %d" % j)
    assert bool((o_big[:, 0] == 0).all()) and bool((o_big[:, Hq + 1] == 0).all()) and bool((ml_big[:, :, Hq] == 0).all())
    # without max_kv_len the bound is the k buffer's height; a workspace that holds one cut only: the ordinary launch
    from loongserve_amd import ops
    assert ops._workspace_cuts(ws[:Tq * Hq * (D + 1)], Tq, Hq, D) == 1


@pytest.mark.parametrize("Hq,Hkv", [(3, 3), (12, 6), (24, 12), (40, 40), (35, 5), (21, 7), (18, 2), (9, 1)])
@pytest.mark.parametrize("P", [5, 7, 13, 64])
def test_launch_geometry_with_divisors_that_are_not_powers_of_two(lsa, Hq, Hkv, P):
    """The kernel derives a workgroup's (sequence, KV head, query head, query tile) and every row's visible keys with
    multiply-high divisions by launch constants (sp_peers, query heads per KV head, KV heads per XCD slot, slices, units per
    slice): head counts and stripe widths that make every one of those divisors a non-power of two, two ragged sequences."""
    D = 128
    qlens, klens = [300, 129], [257, 700]
    qf, kf = [3 * P + 2, 0], [1, 4]                  # striped positions: row m of q at qf + m P, key n at kf + n P
    q = rand_t((sum(qlens), Hq, D), 5100 + Hq + P, torch.float16)
    k = rand_t((sum(klens), Hkv, D), 5200 + Hq + P, torch.float16)
    v = rand_t((sum(klens), Hkv, D), 5300 + Hq + P, torch.float16)
    qm, km = meta(qlens, qf), meta(klens, kf)
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
    o, lse = lsa.prefill_attention_step(q.to(DEV), k.to(DEV), v.to(DEV), *[t.to(DEV) for t in qm], *[t.to(DEV) for t in km], P, max(qlens))
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")

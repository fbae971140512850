"""The five baseline configurations (the shapes the reference's headline figures are quoted on) at full size on the GPU.

Where the whole result is too large for the CPU oracle in seconds, the oracle checks a
seeded sample of rows / requests / heads (it receives exactly the rows it reads) and the
rest is covered by size-independent properties: in-place ring state vs merged fp32
partials, split-K granularity invariance, instance-split invariance, permutation
invariance of the token list, and a bit-exact read-back of scattered KV rows.
"""
import math

import pytest
import torch

import bench
from oracle import attn_oracle as orc
from tests.helpers import assert_lse_close, assert_o_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cpu_i32(x):
    return torch.tensor(x, dtype=torch.int32)


def test_config2_ring_prefill_full_size(lsa):
    from loongserve_amd.simulate import ring_prefill
    w = bench.RingPrefill()
    w.step()
    torch.cuda.synchronize()
    n, qs = w.shard, w.q_shard
    # oracle on sampled query rows (first, diagonal-adjacent, last) and 3 heads, against all 4 KV shards
    rows = [0, 1, 255, 256, 4097, n - 1]
    heads = [0, 13, 31]
    q = w.q[rows][:, heads].cpu()
    parts = []
    for c, j in zip(w.chunks, w.order):
        k = c.kv[:, heads].cpu()
        v = c.kv[:, [w.Hkv + h for h in heads]].cpu()
        # every sampled row is its own one-row "sequence" with its own global position
        qm = (_cpu_i32(list(range(len(rows)))), _cpu_i32([1] * len(rows)), _cpu_i32([qs * n + r for r in rows]))
        km = (_cpu_i32([0] * len(rows)), _cpu_i32([n] * len(rows)), _cpu_i32([j * n] * len(rows)))
        parts.append(orc.attn_step(q, k, v, *qm, *km, 1))
    o_ref, lse_ref = orc.lse_merge(parts)
    assert_o_close(w.out[rows][:, heads], o_ref, "cfg2 O (sampled rows)")
    assert_lse_close(w.lse[rows][:, heads], lse_ref, "cfg2 LSE (sampled rows)")
    # the route with four separate partials and one merge pass agrees with the merge in the epilogues everywhere
    o_acc, lse_acc = w.out.clone(), w.lse.clone()
    w.step_separate_merge()
    torch.cuda.synchronize()
    assert (o_acc - w.out).abs().max().item() <= 1e-6 and torch.allclose(lse_acc, w.lse, rtol=0, atol=1e-5)
    w.bufs = None
    # property: the in-place (o, m, l) ring state equals the merged fp32 partials everywhere
    o, m, l = ring_prefill(w.q, w.chunks, w.qs, w.ql, w.qf, 1, n, w.Hkv)
    torch.cuda.synchronize()
    lse_state = 0.6931471805599453 * (m.double() + torch.log2(l.double()))
    assert torch.allclose(lse_state.float(), w.lse, rtol=1e-4, atol=1e-4)
    err = (o.float() - w.out).abs().max().item()
    assert err <= 2e-3, "in-place ring vs merged partials: max-abs %.3e" % err
    # property: a softmax-weighted average stays inside the value range
    assert w.out.abs().max().item() <= w.chunks[0].kv.abs().max().item() * 1.001 + 1.0


def test_config3_token_decode_full_size(lsa):
    d = bench.TokenDecode()
    d.step()
    torch.cuda.synchronize()
    # oracle on three requests (shortest, longest, one in between); it receives exactly the rows it reads
    order = sorted(range(d.B), key=lambda b: d.lens[b])
    for b in (order[0], order[d.B // 2], order[-1]):
        n = d.lens[b]
        rows = d.table[b, :n].long()
        kv = d.kv[rows].cpu()
        table = torch.arange(n, dtype=torch.int32)[None]
        o_ref, l_ref = orc.decode_full(d.q[b:b + 1].cpu(), kv[:, :d.Hkv], kv[:, d.Hkv:], table, _cpu_i32([0]), _cpu_i32([n]))
        assert_o_close(d.o[b:b + 1], o_ref, "cfg3 O request %d" % b)
        assert_lse_close(d.lse[b:b + 1], l_ref, "cfg3 LSE request %d" % b)
    o1, l1 = d.o.clone(), d.lse.clone()
    # property: the split-K granularity does not change the result
    BS2 = 64
    nblk = (d.max_len + BS2 - 1) // BS2
    mo = torch.empty((nblk, d.B, d.Hq, d.D), dtype=torch.float32, device=DEV)
    ml = torch.empty((nblk, d.B, d.Hq), dtype=torch.float32, device=DEV)
    o2, l2 = lsa.longserve_token_decode_attention_flash_decoding(d.q, d.table, d.b_req, d.b_len, mo, ml, d.B, d.max_len, d.Hq, d.D,
                                                                 d.kv[:, :d.Hkv], d.kv[:, d.Hkv:], BS2)
    torch.cuda.synchronize()
    assert (o2 - o1).abs().max().item() <= 2e-5
    assert torch.allclose(l2, l1, rtol=1e-5, atol=1e-5)
    del mo, ml
    # property: attention does not depend on the order of a request's token list
    g = torch.Generator().manual_seed(7)
    table2 = d.table.clone()
    for b in range(d.B):
        p = torch.randperm(d.lens[b], generator=g).to(DEV)
        table2[b, :d.lens[b]] = d.table[b, :d.lens[b]][p]
    o3, l3 = lsa.longserve_token_decode_attention_flash_decoding(d.q, table2, d.b_req, d.b_len, d.mid_o, d.mid_l, d.B, d.max_len, d.Hq,
                                                                 d.D, d.kv[:, :d.Hkv], d.kv[:, d.Hkv:], d.BS)
    torch.cuda.synchronize()
    assert (o3 - o1).abs().max().item() <= 2e-5
    assert torch.allclose(l3, l1, rtol=1e-5, atol=1e-5)


def test_config4_elastic_decode_full_size(lsa):
    e = bench.ElasticDecode()
    o, lse = e.step()
    torch.cuda.synchronize()
    assert o.dtype == torch.float16
    # property: 4 instances + merge == one instance holding everything (fp32 output for the comparison)
    BS = 256
    nblk = (e.ctx + BS - 1) // BS
    mo = torch.empty((nblk, e.B, e.H, e.D), dtype=torch.float32, device=DEV)
    ml = torch.empty((nblk, e.B, e.H), dtype=torch.float32, device=DEV)
    o1, l1 = lsa.longserve_token_decode_attention_flash_decoding(e.q, e.full_table, e.b_req, torch.full((e.B,), e.ctx, dtype=torch.int32, device=DEV),
                                                                 mo, ml, e.B, e.ctx, e.H, e.D, e.kv[:, :e.H], e.kv[:, e.H:], BS)
    torch.cuda.synchronize()
    assert (o.float() - o1).abs().max().item() <= 2e-3  # fp16 output rounding
    assert torch.allclose(lse, l1, rtol=1e-5, atol=1e-5)
    # oracle: request 2, heads 5 and 31, all 524288 tokens (the CPU receives only those two heads' rows)
    b, heads = 2, [5, 31]
    rows = e.full_table[b].long()
    k = e.kv[rows][:, heads].cpu()
    v = e.kv[rows][:, [e.H + h for h in heads]].cpu()
    table = torch.arange(e.ctx, dtype=torch.int32)[None]
    o_ref, l_ref = orc.decode_full(e.q[b:b + 1, heads].cpu(), k, v, table, _cpu_i32([0]), _cpu_i32([e.ctx]))
    assert_o_close(o1[b:b + 1, heads], o_ref, "cfg4 O")
    assert_lse_close(l1[b:b + 1, heads], l_ref, "cfg4 LSE")


def test_config5_varlen_prefill_full_size(lsa):
    v = bench.VarlenPrefill()
    v.step()
    torch.cuda.synchronize()
    lens = v.lens
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    # oracle on sampled rows of the shortest, the longest and two other sequences, 2 query heads of different KV heads
    order = sorted(range(len(lens)), key=lambda i: lens[i])
    heads = [3, 30]
    kvh = [h // (v.Hq // v.Hkv) for h in heads]
    lse_state = (0.6931471805599453 * (v.m.double() + torch.log2(v.l.double()))).float()
    # the same step on the fp32-partial route (bf16 in, fp32 (O, LSE) out), which is held to the stated bars
    o32 = torch.empty((v.T, v.Hq, v.D), dtype=torch.float32, device=DEV)
    l32 = torch.empty((v.T, v.Hq), dtype=torch.float32, device=DEV)
    lsa.prefill_attention_step(v.q, v.kv[:, :v.Hkv], v.kv[:, v.Hkv:], v.start, v.len, v.first, v.start, v.len, v.first, 1, v.max_len,
                               out=o32, lse=l32, v_f16=v.v_f16, v_f16_valid=True)
    torch.cuda.synchronize()
    for i in (order[0], order[5], order[-2], order[-1]):
        n, s0 = lens[i], starts[i]
        rows = sorted(set([0, 1, 63, 64, n // 3, n - 2, n - 1]))
        q = v.q[[s0 + r for r in rows]][:, heads].cpu()
        o_ref = torch.empty(len(rows), len(heads), v.D)
        l_ref = torch.empty(len(rows), len(heads))
        for hi, kh in enumerate(kvh):
            k = v.kv[s0:s0 + n, kh:kh + 1].cpu()
            vv = v.kv[s0:s0 + n, v.Hkv + kh:v.Hkv + kh + 1].cpu()
            qm = (_cpu_i32(list(range(len(rows)))), _cpu_i32([1] * len(rows)), _cpu_i32(rows))
            km = (_cpu_i32([0] * len(rows)), _cpu_i32([n] * len(rows)), _cpu_i32([0] * len(rows)))
            oo, ll = orc.attn_step(q[:, hi:hi + 1], k, vv, *qm, *km, 1)
            o_ref[:, hi], l_ref[:, hi] = oo[:, 0], ll[:, 0]
        got = v.o[[s0 + r for r in rows]][:, heads]
        # o is stored in bfloat16 (8 significant bits): bar scaled to 2^-8
        assert_o_close(got, o_ref, "cfg5 o seq %d" % i, max_abs=8e-3, rel=4e-3)
        assert_lse_close(lse_state[[s0 + r for r in rows]][:, heads], l_ref, "cfg5 LSE seq %d" % i)
        assert_o_close(o32[[s0 + r for r in rows]][:, heads], o_ref, "cfg5 fp32 partial O seq %d" % i)  # 2e-3 / 1e-3
        assert_lse_close(l32[[s0 + r for r in rows]][:, heads], l_ref, "cfg5 fp32 partial LSE seq %d" % i)
    # KV persistence: every scattered row reads back bit-for-bit through the registered table
    for i in (order[0], order[-1]):
        n, s0 = lens[i], starts[i]
        slots = v.req_to_token[i, :n].long()
        assert torch.equal(slots.int(), v.mem_index[s0:s0 + n])
        assert torch.equal(v.pool[slots].view(torch.int16), v.kv[s0:s0 + n].view(torch.int16))
    assert int((v.req_to_token[order[0], lens[order[0]]:] != 2147483647).sum()) == 0

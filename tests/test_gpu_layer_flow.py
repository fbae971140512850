"""The path end to end, the way one attention layer of the reference drives it on a single instance
(longserve_transformer_layer_infer.py:70-96 rotary + KV write, :104-160 prefill, :224-281 decode; longserve_model.py:389-398
and :485-494 slot allocation): slots from the pool allocator, rotary embedding, K/V rows written to their slots, the prefill
step over the packed cache rows, registration in the request table, then several decode steps that each append one token per
request.  Every attention output is compared with dense causal attention over the same (rounded) rows, computed on the CPU
without the pool or the table, so a slip anywhere in the chain of formats shows."""
import math

import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from oracle import elementwise_oracle as ew
from tests.helpers import assert_lse_close, assert_o_close, meta, rand_t

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cos_sin(positions, D):
    inv = 1.0 / (10000.0 ** (torch.arange(0, D // 2, dtype=torch.float64) * 2.0 / D))
    ang = positions.to(torch.float64)[:, None] * inv[None, :]
    return torch.cos(ang).to(torch.float16), torch.sin(ang).to(torch.float16)


def _rotary_cpu(x, cos, sin):
    a = x.numpy().copy()
    ew.rotary_emb(a, cos.numpy(), sin.numpy())
    return torch.from_numpy(a)


def _dense_decode(q, ks, vs):
    """q [Hq, D], ks/vs [n, Hkv, D] -> (O [Hq, D], LSE [Hq]) in float64."""
    Hq, D = q.shape
    Hkv = ks.shape[1]
    qh = q.double().reshape(Hkv, Hq // Hkv, D)
    s = torch.einsum("hgd,nhd->hgn", qh, ks.double()) / math.sqrt(D)
    lse = torch.logsumexp(s, dim=-1)
    o = torch.einsum("hgn,nhd->hgd", torch.exp(s - lse[..., None]), vs.double())
    return o.reshape(Hq, D), lse.reshape(Hq)


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (4, 4)])
def test_prefill_then_decode_through_the_pool(lsa, Hq, Hkv):
    print("case", Hq, Hkv, flush=True)
    D, BLOCK_SEQ, steps = 128, 64, 3
    lens = [200, 77, 513]
    B, T = len(lens), sum(lens)
    mm = lsa.LongServeMemoryManager(3000, torch.float16, Hkv, D, 1)
    rm = lsa.LongServeReqManager(8, 1024, mm)
    # some of the pool is already held by others, so the slots handed out are scattered
    g = torch.Generator().manual_seed(5)
    others = torch.randperm(3000, generator=g)[:900].to(DEV)
    mm.add_refs(others)
    req_rows = rm.alloc(B)
    # the batch builder hands the layer int32 request rows (router/model_infer/pre_process.py:51)
    b_req_idx = torch.tensor(req_rows.cpu().tolist(), dtype=torch.int32, device=DEV)
    slots = mm.alloc(T)
    assert slots.dtype == torch.int64 and not bool(torch.isin(slots, others).any())

    # ---- prefill: rotary, KV rows to their slots, attention over the packed rows, registration
    start, b_len, first = meta(lens)
    pos = torch.cat([torch.arange(n) for n in lens])
    cos, sin = _cos_sin(pos, D)
    q, kv = rand_t((T, Hq, D), 61), rand_t((T, 2 * Hkv, D), 62)
    q_ref = _rotary_cpu(q, cos, sin)
    k_ref, v_ref = _rotary_cpu(kv[:, :Hkv].contiguous(), cos, sin), kv[:, Hkv:].contiguous()

    qd, kvd = q.to(DEV), kv.to(DEV)
    lsa.longserve_cuda_kernels.rotary_emb(qd, kvd[:, :Hkv], cos.to(DEV), sin.to(DEV))
    assert torch.equal(qd.cpu(), q_ref) and torch.equal(kvd[:, :Hkv].cpu(), k_ref)
    lsa.destindex_copy_kv(kvd, slots, mm.kv_buffer[0])                     # longserve_transformer_layer_infer.py:377
    od = torch.empty(T, Hq, D, dtype=torch.float16, device=DEV)
    md = torch.full((T, Hq), float("-inf"), device=DEV)
    ld = torch.zeros(T, Hq, device=DEV)
    sd, bd, fd = start.to(DEV), b_len.to(DEV), first.to(DEV)
    lsa.context_attention_fwd(qd, kvd[:, :Hkv], kvd[:, Hkv:], od, sd, bd, fd, sd, bd, fd, 1, max(lens), md, ld)
    lsa.init_req_to_token_indexes(rm.req_to_token_indexs, b_req_idx, bd, slots)
    torch.cuda.synchronize()
    o_ref, lse_ref = orc.attn_step(q_ref, k_ref, v_ref, start, b_len, first, start, b_len, first, 1)
    assert_o_close(od, o_ref, "prefill o")
    assert_lse_close(orc.state_lse(md.cpu(), ld.cpu()).float(), lse_ref, "prefill state")

    # ---- decode: one new token per request and step
    ks = [k_ref[int(s):int(s) + n] for s, n in zip(start, lens)]
    vs = [v_ref[int(s):int(s) + n] for s, n in zip(start, lens)]
    cache_k, cache_v = mm.kv_buffer[0][:, :Hkv], mm.kv_buffer[0][:, Hkv:]
    cur = b_len.clone()
    held = [slots]
    for step in range(steps):
        cos, sin = _cos_sin(cur, D)                    # the new token's position is the current length
        qn, kvn = rand_t((B, Hq, D), 70 + step), rand_t((B, 2 * Hkv, D), 80 + step)
        qn_ref = _rotary_cpu(qn, cos, sin)
        kn_ref, vn_ref = _rotary_cpu(kvn[:, :Hkv].contiguous(), cos, sin), kvn[:, Hkv:].contiguous()
        for b in range(B):
            ks[b] = torch.cat([ks[b], kn_ref[b:b + 1]])
            vs[b] = torch.cat([vs[b], vn_ref[b:b + 1]])
        got = mm.alloc_contiguous(B)                   # longserve_model.py:485-494: a contiguous run, else any slots
        new = got[0] if got is not None else mm.alloc(B)
        held.append(new)
        qnd, kvnd = qn.to(DEV), kvn.to(DEV)
        lsa.longserve_cuda_kernels.rotary_emb(qnd, kvnd[:, :Hkv], cos.to(DEV), sin.to(DEV))
        lsa.destindex_copy_kv(kvnd, new, mm.kv_buffer[0])
        cur = cur + 1
        lsa.copy_kv_index_to_req(rm.req_to_token_indexs, b_req_idx, cur.to(DEV), new)   # longserve_model.py:491
        max_len = int(cur.max())
        nblk = (max_len + BLOCK_SEQ - 1) // BLOCK_SEQ
        mid_o = torch.empty(nblk, B, Hq, D, dtype=torch.float32, device=DEV)
        mid_lse = torch.empty(nblk, B, Hq, dtype=torch.float32, device=DEV)
        o, lse = lsa.longserve_token_decode_attention_flash_decoding(
            qnd, rm.req_to_token_indexs, b_req_idx, cur.to(DEV), mid_o, mid_lse, B, max_len, Hq, D, cache_k, cache_v,
            BLOCK_SEQ)
        torch.cuda.synchronize()
        want = [_dense_decode(qn_ref[b], ks[b], vs[b]) for b in range(B)]
        assert_o_close(o, torch.stack([w[0] for w in want]), "decode step %d o" % step)
        assert_lse_close(lse, torch.stack([w[1] for w in want]), "decode step %d lse" % step)

    # ---- the request ends: everything it held goes back, the other holders keep theirs
    rm.free(req_rows, torch.cat(held))
    assert mm.can_use_mem_size == 3000 - 900 and rm.can_use_req_size == 8
    state = mm.mem_state.cpu().numpy()
    expect = np.zeros(3000, dtype=np.int32)
    expect[others.cpu().numpy()] = 1
    assert (state == expect).all()

"""The HIP kernels against the committed known answers (tests/golden/attention_known_answers.npz, written by
tests/golden/make_fixtures.py with float64 loops over the definition): one striped GQA prefill step through each of its
three epilogues, and token-indexed decode through the fused call and through the separate stages."""
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import assert_inplace_o_close, assert_lse_close, assert_o_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
Z = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_known_answers.npz"))


def _t(name):
    return torch.from_numpy(np.ascontiguousarray(Z[name]))


def _starts(name):
    ln = _t(name)
    return (torch.cumsum(ln, 0) - ln).to(torch.int32)


def test_prefill_step_known_answers(lsa):
    q, k, v = _t("pf_q").to(DEV), _t("pf_k").to(DEV), _t("pf_v").to(DEV)
    qm = [_starts("pf_q_len").to(DEV), _t("pf_q_len").to(DEV), _t("pf_q_first").to(DEV)]
    km = [_starts("pf_kv_len").to(DEV), _t("pf_kv_len").to(DEV), _t("pf_kv_first").to(DEV)]
    P, max_q = int(Z["pf_peers"]), int(Z["pf_q_len"].max())
    o_ref, lse_ref = _t("pf_o").float(), _t("pf_lse").float()
    o, lse = lsa.prefill_attention_step(q, k, v, *qm, *km, P, max_q)
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "partial O")
    assert_lse_close(lse, lse_ref, "partial LSE")
    seen = ~torch.isinf(lse_ref)
    assert torch.all(o.cpu()[~seen] == 0)
    # accumulating epilogue from the empty state, in-place epilogue from (-inf, 0)
    o2 = torch.full_like(o, float("nan"))
    lse2 = torch.full_like(lse, float("-inf"))
    lsa.prefill_attention_step(q, k, v, *qm, *km, P, max_q, o2, lse2, accumulate=True)
    od = torch.zeros(q.shape, dtype=torch.float16, device=DEV)
    md = torch.full(q.shape[:2], float("-inf"), device=DEV)
    ld = torch.zeros(q.shape[:2], device=DEV)
    lsa.context_attention_fwd(q, k, v, od, *qm, *km, P, max_q, md, ld)
    torch.cuda.synchronize()
    assert_lse_close(lse2, lse_ref, "accumulated LSE")
    assert_o_close(torch.where(seen[..., None], o2.cpu(), torch.zeros(())), o_ref, "accumulated O")
    state = 0.6931471805599453 * (md.double().cpu() + torch.log2(ld.double().cpu()))
    assert_lse_close(torch.where(seen, state.float(), torch.full((), float("-inf"))), lse_ref, "in-place state")
    # the oracle's in-place state from the same start: o rounded to fp16 once
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    o_st = torch.zeros(q.shape, dtype=torch.float16)
    m_st, l_st = torch.full(q.shape[:2], float("-inf")), torch.zeros(q.shape[:2])
    orc.context_attention_fwd(qc, kc, vc, o_st, *[t.cpu() for t in qm], *[t.cpu() for t in km], P, max_q, m_st, l_st)
    assert_inplace_o_close(od.cpu(), o_st, o_ref, "in-place o")


@pytest.mark.parametrize("block_seq", [16, 64, 256])
def test_decode_known_answers(lsa, block_seq):
    q, pool, table = _t("dc_q").to(DEV), _t("dc_pool").to(DEV), _t("dc_table").to(DEV)
    b_req, b_len = _t("dc_b_req").to(DEV), _t("dc_b_len").to(DEV)
    B, Hq, D = q.shape
    Hkv = pool.shape[1] // 2
    max_len = int(Z["dc_b_len"].max())
    nblk = (max_len + block_seq - 1) // block_seq
    o_ref, lse_ref = _t("dc_o").float(), _t("dc_lse").float()
    mo = torch.empty(nblk, B, Hq, D, device=DEV)
    ml = torch.empty(nblk, B, Hq, device=DEV)
    o, lse = lsa.longserve_token_decode_attention_flash_decoding(q, table, b_req, b_len, mo, ml, B, max_len, Hq, D, pool[:, :Hkv],
                                                                 pool[:, Hkv:], block_seq)
    torch.cuda.synchronize()
    assert_o_close(o, o_ref, "fused o")
    assert_lse_close(lse, lse_ref, "fused lse")
    o2 = torch.empty(B, Hq, D, device=DEV)
    lse2 = torch.empty(B, Hq, device=DEV)
    lsa.longserve_flash_decode_stage1(q, pool[:, :Hkv], pool[:, Hkv:], table, b_req, b_len, max_len, mo, ml, block_seq)
    lsa.longserve_flash_decode_stage2(mo, ml, b_len, o2, lse2, block_seq)
    torch.cuda.synchronize()
    assert_o_close(o2, o_ref, "staged o")
    assert_lse_close(lse2, lse_ref, "staged lse")

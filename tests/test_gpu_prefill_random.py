"""Seeded random sweep of the prefill step against the oracle: ragged batches, GQA groups, striped and offset steps,
empty KV chunks, lengths on both sides of every tile boundary, both dtypes (through the C ABI)."""
import random

import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import assert_inplace_o_close, assert_lse_close, assert_o_close, meta, rand_t

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("prefill_geometry")]
DEV = "cuda:0"


@pytest.mark.parametrize("seed", [1, 7, 23])
def test_random_steps_match_the_oracle(lsa, seed):
    _sweep(lsa, seed, 16, [128])


@pytest.mark.parametrize("seed", [2, 9])
def test_random_steps_of_head_sizes_below_128_match_the_oracle(lsa, seed):
    """The same sweep over the head sizes 16, 32 and 64 (a kernel of their own)."""
    _sweep(lsa, seed, 12, [16, 32, 64])


def _sweep(lsa, seed, cases, head_sizes):
    rng = random.Random(seed)
    for case in range(cases):
        D = rng.choice(head_sizes)
        dtype = rng.choice([torch.float16, torch.bfloat16])
        Hkv = rng.choice([1, 2, 3])
        Hq = Hkv * rng.choice([1, 2, 4])
        B = rng.choice([1, 2, 3])
        P = rng.choice([1, 1, 2, 3, 4])
        qlens = [rng.choice([1, 17, 255, 256, 257, 300, 511, 600, 900, 1400, 2100]) for _ in range(B)]
        klens = [rng.choice([0, 1, 63, 64, 200, 256, 448, 511, 512, 700, 1300, 2500]) for _ in range(B)]
        qf = [rng.choice([0, 1, 5, 300, 1000, 4000]) for _ in range(B)]
        kf = [rng.choice([0, 1, 2, 3, 100, 700]) for _ in range(B)]
        print("case", seed, case, D, dtype, Hq, Hkv, P, qlens, qf, klens, kf, flush=True)
        Tq, Tk = sum(qlens), max(sum(klens), 1)
        q = rand_t((Tq, Hq, D), 1000 * seed + case, dtype)
        k = rand_t((Tk, Hkv, D), 1000 * seed + 100 + case, dtype)
        v = rand_t((Tk, Hkv, D), 1000 * seed + 200 + case, dtype)
        qm, km = meta(qlens, qf), meta(klens, kf)
        o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
        o, lse = lsa.prefill_attention_step(q.to(DEV), k.to(DEV), v.to(DEV), *[t.to(DEV) for t in qm], *[t.to(DEV) for t in km],
                                            P, max(qlens))
        torch.cuda.synchronize()
        what = "seed %d case %d" % (seed, case)
        assert_o_close(o, o_ref, "O, " + what)
        assert_lse_close(lse, lse_ref, "LSE, " + what)
        # a second random chunk folded into the first step's result, by the accumulating epilogue and by the in-place
        # (o, m, l) one; the oracle merges the two steps' partials
        klens2 = [rng.choice([0, 1, 64, 130, 512, 700, 1300]) for _ in range(B)]
        kf2 = [rng.choice([0, 2, 50, 900]) for _ in range(B)]
        Tk2 = max(sum(klens2), 1)
        k2 = rand_t((Tk2, Hkv, D), 1000 * seed + 300 + case, dtype)
        v2 = rand_t((Tk2, Hkv, D), 1000 * seed + 400 + case, dtype)
        km2 = meta(klens2, kf2)
        o2_ref, lse2_ref = orc.lse_merge([(o_ref, lse_ref), orc.attn_step(q, k2, v2, *qm, *km2, P)])
        qd, qmd = q.to(DEV), [t.to(DEV) for t in qm]
        lsa.prefill_attention_step(qd, k2.to(DEV), v2.to(DEV), *qmd, *[t.to(DEV) for t in km2], P, max(qlens), o, lse,
                                   accumulate=True)
        od = torch.full((Tq, Hq, D), float("nan"), dtype=dtype, device=DEV)
        md = torch.full((Tq, Hq), float("-inf"), device=DEV)
        ld = torch.zeros(Tq, Hq, device=DEV)
        o_st = torch.zeros((Tq, Hq, D), dtype=dtype)  # the oracle's in-place state over the same two steps
        m_st, l_st = torch.full((Tq, Hq), float("-inf")), torch.zeros(Tq, Hq)
        for kk, vv, kmm in ((k, v, km), (k2, v2, km2)):
            lsa.context_attention_fwd(qd, kk.to(DEV), vv.to(DEV), od, *qmd, *[t.to(DEV) for t in kmm], P, max(qlens), md, ld)
            orc.context_attention_fwd(q, kk, vv, o_st, *qm, *kmm, P, max(qlens), m_st, l_st)
        torch.cuda.synchronize()
        assert_o_close(o, o2_ref, "accumulated O, " + what)
        assert_lse_close(lse, lse2_ref, "accumulated LSE, " + what)
        seen = ~torch.isinf(lse2_ref)
        od_seen = torch.where(seen[..., None], od.cpu(), torch.zeros((), dtype=dtype))  # (rows that saw no key keep what o held)
        assert_inplace_o_close(od_seen, torch.where(seen[..., None], o_st, torch.zeros((), dtype=dtype)), o2_ref, "in-place o, " + what)
        assert_lse_close(orc.state_lse(md.cpu(), ld.cpu()).float(), lse2_ref, "in-place state, " + what)

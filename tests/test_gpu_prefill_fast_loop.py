"""GPU parity cases aimed at the main loop of the prefill kernel (the part that runs unmasked, four 64-key tiles per
round, behind workgroup barriers) and at its hand-over to the masked general steps: striped (P > 1) and offset chunks long
enough to enter it, every remainder of the tile count modulo four, rows whose maximum is raised late in the sequence (the
rare rescale branch of the speculative softmax), and the in-place (o, m, l) state across ring steps in both dtypes."""
import pytest
import torch

from oracle import attn_oracle as orc
from tests.helpers import assert_inplace_o_close, assert_lse_close, assert_o_close, meta, rand_t

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("prefill_geometry")]
DEV = "cuda:0"


def _step(lsa, q, k, v, qm, km, P, max_q):
    d = lambda ts: [t.to(DEV) for t in ts]
    o, lse = lsa.prefill_attention_step(q.to(DEV), k.to(DEV), v.to(DEV), *d(qm), *d(km), P, max_q)
    torch.cuda.synchronize()
    return o, lse


@pytest.mark.parametrize("n_kv", [448, 449, 511, 512, 576, 640, 704, 768, 1023, 1280, 1344])
def test_full_step_every_tile_count_remainder(lsa, n_kv):
    """Non-causal step (queries far behind the chunk): the main loop takes floor((tiles - 3) / 4) rounds of four tiles, the
    general steps the rest; every remainder and the partial last tile are covered."""
    Hq, Hkv, D, n_q = 2, 1, 128, 300
    q, k, v = rand_t((n_q, Hq, D), 60), rand_t((n_kv, Hkv, D), 61), rand_t((n_kv, Hkv, D), 62)
    qm, km = meta([n_q], [5000]), meta([n_kv], [100])
    o, lse = _step(lsa, q, k, v, qm, km, 1, n_q)
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, 1)
    assert_o_close(o, o_ref, "O n_kv=%d" % n_kv)
    assert_lse_close(lse, lse_ref, "LSE n_kv=%d" % n_kv)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("P,qf,kf", [(4, 3, 1), (2, 0, 1), (3, 2, 2), (1, 2000, 300)])
def test_long_striped_and_offset_steps(lsa, dtype, P, qf, kf):
    """Striped / offset causal steps long enough for the main loop (the diagonal crosses the chunk in its second half)."""
    Hq, Hkv, D = 4, 2, 128
    qlens, klens = [1500, 700], [1400, 900]
    q = rand_t((sum(qlens), Hq, D), 71, dtype)
    k, v = rand_t((sum(klens), Hkv, D), 72, dtype), rand_t((sum(klens), Hkv, D), 73, dtype)
    qm, km = meta(qlens, [qf, qf + 1]), meta(klens, [kf, kf])
    o, lse = _step(lsa, q, k, v, qm, km, P, max(qlens))
    o_ref, lse_ref = orc.attn_step(q, k, v, *qm, *km, P)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")
    empty = torch.isinf(lse_ref)
    assert torch.all(o.cpu()[empty] == 0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_late_maximum_takes_the_rescale_branch(lsa, dtype):
    """Keys planted deep in the sequence that score 2^16 times above everything a row has seen: the speculative
    exponentials overflow the lazy threshold, the running maximum is raised and the sub-tile redone; several rows of
    one wave, rows of different waves, consecutive sub-tiles and the very first sub-tile are hit."""
    T, Hq, Hkv, D = 2304, 2, 1, 128
    q, k, v = rand_t((T, Hq, D), 81, dtype), rand_t((T, Hkv, D), 82, dtype), rand_t((T, Hkv, D), 83, dtype)
    plant = [(2300, 0, 1000), (2301, 0, 1001), (2290, 1, 1033), (2100, 0, 3), (2200, 1, 1600), (2200, 0, 1700), (2047, 0, 1900)]
    for row, h, key in plant:
        k[key, 0] = (q[row, h].float() * 4).to(dtype)   # q.k = 4 |q|^2 ~ 128: ~16 in log2 units after the scale
    m = meta([T])
    o, lse = _step(lsa, q, k, v, m, m, 1, T)
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    assert_o_close(o, o_ref, "O")
    assert_lse_close(lse, lse_ref, "LSE")
    # the planted score stands more than 2^8 above everything the row saw before it (so the branch really was needed)
    s2 = 1.4426950408889634 / 128 ** 0.5
    for row, h, key in plant:
        before = (k[:key, 0].float() @ q[row, h].float()).max().item() if key > 0 else float("-inf")
        assert (k[key, 0].float() @ q[row, h].float()).item() * s2 > before * s2 + 8


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_inplace_state_over_a_long_striped_ring(lsa, dtype):
    """context_attention_fwd's (o, m, l) state over P = 4 striped ring steps of a 6000-token sequence equals monolithic
    causal attention; o is stored in q's dtype."""
    T, Hq, Hkv, D, P = 6000, 4, 2, 128, 4
    q, k, v = rand_t((T, Hq, D), 91, dtype), rand_t((T, Hkv, D), 92, dtype), rand_t((T, Hkv, D), 93, dtype)
    m = meta([T])
    o_ref, lse_ref = orc.attn_step(q, k, v, *m, *m, 1)
    r = 1                                                  # this rank's stripe
    qi = q[r::P].contiguous().to(DEV)
    n = qi.shape[0]
    o = torch.zeros((n, Hq, D), dtype=dtype, device=DEV)
    ms = torch.full((n, Hq), float("-inf"), device=DEV)
    ls = torch.zeros((n, Hq), device=DEV)
    qs, ql, qf = [t.to(DEV) for t in meta([n], [r])]
    o_st = torch.zeros((n, Hq, D), dtype=dtype)  # the oracle's in-place state over the same steps
    m_st, l_st = torch.full((n, Hq), float("-inf")), torch.zeros(n, Hq)
    for i in range(P):
        j = (r - i) % P
        kj, vj = k[j::P].contiguous(), v[j::P].contiguous()
        kmeta = meta([kj.shape[0]], [j])
        ks, kl, kf = [t.to(DEV) for t in kmeta]
        lsa.context_attention_fwd(qi, kj.to(DEV), vj.to(DEV), o, qs, ql, qf, ks, kl, kf, P, n, ms, ls)
        orc.context_attention_fwd(q[r::P].contiguous(), kj, vj, o_st, *meta([n], [r]), *kmeta, P, n, m_st, l_st)
    torch.cuda.synchronize()
    assert_inplace_o_close(o.cpu(), o_st, o_ref[r::P], "in-place O")
    assert_lse_close(orc.state_lse(ms.cpu(), ls.cpu()).float(), lse_ref[r::P], "state LSE")

"""Shared input builders and the parity bars for the GPU tests."""
import math

import torch

from oracle import attn_oracle as orc

# parity bars of this build (per element / per tensor), written once:
O_MAX_ABS = 2e-3      # max |O_gpu - O_oracle|
O_REL = 1e-3          # ||O_gpu - O_oracle||_F / ||O_oracle||_F
LSE_REL = 1e-4        # max |LSE_gpu - LSE_oracle| / max(|LSE_oracle|, 1)


def rand_t(shape, seed, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 0.5).to(dtype)


def meta(lens, firsts=None):
    lens = torch.tensor(lens, dtype=torch.int32)
    start = (torch.cumsum(lens, 0) - lens).to(torch.int32)
    firsts = torch.zeros_like(lens) if firsts is None else torch.tensor(firsts, dtype=torch.int32)
    return start, lens, firsts


def assert_o_close(o_gpu, o_ref, what="", max_abs=O_MAX_ABS, rel=O_REL):
    a = o_gpu.detach().float().cpu()
    b = o_ref.float()
    assert a.shape == b.shape, (a.shape, b.shape)
    assert torch.isfinite(a).all(), what + ": non-finite output"
    err = (a - b).abs().max().item()
    fro = ((a - b).norm() / b.norm().clamp_min(1e-30)).item()
    assert err <= max_abs, "%s: max-abs %.3e > %.1e" % (what, err, max_abs)
    assert fro <= rel, "%s: relative %.3e > %.1e" % (what, fro, rel)


def assert_inplace_o_close(o_gpu, o_state_ref, o_exact, what=""):
    """The running `o` of context_attention_fwd, stored in q's dtype and re-rounded to it at every step.
    o_state_ref is the oracle's state after the same steps with the same storage dtype (oracle.context_attention_fwd
    rounds at every step too): held to the stated bars for float16; for bfloat16 to the same relative bar doubled and to
    one unit in the last place of that format below |o| = 2 (two roundings of nearly equal fp32 values differ by at
    most that).  o_exact, the fp32 answer, is a second, looser check that the state has not drifted."""
    if o_gpu.dtype == torch.float16:
        assert_o_close(o_gpu, o_state_ref, what + " (vs the oracle's fp16 state)", max_abs=O_MAX_ABS, rel=O_REL)
        assert_o_close(o_gpu, o_exact, what + " (vs the fp32 answer)", max_abs=2e-3, rel=1.5e-3)
    else:
        assert_o_close(o_gpu, o_state_ref, what + " (vs the oracle's bf16 state)", max_abs=2.0 ** -7, rel=2 * O_REL)
        assert_o_close(o_gpu, o_exact, what + " (vs the fp32 answer)", max_abs=2e-2, rel=6e-3)


def assert_lse_close(l_gpu, l_ref, what="", rel=LSE_REL):
    a = l_gpu.detach().float().cpu()
    b = l_ref.float()
    inf_a, inf_b = torch.isinf(a) & (a < 0), torch.isinf(b) & (b < 0)
    assert torch.equal(inf_a, inf_b), what + ": -inf pattern differs"
    fin = ~inf_b
    assert torch.isfinite(a[fin]).all(), what + ": non-finite LSE"
    err = ((a[fin] - b[fin]).abs() / b[fin].abs().clamp_min(1.0)).max().item() if fin.any() else 0.0
    assert err <= rel, "%s: LSE rel %.3e > %.1e" % (what, err, rel)


def decode_case(seed, B, Hq, Hkv, D, lens, pool, dtype=torch.float16, extra_req=2, pad_seq=5):
    """Token-indexed pool [pool, 2*Hkv, D] + req_to_token table with scattered slots."""
    g = torch.Generator().manual_seed(seed)
    q = rand_t((B, Hq, D), seed + 1, dtype)
    kv = rand_t((pool, 2 * Hkv, D), seed + 2, dtype)
    perm = torch.randperm(pool, generator=g).to(torch.int32)
    max_seq = max(max(lens), 1) + pad_seq
    table = torch.full((B + extra_req, max_seq), orc.INT32_PAD, dtype=torch.int32)
    b_req = torch.randperm(B + extra_req, generator=g)[:B].to(torch.int32)
    off = 0
    for b in range(B):
        table[int(b_req[b]), :lens[b]] = perm[off:off + lens[b]]
        off += lens[b]
    return q, kv, table, b_req, torch.tensor(lens, dtype=torch.int32)

"""Writes tests/golden/attention_known_answers.npz: small seeded inputs of the prefill step and of token-indexed decode with
their exact answers, computed here by plain float64 loops over the definition (numpy only, no oracle, no kernel, nothing of
the reference: it has no vectors for this path).  The fixture freezes those answers: tests/test_oracle_pins.py holds the
oracle to them, tests/test_gpu_golden.py the HIP kernels.

    python tests/golden/make_fixtures.py
"""
import math
import os

import numpy as np

D = 128


def _rand_half(rng, shape, scale=0.5):
    return (rng.standard_normal(shape) * scale).astype(np.float16)


def prefill_case(rng):
    """Two requests, striped positions (P = 2), GQA 4/2: row m of request b sits at global position q_first[b] + m P and sees
    key n of the chunk iff q_first[b] + m P >= kv_first[b] + n P (ring_context_flashattention_nopad.py:156-159)."""
    P, Hq, Hkv = 2, 4, 2
    q_len, kv_len = [37, 20], [33, 25]
    q_first, kv_first = [1, 0], [0, 1]
    q = _rand_half(rng, (sum(q_len), Hq, D))
    k = _rand_half(rng, (sum(kv_len), Hkv, D))
    v = _rand_half(rng, (sum(kv_len), Hkv, D))
    o = np.zeros((sum(q_len), Hq, D), dtype=np.float64)
    lse = np.full((sum(q_len), Hq), -np.inf, dtype=np.float64)
    scale = 1.0 / math.sqrt(D)
    qs = ks = 0
    for b in range(2):
        for m in range(q_len[b]):
            for h in range(Hq):
                g = h // (Hq // Hkv)
                keys = [n for n in range(kv_len[b]) if q_first[b] + m * P >= kv_first[b] + n * P]
                if not keys:
                    continue
                s = np.array([float(np.dot(q[qs + m, h].astype(np.float64), k[ks + n, g].astype(np.float64))) * scale for n in keys])
                mx = s.max()
                w = np.exp(s - mx)
                lse[qs + m, h] = mx + math.log(w.sum())
                o[qs + m, h] = sum(w[i] * v[ks + n, g].astype(np.float64) for i, n in enumerate(keys)) / w.sum()
        qs += q_len[b]
        ks += kv_len[b]
    return dict(pf_q=q, pf_k=k, pf_v=v, pf_q_len=np.array(q_len, np.int32), pf_kv_len=np.array(kv_len, np.int32),
                pf_q_first=np.array(q_first, np.int32), pf_kv_first=np.array(kv_first, np.int32), pf_peers=np.int32(P),
                pf_o=o, pf_lse=lse)


def decode_case(rng):
    """Two requests over a scattered pool [slots, 2 Hkv, D] (K heads, then V heads) through a request table."""
    Hq, Hkv, slots = 4, 2, 300
    lens = [50, 131]
    pool = _rand_half(rng, (slots, 2 * Hkv, D))
    q = _rand_half(rng, (2, Hq, D))
    perm = rng.permutation(slots).astype(np.int32)
    table = np.full((3, 140), 2147483647, dtype=np.int32)
    b_req = np.array([2, 0], dtype=np.int32)
    off = 0
    for b, n in enumerate(lens):
        table[b_req[b], :n] = perm[off:off + n]
        off += n
    o = np.zeros((2, Hq, D), dtype=np.float64)
    lse = np.zeros((2, Hq), dtype=np.float64)
    scale = 1.0 / math.sqrt(D)
    for b, n in enumerate(lens):
        for h in range(Hq):
            g = h // (Hq // Hkv)
            rows = table[b_req[b], :n]
            s = np.array([float(np.dot(q[b, h].astype(np.float64), pool[r, g].astype(np.float64))) * scale for r in rows])
            mx = s.max()
            w = np.exp(s - mx)
            lse[b, h] = mx + math.log(w.sum())
            o[b, h] = sum(w[i] * pool[r, Hkv + g].astype(np.float64) for i, r in enumerate(rows)) / w.sum()
    return dict(dc_q=q, dc_pool=pool, dc_table=table, dc_b_req=b_req, dc_b_len=np.array(lens, np.int32), dc_o=o, dc_lse=lse)


if __name__ == "__main__":
    rng = np.random.default_rng(20240)
    data = {}
    data.update(prefill_case(rng))
    data.update(decode_case(rng))
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_known_answers.npz")
    np.savez_compressed(out, **data)
    print("wrote", out, os.path.getsize(out), "bytes")

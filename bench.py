#!/usr/bin/env python3
"""Benchmark of the per-GPU attention hot path on one MI355X.

A step is one pass of the ring-prefill workload (BASELINE config 2): the 16384 queries of
shard 3 of a 131072-token sequence attend to KV shards 3 (causal), 0, 1, 2 (full), one
kernel launch per shard, then the fp32 partials are LSE-merged.  The same run also times
the token-indexed decode workload (config 3) and reports it next to the prefill number.
Inputs are synthetic (seeded N(0,1)*0.5) and resident in HBM before the timed region.

One JSON line goes to stdout; `--all` adds one (non-contract) line per other config.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_TFLOPS = 2500.0  # dense fp16/bf16 MFMA, MI355X
PEAK_HBM_GBS = 8000.0
DEV = "cuda:0"


def _randn_half(shape, seed, dtype=torch.float16, chunk_rows=1 << 18):
    """N(0,1)*0.5 in `dtype`, generated on the device in chunks (bounded fp32 scratch)."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    out = torch.empty(shape, dtype=dtype, device=DEV)
    flat = out.view(shape[0], -1)
    for r0 in range(0, shape[0], chunk_rows):
        r1 = min(shape[0], r0 + chunk_rows)
        flat[r0:r1] = (torch.randn((r1 - r0, flat.shape[1]), generator=g, device=DEV) * 0.5).to(dtype)
    return out


def _i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def _time_events(fn, steps, warmup):
    """Per-step wall times (ms) from HIP events on the stream the kernels are launched on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


# --------------------------------------------------------------------------------------
# config 2: ring prefill, shard 3 of 8 x 16384
# --------------------------------------------------------------------------------------
class RingPrefill:
    def __init__(self, shard=16384, n_shards_total=8, q_shard=3, heads=32, kv_heads=32, D=128, dtype=torch.float16, seed=2000):
        from loongserve_amd.simulate import KVChunk
        self.shard, self.q_shard, self.H, self.Hkv, self.D = shard, q_shard, heads, kv_heads, D
        self.q = _randn_half((shard, heads, D), seed, dtype)
        self.qs, self.ql, self.qf = _i32([0]), _i32([shard]), _i32([q_shard * shard])
        # ring order: local (diagonal) chunk first, then the shards that arrive over the ring
        self.order = [q_shard] + list(range(q_shard))
        self.chunks = []
        for j in self.order:
            kv = _randn_half((shard, 2 * kv_heads, D), seed + 1 + j, dtype)
            self.chunks.append(KVChunk(kv, _i32([0]), _i32([shard]), _i32([j * shard])))
        self.bufs = [(torch.empty((shard, heads, D), dtype=torch.float32, device=DEV),
                      torch.empty((shard, heads), dtype=torch.float32, device=DEV)) for _ in self.order]
        self.out = torch.empty((shard, heads, D), dtype=torch.float32, device=DEV)
        self.lse = torch.empty((shard, heads), dtype=torch.float32, device=DEV)
        n = shard
        self.pairs = q_shard * n * n + n * (n + 1) // 2
        self.flops = 4 * D * heads * self.pairs
        self.launches = len(self.order)

    def step(self):
        from loongserve_amd.simulate import ring_prefill_partials
        ring_prefill_partials(self.q, self.chunks, self.qs, self.ql, self.qf, 1, self.shard, self.Hkv, self.bufs, self.out, self.lse)

    def kernel_only(self):
        """The four attention launches without the merge (for the per-launch roofline figure)."""
        import loongserve_amd as lsa
        for c, (ob, lb) in zip(self.chunks, self.bufs):
            lsa.prefill_attention_step(self.q, c.k(self.Hkv), c.v(self.Hkv), self.qs, self.ql, self.qf, c.b_start_loc, c.b_seq_len,
                                       c.first_token_global_idx, 1, self.shard, ob, lb)

    def cpu_baseline(self, heads=4, rows=2048):
        """Oracle (PyTorch CPU fp32) on a slice: `heads` heads, the last `rows` query rows of the
        shard, against all four KV shards; scaled by algorithmic FLOPs."""
        from oracle import attn_oracle as orc
        torch.set_num_threads(os.cpu_count() or 1)
        n = self.shard
        q = self.q[n - rows:, :heads].cpu()
        qm = (torch.tensor([0], dtype=torch.int32), torch.tensor([rows], dtype=torch.int32),
              torch.tensor([self.q_shard * n + n - rows], dtype=torch.int32))
        parts_in = [(c.kv[:, :heads].cpu(), c.kv[:, self.Hkv:self.Hkv + heads].cpu(), c) for c in self.chunks]
        t0 = time.perf_counter()
        parts = []
        pairs = 0
        for (k, v, c), j in zip(parts_in, self.order):
            km = (torch.tensor([0], dtype=torch.int32), torch.tensor([n], dtype=torch.int32), torch.tensor([j * n], dtype=torch.int32))
            parts.append(orc.attn_step(q, k, v, *qm, *km, 1, q_chunk=512))
            pairs += rows * n if j != self.q_shard else sum(n - rows + i + 1 for i in range(rows))
        orc.lse_merge(parts)
        dt = time.perf_counter() - t0
        flops = 4 * self.D * heads * pairs
        return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": "config 2 slice: %d of %d heads, last %d of %d query rows of shard %d vs all 4 KV shards, "
                          "%.3f TFLOP in %.2f s (oracle/attn_oracle.py, PyTorch CPU fp32)" % (heads, self.H, rows, n, self.q_shard, flops / 1e12, dt)}


# --------------------------------------------------------------------------------------
# config 3: token-indexed decode, B=64, ctx U[4096, 32768], GQA 32/8
# --------------------------------------------------------------------------------------
class TokenDecode:
    def __init__(self, B=64, lo=4096, hi=32768, Hq=32, Hkv=8, D=128, pool=2_500_000, dtype=torch.float16, seed=3000, lens=None,
                 block_seq=None):
        g = torch.Generator().manual_seed(20243)
        self.lens = lens if lens is not None else torch.randint(lo, hi + 1, (B,), generator=g).tolist()
        self.B, self.Hq, self.Hkv, self.D = B, Hq, Hkv, D
        total = sum(self.lens)
        assert total <= pool
        self.kv = _randn_half((pool, 2 * Hkv, D), seed, dtype)
        self.q = _randn_half((B, Hq, D), seed + 1, dtype)
        perm = torch.randperm(pool, generator=g)[:total].to(torch.int32)
        self.max_len = max(self.lens)
        table = torch.full((B, self.max_len), 2147483647, dtype=torch.int32)
        off = 0
        for b, n in enumerate(self.lens):
            table[b, :n] = perm[off:off + n]
            off += n
        self.table = table.to(DEV)
        self.b_req = torch.arange(B, dtype=torch.int32, device=DEV)
        self.b_len = _i32(self.lens)
        from loongserve_amd.simulate import decode_block_seq
        self.BS = decode_block_seq(self.max_len) if block_seq is None else block_seq
        nblk = (self.max_len + self.BS - 1) // self.BS
        self.mid_o = torch.empty((nblk, B, Hq, D), dtype=torch.float32, device=DEV)
        self.mid_l = torch.empty((nblk, B, Hq), dtype=torch.float32, device=DEV)
        self.o = torch.empty((B, Hq, D), dtype=torch.float32, device=DEV)
        self.lse = torch.empty((B, Hq), dtype=torch.float32, device=DEV)
        # algorithmic bytes: K+V row per KV head + 4-byte index per token, plus q and the final outputs
        self.bytes = total * (2 * Hkv * D * 2 + 4) + self.q.numel() * 2 + self.o.numel() * 4 + self.lse.numel() * 4
        self.tokens = total

    def step(self):
        import loongserve_amd as lsa
        lsa.longserve_token_decode_attention_flash_decoding(self.q, self.table, self.b_req, self.b_len, self.mid_o, self.mid_l, self.B,
                                                            self.max_len, self.Hq, self.D, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:],
                                                            self.BS, self.o, self.lse)

    def stage1_only(self):
        import loongserve_amd as lsa
        lsa.longserve_flash_decode_stage1(self.q, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:], self.table, self.b_req, self.b_len,
                                          self.max_len, self.mid_o, self.mid_l, self.BS)

    def cpu_baseline(self, nreq=8):
        from oracle import attn_oracle as orc
        torch.set_num_threads(os.cpu_count() or 1)
        idx = list(range(nreq))
        lens = [self.lens[b] for b in idx]
        # hand the CPU exactly the rows it reads, re-indexed into a compact pool
        rows = torch.cat([self.table[b, :self.lens[b]] for b in idx]).long()
        kv = self.kv[rows].cpu()
        table = torch.full((nreq, max(lens)), 2147483647, dtype=torch.int32)
        off = 0
        for i, n in enumerate(lens):
            table[i, :n] = torch.arange(off, off + n, dtype=torch.int32)
            off += n
        q = self.q[:nreq].cpu()
        b_req = torch.arange(nreq, dtype=torch.int32)
        b_len = torch.tensor(lens, dtype=torch.int32)
        nblk = (max(lens) + self.BS - 1) // self.BS
        mid_o = torch.empty(nblk, nreq, self.Hq, self.D)
        mid_l = torch.empty(nblk, nreq, self.Hq)
        t0 = time.perf_counter()
        orc.token_decode_attention_flash_decoding(q, table, b_req, b_len, mid_o, mid_l, nreq, max(lens), self.Hq, self.D,
                                                  kv[:, :self.Hkv], kv[:, self.Hkv:], self.BS)
        dt = time.perf_counter() - t0
        nbytes = sum(lens) * (2 * self.Hkv * self.D * 2 + 4)
        return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
                "sample": "config 3 slice: first %d of %d requests (%d tokens), %.3f GB in %.2f s "
                          "(oracle/attn_oracle.py, PyTorch CPU fp32)" % (nreq, self.B, sum(lens), nbytes / 1e9, dt)}


def _stats(ms):
    s = sorted(ms)
    n = len(s)
    return {"median_ms": s[n // 2], "p10_ms": s[int(0.1 * (n - 1))], "p90_ms": s[int(math.ceil(0.9 * (n - 1)))], "mean_ms": sum(s) / n}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only", choices=["prefill", "decode"], default=None, help="time one workload only (profiling aid)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no second GPU); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import loongserve_amd  # noqa: F401  (raises if liblsattn.so is missing)
    torch.cuda.set_device(0)

    line = {
        "metric": "prefill attn TFLOP/s + decode KV GB/s, as % of MI355X roofline (1 GPU)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
    }

    if args.only != "decode":
        w = RingPrefill()
        torch.cuda.synchronize()
        step_ms = _time_events(w.step, args.steps, args.warmup)
        # wall clock around exactly K steps, bracketed by synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            w.step()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        kern_ms = _time_events(w.kernel_only, args.steps, 1)
        st = _stats(step_ms)
        tflops = w.flops / (wall_ms * 1e-3) / 1e12
        per_launch_ms = (sum(kern_ms) / len(kern_ms)) / w.launches
        ach = (w.flops / w.launches) / (per_launch_ms * 1e-3) / 1e12
        line.update({
            "value": tflops, "unit": "TFLOP/s", "ms_per_step": wall_ms,
            "pct_of_mfma_peak": 100.0 * tflops / PEAK_MFMA_TFLOPS,
            "config": {"workload": "config 2: ring prefill on one GPU, queries of shard 3 (16384 rows) of a 131072-token sequence vs KV "
                                   "shards 3 (causal), 0, 1, 2 (full) + LSE merge; 32 heads MHA, head_dim 128, fp16",
                       "algorithmic_tflop_per_step": w.flops / 1e12, "launches_per_step": w.launches + 1, "step_stats": st},
            "roofline": {"kernel": "prefill_kernel<F16,0>", "bound": "mfma", "achieved": ach, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                         "frac": ach / PEAK_MFMA_TFLOPS, "traffic": None,
                         "per_launch_ms": per_launch_ms, "algorithmic_tflop_per_launch": w.flops / w.launches / 1e12},
        })
        if not args.no_cpu:
            line["cpu_baseline"] = w.cpu_baseline()
        del w
        torch.cuda.empty_cache()

    if args.only != "prefill":
        d = TokenDecode()
        torch.cuda.synchronize()
        dsteps = max(args.steps, 10)
        d_ms = _time_events(d.step, dsteps, max(args.warmup, 2))
        s1_ms = _time_events(d.stage1_only, dsteps, 1)
        st = _stats(d_ms)
        gbs = d.bytes / (st["mean_ms"] * 1e-3) / 1e9
        s1 = sum(s1_ms) / len(s1_ms)
        ach = d.bytes / (s1 * 1e-3) / 1e9
        dec = {
            "value": gbs, "unit": "GB/s", "ms_per_step": st["mean_ms"], "pct_of_hbm_peak": 100.0 * gbs / PEAK_HBM_GBS,
            "config": {"workload": "config 3: token-indexed decode, batch 64, ctx U[4096,32768], GQA 32/8, head_dim 128, fp16, "
                                   "2.5M-slot scattered pool; stage1 (split-K, block_seq %d) + stage2" % d.BS,
                       "tokens": d.tokens, "algorithmic_gb_per_step": d.bytes / 1e9, "step_stats": st},
            "roofline": {"kernel": "decode_stage1_kernel<F16,4,4>", "bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": ach / PEAK_HBM_GBS, "traffic": None, "per_launch_ms": s1},
        }
        if not args.no_cpu:
            dec["cpu_baseline"] = d.cpu_baseline()
        if args.only == "decode":
            line.update({"value": gbs, "unit": "GB/s", "ms_per_step": st["mean_ms"], "config": dec["config"], "roofline": dec["roofline"]})
            if "cpu_baseline" in dec:
                line["cpu_baseline"] = dec["cpu_baseline"]
        else:
            line["decode"] = dec
    print(json.dumps(line))


if __name__ == "__main__":
    main()

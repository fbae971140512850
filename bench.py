#!/usr/bin/env python3
"""Benchmark of the per-GPU attention hot path on one MI355X.

A step is one pass of the ring-prefill workload (baseline configuration 2 of five): the 16384 queries of
shard 3 of a 131072-token sequence attend to KV shards 3 (causal), 0, 1, 2 (full), one
kernel launch per shard, each later launch LSE-merging its partial into the running result.
The same run times the token-indexed decode workload (config 3), the other three baseline configs (1, 4, 5), a
few batches of short prompts, and what the box sustains with nothing in the way (a stream of fp16 MFMAs on random
operands, a streaming read of 4 GiB: libls_ceiling.so), so that every fraction of the nominal peak stands beside the
fraction of what this box delivered in this run.
Inputs are synthetic (seeded N(0,1)*0.5) and resident in HBM before the timed region.

One compact JSON line goes to stdout: the headline (config 2) with `roofline` and `cpu_baseline`, which also carry the
scalar figures of decode and of configs 1, 4, 5, and a `summary` of all five configs as the last key.
`--sweeps` also times the launch-size, decode-latency, large-group and mixed-length sweeps and `--all` the steps around
attention; both go to the file `--details-out` names (default gpurun_out/bench_details.json), not into the line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of each workload's dominant kernel: rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the same
# counter reads for a plain copy of 1 GiB.  Not measured by this run: taken from profiles/bench_default_hbm_traffic.txt,
# which is regenerated with the kernels (the JSON line says so in "traffic_source").
TRAFFIC_SOURCE = "profiles/bench_default_hbm_traffic.txt (rocprofv3 --pmc, scaled by a 1 GiB copy); constants of bench.py, not measured in this run"
TRAFFIC_BYTES = {
    "config2": 1305.9e6,    # per launch, averaged over the four launches of a ring step (one diagonal + three full)
    "config3": 5186.9e6,    # the fused call: stage 1 in equal shares (5180.2) + the merge behind it (6.7)
    "config1": 92.6e6,
    "config4": 8614.1e6,    # stage 1 over one instance's 4 x 131072 tokens
    "config5": 104980.5e6,    # the attention launch (K/V re-fetched from HBM about 25 times)
    "decode_8_1": 657.6e6,  # stage 1 of the large-group cases
    "decode_16_2": 1308.9e6,
    "decode_64_8": 5222.4e6,
}
PEAK_MFMA_TFLOPS = 2500.0  # dense fp16/bf16 MFMA, MI355X
PEAK_HBM_GBS = 8000.0
DEV = "cuda:0"
D = 128  # head_dim of every workload here


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


def _time_graph(fn, launches=20, reps=10, warm_reps=2, every=False):
    """Device time (ms) of one call of `fn`, for calls too short to time from the host: `launches` calls are recorded
    into one HIP graph, whose replays are timed with HIP events; `warm_reps` replays are thrown away, then the median
    over `reps` replays, per call (every=True: the list of all of them)."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(launches):
            fn()
    # warm-up: at least warm_reps replays and at least 50 ms of them (a GPU that has sat idle, as during the CPU baseline,
    # takes a while to bring its clocks up, and a graph of short launches is over before it has)
    t0 = time.perf_counter()
    n_warm = 0
    while n_warm < max(1, warm_reps) or (time.perf_counter() - t0 < 0.05 and n_warm < 2000):
        g.replay()
        n_warm += 1
        if n_warm % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b) / launches)
    return ts if every else sorted(ts)[len(ts) // 2]


def _r(x, nd=4):
    return None if x is None else round(float(x), nd)


class Ceiling:
    """What this box sustains with nothing in the way (libls_ceiling.so, include/ls_ceiling.h)."""

    def __init__(self):
        path = os.path.join(ROOT, "loongserve_amd", "libls_ceiling.so")
        if not os.path.exists(path):
            raise RuntimeError("bench.py: %s is missing; build it with `python -m loongserve_amd.build`" % path)
        self.lib = ctypes.CDLL(path)
        vp = ctypes.c_void_p
        self.lib.ls_ceiling_mfma_f16.restype = ctypes.c_int
        self.lib.ls_ceiling_mfma_f16.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp]
        self.lib.ls_ceiling_mfma_f16_flop.restype = ctypes.c_double
        self.lib.ls_ceiling_mfma_f16_flop.argtypes = [ctypes.c_int, ctypes.c_int]
        self.lib.ls_ceiling_read.restype = ctypes.c_int
        self.lib.ls_ceiling_read.argtypes = [vp, ctypes.c_uint64, vp, vp]
        self.lib.ls_ceiling_read_with_stores.restype = ctypes.c_int
        self.lib.ls_ceiling_read_with_stores.argtypes = [vp, ctypes.c_uint64, vp, ctypes.c_uint32, ctypes.c_int, vp, vp]
        self.lib.ls_ceiling_read_with_stores_bytes.restype = ctypes.c_uint64
        self.lib.ls_ceiling_read_with_stores_bytes.argtypes = [ctypes.c_uint64, ctypes.c_uint32]

    def mfma_tflops(self, iters=60000, workgroups=256, launches=24, warm=8):
        """A stream of v_mfma_f32_16x16x32_f16 on random fp16 operands, one wave per SIMD, nothing else; launches of
        about 10 ms back to back, the first `warm` thrown away (the clock settles under the power limit), the median."""
        ops = _randn_half((1024, 128), 8001)  # 256 KiB of N(0,1)*0.5 fp16 values
        sink = torch.zeros(256 * workgroups, dtype=torch.float32, device=DEV)
        st = torch.cuda.current_stream().cuda_stream

        def call():
            if self.lib.ls_ceiling_mfma_f16(ops.data_ptr(), sink.data_ptr(), iters, workgroups, st) != 0:
                raise RuntimeError("ls_ceiling_mfma_f16 failed")
        ms = _time_events(call, launches, warm)
        flop = self.lib.ls_ceiling_mfma_f16_flop(iters, workgroups)
        med = sorted(ms)[len(ms) // 2]
        return flop / (med * 1e-3) / 1e12, med

    def read_gbs(self, nbytes=4 << 30, launches=20, warm=5):
        """A plain streaming read of 4 GiB (16 bytes per lane and load, non-temporal), the median launch."""
        src = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        src.view(torch.int32).random_(0, 1 << 30)
        sink = torch.zeros(256, dtype=torch.int32, device=DEV)
        st = torch.cuda.current_stream().cuda_stream

        def call():
            if self.lib.ls_ceiling_read(src.data_ptr(), nbytes, sink.data_ptr(), st) != 0:
                raise RuntimeError("ls_ceiling_read failed")
        ms = _time_events(call, launches, warm)
        med = sorted(ms)[len(ms) // 2]
        del src
        torch.cuda.empty_cache()
        return nbytes / (med * 1e-3) / 1e9, med


    def read_with_stores_gbs(self, every=64, nbytes=4 << 30, launches=20, warm=5):
        """The same read with 8 KB stores mixed into one of every `every` trips of a wave (64: 1.6 % of the bytes, what one
        fp32 partial per 256 tokens is to config 3's gather): GB/s of the read with ordinary stores and with stores that
        are written through to memory as they are issued (what the decode kernel's partials use)."""
        src = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        src.view(torch.int32).random_(0, 1 << 30)
        dst = torch.empty(int(self.lib.ls_ceiling_read_with_stores_bytes(nbytes, every)), dtype=torch.uint8, device=DEV)
        sink = torch.zeros(256, dtype=torch.int32, device=DEV)
        st = torch.cuda.current_stream().cuda_stream
        out = []
        for system_scope in (0, 1):
            def call():
                if self.lib.ls_ceiling_read_with_stores(src.data_ptr(), nbytes, dst.data_ptr(), every, system_scope, sink.data_ptr(), st) != 0:
                    raise RuntimeError("ls_ceiling_read_with_stores failed")
            ms = _time_events(call, launches, warm)
            out.append(nbytes / (sorted(ms)[len(ms) // 2] * 1e-3) / 1e9)
        del src, dst
        torch.cuda.empty_cache()
        return out[0], out[1], 1.0 / every


def _roof(kernel, bound, achieved, per_launch_ms, traffic_key, **extra):
    peak = PEAK_MFMA_TFLOPS if bound == "mfma" else PEAK_HBM_GBS
    r = {"kernel": kernel, "bound": bound, "achieved": achieved, "peak": peak, "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
         "frac": achieved / peak, "traffic": TRAFFIC_BYTES.get(traffic_key), "traffic_source": TRAFFIC_SOURCE,
         "per_launch_ms": per_launch_ms}
    r.update(extra)
    return r


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
        self.bufs = None  # per-step partial buffers, only for the separate-merge route
        self.state = None  # (o, m, l) of the in-place route
        self.out = torch.empty((shard, heads, D), dtype=torch.float32, device=DEV)
        self.lse = torch.empty((shard, heads), dtype=torch.float32, device=DEV)
        n = shard
        self.pairs = q_shard * n * n + n * (n + 1) // 2
        self.flops = 4 * D * heads * self.pairs
        self.launches = len(self.order)

    def step(self):
        """Four launches in ring order; the first writes the fp32 partial (O, LSE) of the diagonal step, each later one
        LSE-merges its own partial into it in its epilogue."""
        from loongserve_amd.simulate import ring_prefill_accumulate
        ring_prefill_accumulate(self.q, self.chunks, self.qs, self.ql, self.qf, 1, self.shard, self.Hkv, self.out, self.lse)

    def step_in_place(self):
        """The same four steps through context_attention_fwd, the reference's operator: (o fp16, m, l) updated in place."""
        from loongserve_amd.simulate import ring_prefill
        if self.state is None:
            self.state = (torch.empty_like(self.q), torch.empty((self.shard, self.H), dtype=torch.float32, device=DEV),
                          torch.empty((self.shard, self.H), dtype=torch.float32, device=DEV))
        ring_prefill(self.q, self.chunks, self.qs, self.ql, self.qf, 1, self.shard, self.Hkv, *self.state)

    def step_separate_merge(self):
        """The same four steps as four separate fp32 partials and one lsattn_lse_merge pass over them."""
        from loongserve_amd.simulate import ring_prefill_partials
        if self.bufs is None:
            self.bufs = [(torch.empty((self.shard, self.H, self.D), dtype=torch.float32, device=DEV),
                          torch.empty((self.shard, self.H), dtype=torch.float32, device=DEV)) for _ in self.order]
        ring_prefill_partials(self.q, self.chunks, self.qs, self.ql, self.qf, 1, self.shard, self.Hkv, self.bufs, self.out, self.lse)

    def cpu_baseline(self, heads=16, rows=6144):
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
        # the fused call splits the context more coarsely than BLOCK_SEQ between its two stages (mid_o is scratch there)
        from loongserve_amd.decoding import _fused_block_seq
        self.split = _fused_block_seq(self.BS, B, self.max_len, Hkv)
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

    def step_separate_stages(self):
        """Stage 1 and stage 2 as two calls at BLOCK_SEQ, the way the master of a decode step makes them
        (longserve_transformer_layer_infer.py:272-281, :360-367)."""
        import loongserve_amd as lsa
        lsa.longserve_flash_decode_stage1(self.q, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:], self.table, self.b_req, self.b_len,
                                          self.max_len, self.mid_o, self.mid_l, self.BS)
        lsa.longserve_flash_decode_stage2(self.mid_o, self.mid_l, self.b_len, self.o, self.lse, self.BS)

    def step_separate_stages_merged(self):
        """The same two calls with groups of blocks merged into one partial by stage 1 (the opt-in layout)."""
        from loongserve_amd import decoding
        decoding.STAGE1_MERGES_BLOCKS = True
        try:
            self.step_separate_stages()
        finally:
            decoding.STAGE1_MERGES_BLOCKS = False

    def stage1_only(self):
        import loongserve_amd as lsa
        lsa.longserve_flash_decode_stage1(self.q, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:], self.table, self.b_req, self.b_len,
                                          self.max_len, self.mid_o, self.mid_l, self.split)

    def cpu_baseline(self, nreq=64):
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


# --------------------------------------------------------------------------------------
# config 4: long-context elastic decode, B=4 x 524288, MHA 32, 4 simulated instances
# --------------------------------------------------------------------------------------
class ElasticDecode:
    def __init__(self, B=4, ctx=524288, H=32, D=128, n_inst=4, pool=2_200_000, dtype=torch.float16, seed=4000):
        from loongserve_amd.simulate import DecodeInstance
        g = torch.Generator().manual_seed(20244)
        self.B, self.H, self.D, self.ctx, self.n_inst = B, H, D, ctx, n_inst
        total = B * ctx
        assert total <= pool
        self.kv = _randn_half((pool, 2 * H, D), seed, dtype, chunk_rows=1 << 15)
        self.q = _randn_half((B, H, D), seed + 1, dtype)
        self.perm = torch.randperm(pool, generator=g)[:total].to(torch.int32).view(B, ctx)
        part = ctx // n_inst
        self.b_req = torch.arange(B, dtype=torch.int32, device=DEV)
        self.instances = []
        for r in range(n_inst):
            table = self.perm[:, r * part:(r + 1) * part].contiguous().to(DEV)
            self.instances.append(DecodeInstance(self.kv, table, self.b_req, _i32([part] * B), part))
        self.full_table = self.perm.to(DEV)
        self.ws = {}
        self.out = torch.empty((B, H, D), dtype=dtype, device=DEV)
        self.bytes = total * (2 * H * D * 2 + 4) + self.q.numel() * 2 + self.out.numel() * 2 + B * H * 4
        self.tokens = total

    def step(self):
        from loongserve_amd.simulate import multi_instance_decode
        return multi_instance_decode(self.q, self.instances, self.H, out=self.out, workspace=self.ws)

    def stage1_of_one_instance(self):
        """Stage 1 alone over the 4 x 131072 tokens of one instance, at the split the fused call uses there."""
        import loongserve_amd as lsa
        from loongserve_amd.decoding import _fused_block_seq
        from loongserve_amd.simulate import decode_block_seq
        inst = self.instances[1]
        part = self.ctx // self.n_inst
        if not hasattr(self, "s1"):
            split = _fused_block_seq(decode_block_seq(part), self.B, part, self.H)
            nblk = (part + split - 1) // split
            self.s1 = (split, torch.empty((nblk, self.B, self.H, self.D), dtype=torch.float32, device=DEV),
                       torch.empty((nblk, self.B, self.H), dtype=torch.float32, device=DEV), _i32([part] * self.B))
        split, mo, ml, blen = self.s1
        lsa.longserve_cuda_kernels.flash_decoding_stage1(mo, ml, self.q, self.kv[:, :self.H], self.kv[:, self.H:], inst.req_to_token,
                                                         self.b_req, blen, part, split)
        return part * self.B * (2 * self.H * self.D * 2 + 4)


# --------------------------------------------------------------------------------------
# config 5: mixed varlen prefill, 24 sequences log-uniform in [1024, 200000], GQA 32/8, bf16,
# K/V rows scattered to pool slots and registered during the pass
# --------------------------------------------------------------------------------------
class VarlenPrefill:
    def __init__(self, n_seq=24, lo=1024, hi=200000, Hq=32, Hkv=8, D=128, dtype=torch.bfloat16, seed=5000, lens=None):
        g = torch.Generator().manual_seed(20245)
        if lens is None:
            u = torch.rand(n_seq, generator=g, dtype=torch.float64)
            lens = torch.round(torch.exp(math.log(lo) + u * (math.log(hi) - math.log(lo)))).to(torch.int64).tolist()
        self.lens, self.Hq, self.Hkv, self.D = lens, Hq, Hkv, D
        T = sum(lens)
        self.T = T
        self.q = _randn_half((T, Hq, D), seed, dtype, chunk_rows=1 << 16)
        self.kv = _randn_half((T, 2 * Hkv, D), seed + 1, dtype)
        self.o = torch.empty((T, Hq, D), dtype=dtype, device=DEV)
        self.m = torch.empty((T, Hq), dtype=torch.float32, device=DEV)
        self.l = torch.empty((T, Hq), dtype=torch.float32, device=DEV)
        lens_t = torch.tensor(lens, dtype=torch.int64)
        self.start = (torch.cumsum(lens_t, 0) - lens_t).to(torch.int32).to(DEV)
        self.len = lens_t.to(torch.int32).to(DEV)
        self.first = torch.zeros(n_seq if lens is None else len(lens), dtype=torch.int32, device=DEV)
        self.max_len = max(lens)
        pool_slots = T + 4096
        self.pool = torch.zeros((pool_slots, 2 * Hkv, D), dtype=dtype, device=DEV)
        self.mem_index = torch.randperm(pool_slots, generator=g)[:T].to(torch.int32).to(DEV)
        self.b_req = torch.arange(len(lens), dtype=torch.int32, device=DEV)
        self.req_to_token = torch.full((len(lens), self.max_len), 2147483647, dtype=torch.int32, device=DEV)
        self.pairs = sum(n * (n + 1) // 2 for n in lens)
        self.flops = 4 * D * Hq * self.pairs
        self.scatter_bytes = T * 2 * Hkv * D * 2 * 2  # read + write of every K/V row
        self.v_f16 = torch.empty((T, Hkv, D), dtype=torch.float16, device=DEV)  # the caller's buffer for the fp16 copy of V
        self.bound_rows = True  # pass total_q_len = the rows of the packed q (the batch is skewed: 1 K to 200 K tokens)

    def attention(self):
        import loongserve_amd as lsa
        self.m.fill_(float("-inf"))
        self.l.zero_()
        lsa.context_attention_fwd(self.q, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:], self.o, self.start, self.len, self.first,
                                  self.start, self.len, self.first, 1, self.max_len, self.m, self.l, v_f16=self.v_f16,
                                  total_q_len=self.T if self.bound_rows else None)

    def attention_kernel_only(self):
        """The attention launch alone: (m, l) not reset (the result is not used), V's fp16 copy taken as it stands."""
        import loongserve_amd as lsa
        lsa.context_attention_fwd(self.q, self.kv[:, :self.Hkv], self.kv[:, self.Hkv:], self.o, self.start, self.len, self.first,
                                  self.start, self.len, self.first, 1, self.max_len, self.m, self.l, v_f16=self.v_f16,
                                  v_f16_valid=True, total_q_len=self.T if self.bound_rows else None)

    def persist(self):
        import loongserve_amd as lsa
        lsa.kv_scatter(self.kv, self.mem_index, self.pool)
        lsa.init_req_to_token_indexes(self.req_to_token, self.b_req, self.len, self.mem_index, self.start, self.max_len)

    def migrate(self):
        """The same rows through the context-migration path: every sequence hands over all its rows
        (ranges [0, len)), copy + registration fused in one launch."""
        import loongserve_amd as lsa
        if not hasattr(self, "len_sum"):
            self.len_sum = torch.cumsum(self.len, 0, dtype=torch.int64)
            self.zero = torch.zeros_like(self.len)
        lsa.destindex_copy_and_register_kv(len(self.lens), self.len, self.zero, self.len, self.len_sum, self.kv, self.start, self.zero,
                                           self.mem_index, self.pool, self.req_to_token, self.b_req, 0, self.max_len, True)

    def write_back_setup(self):
        """The write-back of the step's tokens (rotary of q and k, K/V rows to their pool slots, registration) runs in
        fp16, as the reference's rotary kernel does: the same buffers are read as fp16 bit patterns (timing only, the
        rotation overwrites q and k)."""
        self.q16, self.kv16, self.pool16 = self.q.view(torch.float16), self.kv.view(torch.float16), self.pool.view(torch.float16)
        self.cos = _randn_half((self.T, self.D // 2), 5101, torch.float16)
        self.sin = _randn_half((self.T, self.D // 2), 5102, torch.float16)
        # bytes the fused launch has to move: q read + written, K/V rows read, K written back in place, pool rows written,
        # cos/sin read, slot numbers read, table written
        self.write_back_bytes = self.T * (2 * self.Hq * self.D * 2 + 2 * self.Hkv * self.D * 2 + self.Hkv * self.D * 2
                                          + 2 * self.Hkv * self.D * 2 + 2 * (self.D // 2) * 2 + 8)

    def write_back_separate(self):
        import loongserve_amd as lsa
        lsa.longserve_cuda_kernels.rotary_emb(self.q16, self.kv16[:, :self.Hkv], self.cos, self.sin)
        lsa.kv_scatter(self.kv16, self.mem_index, self.pool16)
        lsa.init_req_to_token_indexes(self.req_to_token, self.b_req, self.len, self.mem_index, self.start, self.max_len)

    def write_back_fused(self):
        import loongserve_amd as lsa
        lsa.rotary_emb_write_kv(self.q16, self.kv16, self.cos, self.sin, self.mem_index, self.pool16, self.req_to_token, self.b_req,
                                self.len, self.start, self.max_len)

    def step(self):
        self.attention()
        self.persist()


def _stats(ms):
    s = sorted(ms)
    n = len(s)
    return {"median_ms": s[n // 2], "p10_ms": s[int(0.1 * (n - 1))], "p90_ms": s[int(math.ceil(0.9 * (n - 1)))], "mean_ms": sum(s) / n}


def config1():
    """Config 1: single causal prefill, 2048 tokens, 32/32 heads, fp16, one ring step, one launch."""
    import loongserve_amd as lsa
    T, H = 2048, 32
    q, kv = _randn_half((T, H, D), 1001), _randn_half((T, 2 * H, D), 1002)
    s0, ln, f0 = _i32([0]), _i32([T]), _i32([0])
    ob = torch.empty((T, H, D), dtype=torch.float32, device=DEV)
    lb = torch.empty((T, H), dtype=torch.float32, device=DEV)
    call = lambda: lsa.prefill_attention_step(q, kv[:, :H], kv[:, H:], s0, ln, f0, s0, ln, f0, 1, T, ob, lb)  # noqa: E731
    eager = _stats(_time_events(call, 50, 10))
    # device time per launch: 20 launches recorded in one HIP graph (the launch is shorter than the host's call), 12 replays
    st = _stats(_time_graph(call, launches=20, reps=12, warm_reps=3, every=True))
    fl = 4 * D * H * (T * (T + 1) // 2)
    ms = st["median_ms"]
    return {"workload": "config 1: 1 x 2048 tokens causal, MHA 32, fp16, fp32 (O, LSE) out, one launch",
            "value": fl / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms": ms, "p10_ms": st["p10_ms"], "p90_ms": st["p90_ms"],
            "frac": fl / (ms * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "kernel": "prefill_kernel<F16,0,true,false,true> (four-wave 128-row workgroups, two per CU, folded grid)",
            "timing": "per launch, 20 launches in a HIP graph x 12 replays", "eager_call_ms": eager["median_ms"],
            "algorithmic_tflop": fl / 1e12, "traffic": TRAFFIC_BYTES["config1"]}


def config4():
    """Config 4: long-context elastic decode, 4 x 524288, MHA 32, four instances, merge at the master."""
    e = ElasticDecode()
    st = _stats(_time_events(e.step, 50, 10))
    nbytes1 = e.stage1_of_one_instance()
    s1 = _stats(_time_events(e.stage1_of_one_instance, 50, 10))
    gbs1 = nbytes1 / (s1["median_ms"] * 1e-3) / 1e9
    out = {"workload": "config 4: decode 4 x 524288 tokens, MHA 32, fp16, scattered pool; 4 simulated instances (3 peers fused, "
                       "master stage 1 + block_seq=1 merge of all partials)",
           "value": e.bytes / (st["median_ms"] * 1e-3) / 1e9, "unit": "GB/s", "ms": st["median_ms"], "p10_ms": st["p10_ms"],
           "p90_ms": st["p90_ms"], "frac": e.bytes / (st["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
           "kernel": "decode_stage1_mfma_kernel<F16,false>", "kernel_ms": s1["median_ms"], "kernel_gbs": gbs1,
           "kernel_frac": gbs1 / PEAK_HBM_GBS, "algorithmic_gb": e.bytes / 1e9, "kernel_algorithmic_gb": nbytes1 / 1e9,
           "traffic": TRAFFIC_BYTES["config4"]}
    del e
    torch.cuda.empty_cache()
    return out


def config5(details=None):
    """Config 5: mixed varlen prefill, bf16, GQA 32/8, K/V rows written to pool slots and registered."""
    v = VarlenPrefill()
    sa = _stats(_time_events(v.attention, 5, 1))
    sk = _stats(_time_events(v.attention_kernel_only, 5, 1))
    sp = _stats(_time_events(v.persist, 20, 3))
    whole_ms = sa["median_ms"] + sp["median_ms"]
    tf = v.flops / (sk["median_ms"] * 1e-3) / 1e12
    out = {"workload": "config 5: 24 packed sequences, lengths log-uniform in [1024, 200000], %d tokens, GQA 32/8, bf16, causal, "
                       "context_attention_fwd ((m, l) reset, fp16 copy of V, one launch, total_q_len = the rows of q) + K/V rows to "
                       "pool slots + registration" % v.T,
           "value": v.flops / (whole_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms": whole_ms,
           "frac": v.flops / (whole_ms * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "kernel": "prefill_kernel<BF16,1,true,false>",
           "kernel_ms": sk["median_ms"], "kernel_p10_ms": sk["p10_ms"], "kernel_p90_ms": sk["p90_ms"], "kernel_tflops": tf,
           "kernel_frac": tf / PEAK_MFMA_TFLOPS, "kv_write_ms": sp["median_ms"],
           "kv_write_gbs": v.scatter_bytes / (sp["median_ms"] * 1e-3) / 1e9, "algorithmic_tflop": v.flops / 1e12,
           "traffic": TRAFFIC_BYTES["config5"]}
    if details is not None:
        sm = _stats(_time_events(v.migrate, 10, 2))
        v.write_back_setup()
        wsep = _stats(_time_events(v.write_back_separate, 10, 2))
        wfus = _stats(_time_events(v.write_back_fused, 10, 2))
        details["config5_write_back"] = {
            "what": "rotary of q and k + K/V rows to their pool slots + registration on the same buffers read as fp16: the "
                    "layer's four launches against lsattn_rotary_kv_write; the rows through lsattn_kv_copy_register",
            "separate_ms": wsep["median_ms"], "fused_ms": wfus["median_ms"], "bytes": v.write_back_bytes,
            "fused_gbs": v.write_back_bytes / (wfus["median_ms"] * 1e-3) / 1e9,
            "migration_copy_register_ms": sm["median_ms"], "migration_copy_register_gbs": v.scatter_bytes / (sm["median_ms"] * 1e-3) / 1e9}
    del v
    torch.cuda.empty_cache()
    return out


def _causal_case(N, Hq, Hkv, B):
    """A batch of B causal prompts of N tokens: the fp32-partial call, the reference operator's in-place call on rows in
    their start state with the call that resets them (m = -inf, l = 0), flops, and the bytes either route has to move."""
    q = _randn_half((B * N, Hq, D), 4100 + N + B)
    kv = _randn_half((B * N, 2 * Hkv, D), 4200 + N + B)
    st = torch.arange(B, dtype=torch.int32, device=DEV) * N
    ln = torch.full((B,), N, dtype=torch.int32, device=DEV)
    z = torch.zeros(B, dtype=torch.int32, device=DEV)
    o = torch.empty((B * N, Hq, D), dtype=torch.float32, device=DEV)
    lse = torch.empty((B * N, Hq), dtype=torch.float32, device=DEV)
    o16 = torch.zeros((B * N, Hq, D), dtype=torch.float16, device=DEV)
    m = torch.full((B * N, Hq), float("-inf"), device=DEV)
    l = torch.zeros((B * N, Hq), device=DEV)
    import loongserve_amd as lsa
    fn = lambda: lsa.prefill_attention_step(q, kv[:, :Hkv], kv[:, Hkv:], st, ln, z, st, ln, z, 1, N, out=o, lse=lse, kv_splits=1)  # noqa: E731

    def reset():
        m.fill_(float("-inf"))
        l.zero_()

    def inplace():
        reset()
        lsa.context_attention_fwd(q, kv[:, :Hkv], kv[:, Hkv:], o16, st, ln, z, st, ln, z, 1, N, m, l)

    rows = B * N * Hq
    bytes_partial = 2 * (q.numel() + kv.numel()) + 4 * rows * (D + 1)
    bytes_inplace = 2 * (q.numel() + kv.numel()) + 2 * rows * D + 4 * 4 * rows  # (o written, m and l read and written)
    return fn, 4.0 * D * Hq * B * N * (N + 1) / 2, inplace, reset, bytes_partial, bytes_inplace


def short_prompts():
    """Batches of short prompts (outside the five configs; the regime of the reference's published 1 x 100 / 1 x 1000
    token rows): causal, fp16, device time per launch from a HIP graph of 20 launches, median of 10 replays.  `us` is the
    fp32-partial call, `inplace_us` the reference's operator (o in fp16, (m, l) in place) on rows in their start state,
    with the time of the two fills that reset them taken off.  The smaller launches move more bytes than they
    compute: `hbm_frac` is the bytes either route has to move over 8 TB/s against its time, `frac` the MFMA fraction."""
    rows = {}
    for name, (N, Hq, Hkv, B) in (("16x256_mha", (256, 32, 32, 16)), ("8x512_gqa", (512, 32, 8, 8)), ("32x1024_gqa", (1024, 32, 8, 32)),
                                  ("6x2048_gqa", (2048, 32, 8, 6)), ("1x4096_mha", (4096, 32, 32, 1)), ("1x8192_gqa", (8192, 32, 8, 1))):
        fn, fl, inplace, reset, by_p, by_i = _causal_case(N, Hq, Hkv, B)
        ms = _time_graph(fn, launches=20, reps=10, warm_reps=3)
        ms_i = _time_graph(inplace, launches=20, reps=10, warm_reps=3) - _time_graph(reset, launches=20, reps=10, warm_reps=3)
        rows[name] = {"us": _r(ms * 1e3, 1), "frac": _r(fl / (ms * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS),
                      "hbm_frac": _r(by_p / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS), "inplace_us": _r(ms_i * 1e3, 1),
                      "inplace_frac": _r(fl / (ms_i * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS),
                      "inplace_hbm_frac": _r(by_i / (ms_i * 1e-3) / 1e9 / PEAK_HBM_GBS)}
        torch.cuda.empty_cache()
    return rows


def chunked_prefill_step():
    """A chunked-prefill step of a long request (outside the five configs): 100 query rows against a KV chunk of 131072
    keys, GQA 32/8, fp16, all keys visible.  Through prefill_attention_step (fp32 partial, KV cut chosen by the library),
    through the reference's operator context_attention_fwd with a caller workspace (the same cut, folded into (o, m, l)),
    and through context_attention_fwd as the reference calls it (no workspace: one workgroup per 128 rows and head).
    Device time per call from a HIP graph of 10 calls, median of 10 replays."""
    import loongserve_amd as lsa
    Tq, Tk, Hq, Hkv = 100, 131072, 32, 8
    q = _randn_half((Tq, Hq, D), 4601)
    kv = _randn_half((Tk, 2 * Hkv, D), 4602)
    qm = (_i32([0]), _i32([Tq]), _i32([Tk]))
    km = (_i32([0]), _i32([Tk]), _i32([0]))
    o32 = torch.empty((Tq, Hq, D), dtype=torch.float32, device=DEV)
    l32 = torch.empty((Tq, Hq), dtype=torch.float32, device=DEV)
    o16 = torch.zeros((Tq, Hq, D), dtype=torch.float16, device=DEV)
    m = torch.full((Tq, Hq), float("-inf"), device=DEV)
    l = torch.zeros((Tq, Hq), device=DEV)
    from loongserve_amd.ops import kv_split_count
    S = kv_split_count(1, Hq, Tq, Tk, Hkv)
    ws = torch.empty(S * Tq * Hq * (D + 1), dtype=torch.float32, device=DEV)
    step = lambda: lsa.prefill_attention_step(q, kv[:, :Hkv], kv[:, Hkv:], *qm, *km, 1, Tq, out=o32, lse=l32, kv_split_workspace=ws)  # noqa: E731
    op_ws = lambda: lsa.context_attention_fwd(q, kv[:, :Hkv], kv[:, Hkv:], o16, *qm, *km, 1, Tq, m, l, workspace=ws)  # noqa: E731
    op = lambda: lsa.context_attention_fwd(q, kv[:, :Hkv], kv[:, Hkv:], o16, *qm, *km, 1, Tq, m, l)  # noqa: E731
    out = {"workload": "100 query rows x 131072 keys, GQA 32/8, fp16", "kv_cuts": S}
    for key, fn in (("prefill_attention_step_us", step), ("context_attention_fwd_workspace_us", op_ws), ("context_attention_fwd_us", op)):
        out[key] = _r(_time_graph(fn, launches=10, reps=10, warm_reps=2) * 1e3, 1)
    gb = Tk * 2 * Hkv * D * 2 / 1e9
    out["kv_gbs_workspace_route"] = _r(gb / (out["context_attention_fwd_workspace_us"] * 1e-6), 0)
    torch.cuda.empty_cache()
    return out


def _tiles_256x64(N, Hq, B, pack=1):
    """64-key tiles that 256-row workgroups walk for B causal sequences of N tokens (pack query heads side by side)."""
    rows = 256 // pack
    nz = (N + rows - 1) // rows
    return B * (Hq // pack) * sum(min((z + 1) * rows, N) // 64 + (1 if min((z + 1) * rows, N) % 64 else 0) for z in range(nz))


def prefill_launch_sizes(tile_us):
    """Causal prefill launches from a quarter of a round of workgroups to a few rounds (outside the five baseline configs):
    fp16, head_dim 128, fp32 (O, LSE) out, device time per launch from a HIP graph of 20 launches, median of 10 replays.
    chosen_us is the library's own choice of workgroup height and grid order; the other columns force 128-row workgroups,
    256-row workgroups one KV head at a time per XCD, 256-row workgroups with the heaviest query tiles of all heads
    first, the four-wave shape of which two workgroups share a CU, and one query head per workgroup instead of the heads
    of a KV head side by side (lsattn_set_tuning).  tiles_only_floor_us: the 64-key tiles that 256-row workgroups walk,
    spread evenly over 256 CUs, at the rate per tile that config 2's full launches ran at in this run: what the launch
    would take if workgroups cost nothing besides their tiles."""
    import loongserve_amd as lsa
    rows = []
    try:
        for N, Hq, Hkv, B in ((1024, 32, 8, 1), (2048, 32, 32, 1), (512, 32, 8, 8), (4096, 32, 32, 1), (2048, 32, 8, 6), (1024, 32, 8, 32),
                              (256, 32, 32, 16), (8192, 32, 8, 1)):
            fn, fl = _causal_case(N, Hq, Hkv, B)[:2]
            row = {"tokens": N, "requests": B, "q_heads": Hq, "kv_heads": Hkv, "workgroups_of_256_rows": B * Hq * ((N + 255) // 256)}
            _time_graph(fn, launches=5, reps=2)  # first touch of the new buffers
            # (the library's choice is timed last: the first timing after new buffers reads a few per cent long)
            for key, choice in (("rows128_us", dict(prefill_rows="128")),
                                ("rows256_head_major_us", dict(prefill_rows="256", prefill_order="head")),
                                ("rows256_tile_major_us", dict(prefill_rows="256", prefill_order="tile")),
                                ("four_waves_us", dict(prefill_rows="half")),
                                ("one_head_per_workgroup_us", dict(prefill_pack="off")), ("chosen_us", {})):
                lsa.set_tuning(**choice)
                row[key] = round(_time_graph(fn, launches=20, reps=10, warm_reps=2) * 1e3, 1)
            row["chosen_tflops"] = round(fl / (row["chosen_us"] * 1e-6) / 1e12, 1)
            group = Hq // Hkv
            pack = 8 if group % 8 == 0 else 4 if group % 4 == 0 else 2 if group % 2 == 0 else 1
            row["tiles_only_floor_us"] = round(_tiles_256x64(N, Hq, B, pack) / 256.0 * tile_us, 1)
            rows.append(row)
    finally:
        lsa.set_tuning()
    torch.cuda.empty_cache()
    return {"what": " ".join(x.strip() for x in prefill_launch_sizes.__doc__.split("\n")), "tile_us": tile_us, "cases": rows}


def decode_latency():
    """Small-batch decode: the host's cost of a call against the device's.  GQA 32/8 (and 8/1: Llama-3-70B's heads per GPU
    under 8-way tensor parallelism), head_dim 128, fp16, scattered slots,
    fused stage 1 + stage 2 call (the operator a decode step of the layer makes, longserve_transformer_layer_infer.py:293-308).
    eager_us: wall clock per call over 200 back-to-back calls and one synchronize (host-bound when the host is slower
    than the kernels); graph_us: the same call replayed from a HIP graph of 20 of them, per call (device time; for the
    cases of a few megabytes the replays read the same K/V out of the caches, so no bandwidth is quoted for them)."""
    rows = []
    for Hq, Hkv, B, ctx in [(32, 8, B, ctx) for B in (1, 4, 16) for ctx in (2048, 8192, 32768)] + [(8, 1, 1, 8192), (8, 1, 8, 8192), (8, 1, 16, 32768)]:
        d = TokenDecode(B=B, Hq=Hq, Hkv=Hkv, lens=[ctx] * B, pool=B * ctx + 1024, seed=3100 + B)
        for _ in range(10):
            d.step()
        torch.cuda.synchronize()
        n = 200
        t0 = time.perf_counter()
        for _ in range(n):
            d.step()
        torch.cuda.synchronize()
        eager = (time.perf_counter() - t0) / n * 1e6
        graph = _time_graph(d.step, launches=20, reps=10) * 1e3
        row = {"q_heads": Hq, "kv_heads": Hkv, "batch": B, "ctx": ctx, "eager_us": round(eager, 2), "graph_us": round(graph, 2)}
        if d.bytes > 512e6:  # beyond what the 256 MB last-level cache can serve on replays
            row["kv_gbs_at_graph_rate"] = round(d.bytes / (graph * 1e-6) / 1e9, 1)
        rows.append(row)
        del d
    torch.cuda.empty_cache()
    return {"what": " ".join(x.strip() for x in decode_latency.__doc__.split("\n")),
            "reference_launch_overhead_us": "100-400 (Triton launch overhead the reference reports, longserve_cuda_kernels/README.md:7-9)",
            "cases": rows}


def decode_large_groups():
    """Token-indexed decode for GQA groups of eight and more query heads per KV head (outside the five baseline configs:
    Llama-3-70B is 64/8, 8/1 per GPU under 8-way tensor parallelism): batch 64, ctx U[4096,32768], scattered pool, fused
    call and stage 1 alone, through the library's own choice of stage-1 kernel (the matrix-pipe one for these shapes) and
    with the lane kernel forced (lsattn_set_tuning), which every smaller group runs on.  Device time per call from a HIP
    graph of 20 calls, median of 10 replays."""
    import loongserve_amd as lsa
    rows = []
    try:
        for Hq, Hkv in ((8, 1), (16, 2), (64, 8)):
            d = TokenDecode(Hq=Hq, Hkv=Hkv, seed=3300 + Hq)
            row = {"q_heads": Hq, "kv_heads": Hkv, "algorithmic_gb_per_step": d.bytes / 1e9}
            for key, choice in (("matrix_pipe", {}), ("lane_kernel", dict(decode_stage1="lane"))):
                lsa.set_tuning(**choice)
                fused = _time_graph(d.step, launches=20, reps=10)
                s1 = _time_graph(d.stage1_only, launches=20, reps=10)
                row[key] = {"fused_ms": fused, "fused_gbs": d.bytes / (fused * 1e-3) / 1e9, "stage1_ms": s1,
                            "stage1_gbs": d.bytes / (s1 * 1e-3) / 1e9}
            row["roofline"] = _roof("decode_stage1_mfma_kernel<F16,false|true> (the shape the library chooses)", "hbm", row["matrix_pipe"]["stage1_gbs"], row["matrix_pipe"]["stage1_ms"],
                                    "decode_%d_%d" % (Hq, Hkv))
            rows.append(row)
            del d
            torch.cuda.empty_cache()
    finally:
        lsa.set_tuning()
    return {"what": " ".join(x.strip() for x in decode_large_groups.__doc__.split("\n")), "cases": rows}


def decode_mixed_lengths(full=True):
    """Token-indexed decode of batches that mix one long request with many short ones (outside the five baseline
    configs), GQA 32/8, scattered pool: the two stages as the master of a decode step calls them (BLOCK_SEQ 256, one
    partial per block) and the fused call, through the library's own choice (stage 1 walks a list of the units of work
    that exist when the plain grid would have 32768 workgroups and more) and with the grid sized by the longest request
    forced (lsattn_set_tuning), as the reference's.  Device time per call from a HIP graph of 10 calls, median of 10 replays."""
    import loongserve_amd as lsa
    rows = []
    try:
        for lens, name in (([131072] + [512] * 255, "1 x 131072 + 255 x 512 tokens"), ([524288] + [2048] * 63, "1 x 524288 + 63 x 2048 tokens")):
            d = TokenDecode(B=len(lens), lens=lens, pool=sum(lens) + 1024, seed=3400 + len(lens))
            row = {"batch": name, "algorithmic_gb_per_step": d.bytes / 1e9}
            for key, choice in (("chosen", {}), ("grid_by_longest_request", dict(decode_listed="off")))[:2 if full else 1]:
                lsa.set_tuning(**choice)
                two = _time_graph(d.step_separate_stages, launches=10, reps=10)
                fused = _time_graph(d.step, launches=10, reps=10)
                row[key] = {"two_stages_ms": two, "two_stages_gbs": d.bytes / (two * 1e-3) / 1e9, "fused_ms": fused,
                            "fused_gbs": d.bytes / (fused * 1e-3) / 1e9}
            rows.append(row)
            del d
            torch.cuda.empty_cache()
    finally:
        lsa.set_tuning()
    return {"what": " ".join(x.strip() for x in decode_mixed_lengths.__doc__.split("\n")), "cases": rows}


def other_steps(steps):
    """The steps around attention (not part of the five baseline configs)."""
    import loongserve_amd as lsa
    out = {}
    # the element-wise steps around attention at config 2's per-GPU shape (16384 tokens, hidden 4096, 32 heads, inter 11008)
    from loongserve_amd import longserve_cuda_kernels as lk
    T, H, I, NH, D = 16384, 4096, 11008, 32, 128
    x = _randn_half((T, H), 7001, torch.float16)
    w = _randn_half((H,), 7002, torch.float16)
    io = _randn_half((T, 2 * I), 7003, torch.float16)
    qkv = _randn_half((T, 3 * NH, D), 7004, torch.float16)
    cs = _randn_half((T, D // 2), 7005, torch.float16)
    sn = _randn_half((T, D // 2), 7006, torch.float16)
    ew = {}
    for name, fn, nbytes in (("rms_norm", lambda: lk.rms_norm(x, w, 1e-5), 2 * T * H * 2 + H * 2),
                             ("silu_and_mul_inplace", lambda: lk.silu_and_mul_inplace(io), 3 * T * I * 2),
                             ("rotary_emb", lambda: lk.rotary_emb(qkv[:, :NH], qkv[:, NH:2 * NH], cs, sn),
                              2 * (2 * T * NH * D * 2) + 2 * 2 * T * (D // 2) * 2)):
        st = _stats(_time_events(fn, steps, 3))
        ew[name] = {"median_ms": st["median_ms"], "gbs": nbytes / (st["median_ms"] * 1e-3) / 1e9,
                    "pct_of_hbm_peak": 100 * nbytes / (st["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS}
    # decoding-stage migration: the last 32768 tokens of 4 requests, 2 layers, MHA 32 (16 KB per token and layer)
    import loongserve_amd as lsa
    Lm, Bm, nm, pool_m = 2, 4, 32768, 300000
    kvc = _randn_half((Lm, pool_m, 64, 128), 7101, torch.float16)
    gm = torch.Generator().manual_seed(20249)
    tab = torch.randperm(pool_m, generator=gm)[:Bm * 2 * nm].to(torch.int32).view(Bm, 2 * nm).to(DEV).contiguous()
    sbuf = torch.empty((Lm, Bm * nm, 64, 128), dtype=torch.float16, device=DEV)
    mstate = torch.ones(pool_m, dtype=torch.int32, device=DEV)
    rid, ntok, blen = _i32(list(range(Bm))), _i32([nm] * Bm), _i32([2 * nm] * Bm)
    st = _stats(_time_events(lambda: lsa.decoding_stage_migration_sender_kernel(sbuf, tab, mstate, kvc, rid, ntok, blen), steps, 2))
    mig_bytes = 2 * Lm * Bm * nm * 64 * 128 * 2
    out["decode_migration_send"] = {"workload": "%d requests x %d tokens, %d layers, 16 KB rows, scattered slots (includes the host read-back of max(num_tokens), as the reference)" % (Bm, nm, Lm),
                                    "median_ms": st["median_ms"], "gbs": mig_bytes / (st["median_ms"] * 1e-3) / 1e9,
                                    "pct_of_hbm_peak": 100 * mig_bytes / (st["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS}
    del kvc, sbuf, tab, mstate
    torch.cuda.empty_cache()
    out["elementwise"] = {"workload": "%d tokens, hidden %d, inter %d, %d heads x %d, fp16" % (T, H, I, NH, D), **ew}
    out["kv_pool_allocator"] = _bench_pool_allocator(steps)
    del x, w, io, qkv, cs, sn
    torch.cuda.empty_cache()
    return out


def _bench_pool_allocator(steps):
    """Slot searches of config 3's pool (2.5 M slots, about half in use, scattered): a decode step's 64 new slots.
    Wall clock per call, host work and read-backs included.  `torch_nonzero_*` times the same searches written as
    the reference writes them (nonzero over the whole pool, then slices), on the same device, for scale."""
    import loongserve_amd as lsa
    size, need = 2_500_000, 64
    mm = lsa.LongServeMemoryManager(size, torch.float16, 1, 8, 1)
    g = torch.Generator().manual_seed(20243)
    mm.add_refs(torch.randperm(size, generator=g)[:size // 2].to(DEV))

    def wall_us(fn, undo):
        for _ in range(3):
            undo(fn())
        torch.cuda.synchronize()
        t = []
        for _ in range(max(steps, 10)):
            t0 = time.perf_counter()
            r = fn()
            torch.cuda.synchronize()
            t.append((time.perf_counter() - t0) * 1e6)
            undo(r)
            torch.cuda.synchronize()
        return sorted(t)[len(t) // 2]

    def ref_alloc():
        can_use = torch.nonzero(mm.mem_state == 0).view(-1)
        sel = can_use[0:need]
        used = torch.count_nonzero(mm.mem_state[sel]).item()
        mm.mem_state[sel] += 1
        return sel

    def ref_contig():
        can_use = torch.nonzero(mm.mem_state == 0).view(-1)
        n = len(can_use)
        hit = can_use[0:n - 8 + 1][(can_use[8 - 1:] - can_use[0:n - 8 + 1]) == 8 - 1]
        return int(hit[0].item()) if hit.shape[0] else -1

    def undo_ref(sel):
        mm.mem_state[sel] -= 1

    res = {"workload": "pool of %d slots, half in use (scattered); alloc(%d) and the first run of 8 free slots" % (size, need),
           "alloc_us": wall_us(lambda: mm.alloc(need), mm.free),
           "find_contiguous_us": wall_us(lambda: mm._slots.first_fit(8), lambda r: None),
           "torch_nonzero_alloc_us": wall_us(ref_alloc, undo_ref),
           "torch_nonzero_find_contiguous_us": wall_us(ref_contig, lambda r: None)}
    ev = _stats(_time_events(lambda: mm._slots.first_fit(8), max(steps, 10), 3))
    res["find_contiguous_device_ms"] = ev["median_ms"]
    res["state_bytes_scanned"] = 2 * size * 4
    del mm
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only", choices=["prefill", "decode", "config1", "config4", "config5", "ceiling", "chunked"], default=None,
                    help="time one workload only (profiling aid)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="only run three plain 1 GiB device-to-device copies (known traffic, for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--sweeps", action="store_true", help="also time the launch-size, decode-latency, large-group and mixed-length sweeps (to --details-out)")
    ap.add_argument("--all", action="store_true", help="also time the steps around attention: element-wise kernels, migration, allocator (to --details-out)")
    ap.add_argument("--details-out", default=os.path.join(ROOT, "gpurun_out", "bench_details.json"),
                    help="file for everything that is not in the JSON line (written when there is something to write)")
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
    if args.calib_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device=DEV)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "3 x copy of 1 GiB (reads 1048576 KiB, writes 1048576 KiB per copy)"}))
        return

    line = {
        "metric": "prefill attn TFLOP/s + decode KV GB/s, as % of MI355X roofline (1 GPU)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
    }
    details, summary, roof, cpu = {}, {}, {}, {}
    ceil = Ceiling()
    only = args.only

    if only in (None, "prefill"):
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
        st = _stats(step_ms)
        tflops = w.flops / (wall_ms * 1e-3) / 1e12
        # a step is nothing but its four launches: the average launch duration is the step's HIP-event time / 4
        per_launch_ms = st["mean_ms"] / w.launches
        ach = (w.flops / w.launches) / (per_launch_ms * 1e-3) / 1e12
        # the box's ceiling right behind the timed steps (same thermal state): an MFMA stream and nothing else
        mfma_peak, _ = ceil.mfma_tflops()
        sep = _stats(_time_events(w.step_separate_merge, max(5, args.steps // 2), 2))
        inp = _stats(_time_events(w.step_in_place, max(5, args.steps // 2), 2))
        line.update({
            "value": tflops, "unit": "TFLOP/s", "ms_per_step": wall_ms,
            "config": {"workload": "config 2: ring prefill on one GPU, 16384 queries of shard 3 of a 131072-token sequence vs KV shards 3 "
                                   "(causal), 0, 1, 2 (full); MHA 32, head_dim 128, fp16; fp32 (O, LSE), each later launch merging its "
                                   "partial into the running result in its epilogue",
                       "algorithmic_tflop_per_step": w.flops / 1e12, "launches_per_step": w.launches,
                       "median_ms": st["median_ms"], "p10_ms": st["p10_ms"], "p90_ms": st["p90_ms"],
                       "separate_merge_ms": sep["median_ms"], "in_place_ms": inp["median_ms"]},
        })
        roof = _roof("prefill_kernel<F16,0,true,false> (diagonal) + prefill_kernel<F16,2,true,false> (three full launches)",
                     "mfma", ach, per_launch_ms, "config2", algorithmic_tflop_per_launch=w.flops / w.launches / 1e12,
                     sustained_peak=mfma_peak, frac_of_sustained=ach / mfma_peak,
                     sustained_peak_what="v_mfma_f32_16x16x32_f16 stream on random fp16 operands, one wave per SIMD, measured in this run (libls_ceiling.so)")
        summary["config2"] = {"value": _r(tflops, 1), "unit": "TFLOP/s", "frac": _r(tflops / PEAK_MFMA_TFLOPS), "ms": _r(wall_ms),
                              "kernel": "prefill_kernel<F16,0|2,true,false>", "frac_of_sustained": _r(ach / mfma_peak)}
        # the rate per 256-row x 64-key tile that the full launches run at, for the tiles-only floors of the sweeps
        tile_us = per_launch_ms * 1e3 * w.launches / ((3 * 256 + 130) * 8.0)  # tiles a CU walks per step: 8 workgroups x (3 x 256 + 130 average on the diagonal)
        if not args.no_cpu:
            cpu = w.cpu_baseline()
        del w
        torch.cuda.empty_cache()
    else:
        tile_us = 1.5

    if only in (None, "decode"):
        d = TokenDecode()
        torch.cuda.synchronize()
        st = _stats(_time_events(d.step, 50, 10))
        s1 = _stats(_time_events(d.stage1_only, 50, 10))
        sep = _stats(_time_events(d.step_separate_stages, 50, 10))
        sepm = _stats(_time_events(d.step_separate_stages_merged, 30, 5))
        read_peak, _ = ceil.read_gbs()
        read_stores_plain, read_stores_through, _ = ceil.read_with_stores_gbs(64)
        gbs = d.bytes / (st["median_ms"] * 1e-3) / 1e9
        # The fused call is two launches from one library call, timed together (HIP events around the call): stage 1 in equal
        # shares (decode_stage1_mfma_range_kernel, all but a few microseconds of it) and the merge of the shares' partials.
        # The same batch's stage 1 alone through the two-stage entry point (the plain grid, one partial per `split` tokens)
        # is reported beside it.
        ach = gbs
        plain = d.bytes / (s1["median_ms"] * 1e-3) / 1e9
        droof = {"decode_kernel": "decode_stage1_mfma_range_kernel<F16> (+ decode_stage2_kernel<float,128,256,true>: the fused call's two launches, timed together)",
                 "decode_achieved_gbs": ach, "decode_frac": ach / PEAK_HBM_GBS,
                 "decode_per_launch_ms": st["median_ms"], "decode_traffic": TRAFFIC_BYTES["config3"], "decode_algorithmic_gb": d.bytes / 1e9,
                 "decode_sustained_peak_gbs": read_peak, "decode_frac_of_sustained": ach / read_peak,
                 "decode_plain_grid_stage1_ms": s1["median_ms"], "decode_plain_grid_stage1_frac": plain / PEAK_HBM_GBS,
                 # the streaming read of the ceiling library with 1.6 % of stores mixed in (the share of one fp32 partial per
                 # 256 tokens in this gather): ordinary stores / stores written through as they are issued (the kernel's)
                 "decode_read_with_partial_stores_gbs": read_stores_plain, "decode_read_with_partial_stores_written_through_gbs": read_stores_through}
        summary["config3"] = {"value": _r(gbs, 1), "unit": "GB/s", "frac": _r(gbs / PEAK_HBM_GBS), "ms": _r(st["median_ms"]),
                              "p10_ms": _r(st["p10_ms"]), "p90_ms": _r(st["p90_ms"]), "kernel": "decode_stage1_mfma_range_kernel<F16> + decode_stage2_kernel",
                              "frac_of_sustained": _r(gbs / read_peak), "plain_grid_stage1_frac": _r(plain / PEAK_HBM_GBS),
                              "two_stages_reference_buffers_ms": _r(sep["median_ms"]),
                              "two_stages_reference_buffers_frac": _r(d.bytes / (sep["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS),
                              "two_stages_merged_blocks_frac": _r(d.bytes / (sepm["median_ms"] * 1e-3) / 1e9 / PEAK_HBM_GBS),
                              "two_stages_frac_of_read_with_as_many_stores": _r(d.bytes / (sep["median_ms"] * 1e-3) / 1e9 / read_stores_through),
                              "workload": "config 3: batch 64, ctx U[4096,32768], GQA 32/8, fp16, 2.5M-slot scattered pool; fused call, BLOCK_SEQ %d, "
                                          "stage 1 in equal shares of 256-token blocks" % d.BS}
        if only == "decode":
            line.update({"value": gbs, "unit": "GB/s", "ms_per_step": st["median_ms"], "steps": 50, "warmup": 10,
                         "config": {"workload": summary["config3"]["workload"]}})
            roof = _roof(droof["decode_kernel"], "hbm", ach, st["median_ms"], "config3", sustained_peak=read_peak, frac_of_sustained=ach / read_peak)
        else:
            roof.update(droof)
        if not args.no_cpu:
            c = d.cpu_baseline()
            if only == "decode":
                cpu = c
            else:
                cpu.update({"decode_value_gbs": c["value"], "decode_sample": c["sample"]})
        del d
        torch.cuda.empty_cache()

    if only in (None, "config1"):
        c1 = config1()
        summary["config1"] = {k: (_r(v) if isinstance(v, float) else v) for k, v in c1.items() if k in ("value", "unit", "frac", "ms", "p10_ms", "p90_ms", "kernel")}
        roof.update({"config1_frac": c1["frac"], "config1_per_launch_ms": c1["ms"], "config1_traffic": c1["traffic"]})
        details["config1"] = c1
    if only in (None, "config4"):
        c4 = config4()
        summary["config4"] = {k: (_r(v) if isinstance(v, float) else v) for k, v in c4.items() if k in ("value", "unit", "frac", "ms", "p10_ms", "p90_ms", "kernel", "kernel_frac")}
        roof.update({"config4_frac": c4["kernel_frac"], "config4_per_launch_ms": c4["kernel_ms"], "config4_traffic": c4["traffic"]})
        details["config4"] = c4
    if only in (None, "config5"):
        c5 = config5(details if (args.sweeps or args.all) else None)
        summary["config5"] = {k: (_r(v) if isinstance(v, float) else v) for k, v in c5.items() if k in ("value", "unit", "frac", "ms", "kernel", "kernel_frac", "kernel_ms", "kv_write_gbs")}
        roof.update({"config5_frac": c5["kernel_frac"], "config5_per_launch_ms": c5["kernel_ms"], "config5_traffic": c5["traffic"]})
        details["config5"] = c5
    if only == "ceiling":
        mfma_peak, mfma_ms = ceil.mfma_tflops()
        read_peak, read_ms = ceil.read_gbs()
        line.update({"value": mfma_peak, "unit": "TFLOP/s", "ms_per_step": mfma_ms, "config": {"workload": "ceilings: MFMA stream, 4 GiB read"}})
        summary["ceiling"] = {"mfma_tflops": _r(mfma_peak, 1), "mfma_ms": _r(mfma_ms), "read_gbs": _r(read_peak, 1), "read_ms": _r(read_ms),
                              "read_with_stores_gbs": {"%.2f %% of the bytes stored" % (100.0 / e): dict(zip(("plain", "written_through"), (_r(a, 1), _r(b, 1))))
                                                       for e in (1024, 256, 64, 16) for a, b, _ in (ceil.read_with_stores_gbs(e),)}}
    if only == "chunked":
        summary["chunked_prefill_step"] = c = chunked_prefill_step()
        line.update({"value": c["kv_gbs_workspace_route"], "unit": "GB/s", "ms_per_step": c["context_attention_fwd_workspace_us"] * 1e-3,
                     "config": {"workload": c["workload"]}})
    if only is None:
        summary["short_prompts"] = short_prompts()
        summary["chunked_prefill_step"] = chunked_prefill_step()
        # decode batches of one long request beside many short ones: the two stages as a decode step's master calls them
        # (one partial per 256 tokens) and the fused call, as fractions of the HBM peak
        summary["decode_mixed_lengths"] = {
            c["batch"].replace(" tokens", "").replace(" ", ""): {
                "two_stages_ms": _r(c["chosen"]["two_stages_ms"]), "two_stages_frac": _r(c["chosen"]["two_stages_gbs"] / PEAK_HBM_GBS),
                "fused_ms": _r(c["chosen"]["fused_ms"]), "fused_frac": _r(c["chosen"]["fused_gbs"] / PEAK_HBM_GBS)}
            for c in decode_mixed_lengths(full=False)["cases"]}
        summary["ceiling"] = {"mfma_tflops": _r(roof.get("sustained_peak"), 1), "read_gbs": _r(roof.get("decode_sustained_peak_gbs"), 1),
                              "read_with_1.6pct_stores_gbs": [_r(roof.get("decode_read_with_partial_stores_gbs"), 1),
                                                             _r(roof.get("decode_read_with_partial_stores_written_through_gbs"), 1)]}
    if args.sweeps:
        details["prefill_launch_sizes"] = prefill_launch_sizes(tile_us)
        details["decode_latency"] = decode_latency()
        details["decode_large_groups"] = decode_large_groups()
        details["decode_mixed_lengths"] = decode_mixed_lengths()
    if args.all:
        details["other"] = other_steps(10)
    if roof:
        line["roofline"] = {k: (_r(v, 5) if isinstance(v, float) else v) for k, v in roof.items()}
    if cpu:
        line["cpu_baseline"] = cpu
    if "value" not in line and summary:  # --only config1/4/5: that workload is the line's value
        k = next(iter(summary))
        line.update({"value": summary[k]["value"], "unit": summary[k]["unit"], "ms_per_step": summary[k]["ms"], "config": {"workload": details[k]["workload"]}})
    line["summary"] = summary  # (last: a reader that keeps the tail of the line keeps all five configs)
    if (args.sweeps or args.all) and details:
        os.makedirs(os.path.dirname(os.path.abspath(args.details_out)), exist_ok=True)
        with open(args.details_out, "w") as f:
            json.dump(details, f, indent=1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

"""One-GPU counterparts of the two callers of the hot path.

`ring_prefill*` plays the ring loop of LongServeTransformerLayerInfer._context_attention_kernel
(loongserve/models/llama/layer_infer/longserve_transformer_layer_infer.py:104-160) with the
KV chunks of all logical peers already resident on this GPU: each ring step is one kernel
launch against one chunk, in sequence, and no send/recv happens.

`multi_instance_decode` plays _token_decode_attention_overlapped (:224-370): every
"instance" holds a part of each request's KV in the token-indexed pool; peers produce
(O fp32, LSE) with stage1+stage2, the master runs stage 1 on its own part into the rows
after the peers' and one stage-2 call with block_seq=1 merges everything
(buffer shapes from loongserve/models/llama/longserve_model.py:505-517, :531-533).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch

from .decoding import (longserve_flash_decode_stage1, longserve_flash_decode_stage2,
                       longserve_token_decode_attention_flash_decoding)
from .ops import context_attention_fwd, lse_merge, prefill_attention_step


@dataclass
class KVChunk:
    """One peer's KV chunk as it would arrive over the ring: an interleaved
    [tokens, 2*Hkv, D] buffer (K heads then V heads) plus its three int32 metadata vectors."""
    kv: torch.Tensor
    b_start_loc: torch.Tensor
    b_seq_len: torch.Tensor
    first_token_global_idx: torch.Tensor

    def k(self, hkv: int) -> torch.Tensor:
        return self.kv[:, :hkv, :]

    def v(self, hkv: int) -> torch.Tensor:
        return self.kv[:, hkv:, :]


def ring_prefill(q, chunks: Sequence[KVChunk], q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                 logical_sp_peers_num: int, max_q_len: int, num_kv_heads: int,
                 out: Optional[torch.Tensor] = None, m: Optional[torch.Tensor] = None,
                 l: Optional[torch.Tensor] = None):
    """In-place ring: chunks[0] must be the local chunk (LI:115-117).  Returns (o, m, l)."""
    o = torch.empty_like(q) if out is None else out
    o.zero_()
    m = torch.empty(q.shape[:2], dtype=torch.float32, device=q.device) if m is None else m
    l = torch.empty(q.shape[:2], dtype=torch.float32, device=q.device) if l is None else l
    m.fill_(float("-inf"))
    l.zero_()
    for c in chunks:
        context_attention_fwd(q, c.k(num_kv_heads), c.v(num_kv_heads), o, q_b_start_loc, q_b_seq_len,
                              q_first_token_global_idx, c.b_start_loc, c.b_seq_len, c.first_token_global_idx,
                              logical_sp_peers_num, max_q_len, m, l, total_q_len=q.shape[0])  # (q is packed: its rows bound the batch)
    return o, m, l


def ring_prefill_partials(q, chunks: Sequence[KVChunk], q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                          logical_sp_peers_num: int, max_q_len: int, num_kv_heads: int,
                          bufs: Optional[List[Tuple[torch.Tensor, torch.Tensor]]] = None,
                          out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None):
    """Each step emits an fp32 partial (O_i, LSE_i); one LSE merge combines them.  Returns (O, LSE)."""
    parts = []
    for i, c in enumerate(chunks):
        ob, lb = bufs[i] if bufs is not None else (None, None)
        parts.append(prefill_attention_step(q, c.k(num_kv_heads), c.v(num_kv_heads), q_b_start_loc, q_b_seq_len,
                                            q_first_token_global_idx, c.b_start_loc, c.b_seq_len,
                                            c.first_token_global_idx, logical_sp_peers_num, max_q_len, ob, lb,
                                            total_q_len=q.shape[0]))
    return lse_merge(parts, out, lse)


def ring_prefill_accumulate(q, chunks: Sequence[KVChunk], q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                            logical_sp_peers_num: int, max_q_len: int, num_kv_heads: int,
                            out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None):
    """The first step writes the fp32 partial (O, LSE); every later step LSE-merges its partial into it in the
    kernel's epilogue: no per-step buffers and no separate merge pass.  Returns (O, LSE)."""
    for i, c in enumerate(chunks):
        out, lse = prefill_attention_step(q, c.k(num_kv_heads), c.v(num_kv_heads), q_b_start_loc, q_b_seq_len,
                                          q_first_token_global_idx, c.b_start_loc, c.b_seq_len, c.first_token_global_idx,
                                          logical_sp_peers_num, max_q_len, out, lse, accumulate=i > 0, total_q_len=q.shape[0])
    return out, lse


def ring_prefill_with_migration(q, chunks: Sequence[KVChunk], q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                                logical_sp_peers_num: int, max_q_len: int, num_kv_heads: int,
                                kv_cache_index_begin, kv_cache_index_end, mem_index, mem_cache, req_to_token_indexs,
                                b_req_idx, should_register_kv: bool = True):
    """The in-place ring with the context migration of longserve_transformer_layer_infer.py:180-220: after each step the
    rows of the chunk at hand whose global token index falls in this instance's window
    [kv_cache_index_begin, kv_cache_index_end) are copied into the pool slots `mem_index` hands out, in the order the
    chunks pass by, and (first layer) registered in the request table after the rows kept so far.  This is how a
    prefill spread over several instances leaves its KV on fewer of them.  Returns (o, m, l, kept rows per request)."""
    from .ops import destindex_copy_and_register_kv, pre_copy_and_register_kv
    o = torch.zeros_like(q)
    m = torch.full(q.shape[:2], float("-inf"), dtype=torch.float32, device=q.device)
    l = torch.zeros(q.shape[:2], dtype=torch.float32, device=q.device)
    batch = q_b_seq_len.shape[0]
    cur_kv_cache_index = torch.zeros(batch, dtype=torch.int32, device=q.device)
    num_used_mem_index = 0
    for c in chunks:
        context_attention_fwd(q, c.k(num_kv_heads), c.v(num_kv_heads), o, q_b_start_loc, q_b_seq_len,
                              q_first_token_global_idx, c.b_start_loc, c.b_seq_len, c.first_token_global_idx,
                              logical_sp_peers_num, max_q_len, m, l, total_q_len=q.shape[0])
        kv_range_begin, kv_range_end, new_kv_cache_len = pre_copy_and_register_kv(
            kv_cache_index_begin, kv_cache_index_end, c.first_token_global_idx, logical_sp_peers_num)
        new_kv_cache_len_sum = torch.cumsum(new_kv_cache_len, dim=0, dtype=torch.int64)
        destindex_copy_and_register_kv(batch, new_kv_cache_len, kv_range_begin, kv_range_end, new_kv_cache_len_sum, c.kv,
                                       c.b_start_loc, cur_kv_cache_index, mem_index, mem_cache, req_to_token_indexs,
                                       b_req_idx, num_used_mem_index, max_q_len + 1, should_register_kv)
        num_used_mem_index += int(new_kv_cache_len_sum[-1].item())  # as the reference: one read-back per step
        cur_kv_cache_index += new_kv_cache_len
    return o, m, l, cur_kv_cache_index


def next_power_of_2(n: int) -> int:
    return 1 if n <= 1 else 1 << (n - 1).bit_length()


def decode_block_seq(max_len_in_batch: int, peer_max_len_in_batch: int = 0) -> int:
    """BLOCK_SEQ rule of loongserve/models/llama/longserve_model.py:505-508."""
    return min(next_power_of_2(max(max_len_in_batch, peer_max_len_in_batch, 16)), 256)


@dataclass
class DecodeInstance:
    """What one (simulated) instance holds for a decode batch."""
    cache_kv: torch.Tensor        # [slots, 2*Hkv, D] token-indexed pool of this instance
    req_to_token: torch.Tensor    # [max_req, max_seq] int32
    b_req_idx: torch.Tensor       # [batch] int32
    b_seq_len: torch.Tensor       # [batch] int32: tokens of each request held here
    max_len_in_batch: int


def multi_instance_decode(q, instances: Sequence[DecodeInstance], num_kv_heads: int, block_seq: Optional[int] = None,
                          out: Optional[torch.Tensor] = None, workspace: Optional[dict] = None):
    """instances[0] is the master, the others are peers.  Returns (o [B,Hq,D] in q.dtype, LSE [B,Hq])."""
    B, Hq, D = q.shape
    P = len(instances)
    master = instances[0]
    peer_max = max([i.max_len_in_batch for i in instances[1:]], default=0)
    BS = decode_block_seq(master.max_len_in_batch, peer_max) if block_seq is None else block_seq
    num_seq_block = (master.max_len_in_batch + BS - 1) // BS  # MODEL:511
    ws = {} if workspace is None else workspace
    dev = q.device

    def buf(name, shape, dtype=torch.float32):
        t = ws.get(name)
        if t is None or tuple(t.shape) != tuple(shape):
            t = torch.empty(shape, dtype=dtype, device=dev)
            ws[name] = t
        return t

    global_mid_o = buf("global_mid_o", (P - 1 + num_seq_block, B, Hq, D))
    global_mid_lse = buf("global_mid_o_logexpsum", (P - 1 + num_seq_block, B, Hq))
    global_out_lse = buf("global_out_logexpsum", (B, Hq))
    # MODEL:516
    merge_len = ((P - 1) + (master.b_seq_len + (BS - 1)) // BS).to(torch.int32).contiguous()

    # peers: stage1 + stage2 over what they hold, fp32 partial straight into the master's rows 0..P-2
    for r, inst in enumerate(instances[1:]):
        nsb = inst.max_len_in_batch // BS + 1  # MODEL:531
        pm = buf("peer_mid_o_%d" % r, (nsb, B, Hq, D))
        pl = buf("peer_mid_lse_%d" % r, (nsb, B, Hq))
        longserve_token_decode_attention_flash_decoding(
            q, inst.req_to_token, inst.b_req_idx, inst.b_seq_len, pm, pl, B, inst.max_len_in_batch, Hq, D,
            inst.cache_kv[:, :num_kv_heads, :], inst.cache_kv[:, num_kv_heads:, :], BS,
            global_mid_o[r], global_mid_lse[r])
    # master: local split-K partials after the peers' rows (LI:272-281)
    longserve_flash_decode_stage1(q, master.cache_kv[:, :num_kv_heads, :], master.cache_kv[:, num_kv_heads:, :],
                                  master.req_to_token, master.b_req_idx, master.b_seq_len, master.max_len_in_batch,
                                  global_mid_o[P - 1:], global_mid_lse[P - 1:], BS)
    o = torch.empty_like(q) if out is None else out
    # LI:360-367
    longserve_flash_decode_stage2(global_mid_o, global_mid_lse, merge_len, o.view(-1, Hq, D), global_out_lse, 1)
    return o, global_out_lse

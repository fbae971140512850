"""CPU oracle for the per-GPU attention hot path (TEST INFRASTRUCTURE, not product code).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  The product path (loongserve_amd) never imports it and has no CPU fallback.

Every function restates, in plain PyTorch on the CPU, the arithmetic of one piece of the
reference; citations are relative to the reference tree:

  RING  = loongserve/models/llama/triton_kernel/ring_context_flashattention_nopad.py
  S1CU  = longserve_cuda_kernels/src/flash_decoding_stage1.cu
  S2CU  = longserve_cuda_kernels/src/flash_decoding_stage2.cu
  ENTRY = longserve_cuda_kernels/src/entrypoints.cpp
  FDPY  = loongserve/models/llama/triton_kernel/longserve_flash_decoding.py
  MODEL = loongserve/models/llama/longserve_model.py

The reference ships no golden vectors and no runnable test for this path (its one
prefill self-test passes 13 of 14 arguments, there is no decode test), so the oracle is
pinned by closed forms and invariants in tests/test_oracle_pins.py: library softmax /
scaled_dot_product_attention, brute-force float64 loops on tiny inputs, single-key,
q=0 and constant-V special cases, ring == monolithic, step-order invariance,
striped == contiguous, stage1+stage2 == one-shot attention over the gathered rows.

Deliberate, documented deviations from the reference *as written* (the oracle follows the
intended mathematics):
  * misaligned causal bounds: the reference's two-phase tile loop (RING:114-169) can visit
    up to BLOCK_N-1 keys twice when the bound is not a multiple of BLOCK_N; the oracle is
    exact masked attention (what RING:287-321 `torch_att` computes);
  * rows / ranges with no visible key: the reference leaves finite garbage (RING:160) or
    uninitialised memory (S1CU:55-57, S2CU:50); the oracle defines O = 0, LSE = -inf.
Pinned: attn_step, lse_merge, context_attention_fwd state update, decode stage1/stage2,
gather, kv scatter.  Not pinned by anything ("parity unpinned"): the reference's fp16
re-rounding trajectory of `o` across ring steps (RING:181-186) and its fast-math
exp/log bit patterns; both are below the stated tolerances and are not reproduced.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

LOG2E = 1.4426950408889634
LN2 = 0.6931471805599453
INT32_PAD = 2147483647  # loongserve/common/longserve_req_manager.py:19 fills unused table entries with this


# --------------------------------------------------------------------------------------
# prefill: one ring / context-parallel attention step
# --------------------------------------------------------------------------------------
def visible_mask(q_len: int, kv_len: int, q_first: int, kv_first: int, peers: int,
                 m0: int = 0, m1: Optional[int] = None) -> torch.Tensor:
    """Boolean [m1-m0, kv_len]: key n visible to local query row m.

    RING:156-159: (q_first + m*P) >= (kv_first + n*P) and n < kv_len.
    """
    m1 = q_len if m1 is None else m1
    qg = q_first + torch.arange(m0, m1, dtype=torch.int64) * peers
    kg = kv_first + torch.arange(0, kv_len, dtype=torch.int64) * peers
    return qg[:, None] >= kg[None, :]


def attn_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
              q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
              kv_b_start_loc, kv_b_seq_len, kv_first_token_global_idx,
              logical_sp_peers_num: int, sm_scale: Optional[float] = None,
              dtype: torch.dtype = torch.float32, q_chunk: int = 2048
              ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Exact attention of local Q against one KV chunk -> (O [Tq,Hq,D], LSE [Tq,Hq]).

    Closed form of what RING:13-188 computes for one call starting from the empty state:
    O = softmax(Q K^T / sqrt(D) + mask) V, LSE = natural-log logsumexp of the masked
    scores.  GQA mapping kv_head = q_head // (Hq // Hkv) (RING:41, :260).  Inputs are
    up-cast from their storage dtype; arithmetic is in `dtype` (float32 or float64).
    Rows with no visible key give O = 0, LSE = -inf.
    """
    Tq, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = (1.0 / math.sqrt(D)) if sm_scale is None else sm_scale
    O = torch.zeros(Tq, Hq, D, dtype=dtype)
    LSE = torch.full((Tq, Hq), float("-inf"), dtype=dtype)
    B = len(q_b_seq_len)
    for b in range(B):
        qs, ql = int(q_b_start_loc[b]), int(q_b_seq_len[b])
        ks, kl = int(kv_b_start_loc[b]), int(kv_b_seq_len[b])
        qf, kf = int(q_first_token_global_idx[b]), int(kv_first_token_global_idx[b])
        if ql <= 0 or kl <= 0:
            continue
        kb = k[ks:ks + kl].to(dtype).permute(1, 0, 2)  # [Hkv, kl, D]
        vb = v[ks:ks + kl].to(dtype).permute(1, 0, 2)
        for m0 in range(0, ql, q_chunk):
            m1 = min(ql, m0 + q_chunk)
            qb = q[qs + m0:qs + m1].to(dtype).permute(1, 0, 2)  # [Hq, m, D]
            mask = visible_mask(ql, kl, qf, kf, logical_sp_peers_num, m0, m1)  # [m, kl]
            # limit the key range to what the last row of the chunk can see
            nvis = int(mask[-1].sum()) if mask.numel() else 0
            if nvis == 0:
                continue
            qg = qb.reshape(Hkv, G * (m1 - m0), D)
            s = torch.bmm(qg, kb[:, :nvis].transpose(1, 2)) * scale  # [Hkv, G*m, nvis]
            s = s.reshape(Hq, m1 - m0, nvis)
            s = s.masked_fill(~mask[None, :, :nvis], float("-inf"))
            lse = torch.logsumexp(s, dim=-1)  # [Hq, m]; -inf where nothing is visible
            p = torch.exp(s - torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)[..., None])
            p = torch.where(torch.isinf(lse)[..., None], torch.zeros_like(p), p)
            o = torch.bmm(p.reshape(Hkv, G * (m1 - m0), nvis), vb[:, :nvis]).reshape(Hq, m1 - m0, D)
            O[qs + m0:qs + m1] = o.permute(1, 0, 2)
            LSE[qs + m0:qs + m1] = lse.permute(1, 0)
    return O, LSE


def lse_merge(parts: Sequence[Tuple[torch.Tensor, torch.Tensor]]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Merge normalised partials (O_i, LSE_i) over disjoint key sets.

    O = sum_i exp(LSE_i - LSE) O_i, LSE = log sum_i exp(LSE_i): the same recurrence as
    S2CU:38-48 / RING:171-188, written as a one-shot reduction.  An all-empty row
    (every LSE_i = -inf) stays (0, -inf).
    """
    lses = torch.stack([p[1] for p in parts], 0)
    os_ = torch.stack([p[0] for p in parts], 0)
    lse = torch.logsumexp(lses, dim=0)
    safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
    w = torch.exp(lses - safe[None])
    w = torch.where(torch.isinf(lse)[None].expand_as(w), torch.zeros_like(w), w)
    return (w[..., None] * os_).sum(0), lse


def context_attention_fwd(q, k, v, o, q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                          kv_b_start_loc, kv_b_seq_len, kv_first_token_global_idx,
                          logical_sp_peers_num: int, max_q_b_seq_len: int, m, l) -> None:
    """In-place ring-state update with the reference operator's signature (RING:191-206).

    State convention (RING:74-75, :171-188; caller init at
    loongserve/models/llama/layer_infer/longserve_transformer_layer_infer.py:123-126):
    `o` is the normalised running output in o.dtype, `m` the running max of
    score*log2(e)/sqrt(D) (log2 domain), `l` the running sum of 2^(score' - m); so the
    natural LSE over all keys seen so far is ln2 * (m + log2 l).  One call folds this
    step's exact partial into (o, m, l) exactly as RING:171-188 does:
        M = max(m_i, m_old); L = l_old 2^(m_old-M) + l_i 2^(m_i-M)
        o = (o_old l_old 2^(m_old-M) + acc_i 2^(m_i-M)) / L
    A step that sees no key for a row leaves that row's state untouched.
    """
    O_i, LSE_i = attn_step(q, k, v, q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                           kv_b_start_loc, kv_b_seq_len, kv_first_token_global_idx,
                           logical_sp_peers_num)
    B = len(q_b_seq_len)
    for b in range(B):
        qs, ql = int(q_b_start_loc[b]), int(q_b_seq_len[b])
        if ql <= 0:
            continue
        sl = slice(qs, qs + ql)
        lse_i = LSE_i[sl]
        has = ~torch.isinf(lse_i)
        # this step's state in the reference representation: choose m_i = log2-domain LSE, l_i = 1
        m_i = torch.where(has, lse_i * LOG2E, torch.full_like(lse_i, float("-inf")))
        l_i = has.to(torch.float32)
        m_old = m[sl].to(torch.float32)
        l_old = l[sl].to(torch.float32)
        M = torch.maximum(m_i, m_old)
        Ms = torch.where(torch.isinf(M), torch.zeros_like(M), M)
        w_old = l_old * torch.exp2(m_old - Ms)
        w_new = l_i * torch.exp2(m_i - Ms)
        L = w_old + w_new
        Ls = torch.where(L == 0, torch.ones_like(L), L)
        out = (o[sl].to(torch.float32) * w_old[..., None] + O_i[sl] * w_new[..., None]) / Ls[..., None]
        o[sl] = out.to(o.dtype)
        m[sl] = M
        l[sl] = L


def state_lse(m: torch.Tensor, l: torch.Tensor) -> torch.Tensor:
    """Natural-log LSE encoded by the reference's (m, l) ring state: ln2 * (m + log2 l)."""
    return LN2 * (m.double() + torch.log2(l.double()))


# --------------------------------------------------------------------------------------
# decode: token-indexed flash decoding
# --------------------------------------------------------------------------------------
def gather_rows(pool: torch.Tensor, req_to_tokens: torch.Tensor, req: int, start: int, end: int) -> torch.Tensor:
    """Bit-exact gather of pool rows named by req_to_tokens[req, start:end] (S1CU:73-75, :86-87)."""
    idx = req_to_tokens[req, start:end].to(torch.int64)
    return pool.index_select(0, idx)


def decode_stage1(q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch: int,
                  mid_o, mid_o_logexpsum, block_seq: int, dtype: torch.dtype = torch.float32) -> None:
    """Split-K partials, argument order of S1PY:78 (longserve_flash_decode_stage1).

    For every request b and block blk with blk*BS < len_b (S1CU:50-57):
      rows = K[table[req_b, blk*BS : min((blk+1)*BS, len_b)]]      (S1CU:73-75, :86)
      s = (q_b . rows) / sqrt(D)                                   (S1CU:85-93, ENTRY:142)
      mid_o_logexpsum[blk,b,h] = log sum exp s                     (S1CU:97-116)
      mid_o[blk,b,h,:] = softmax(s) @ V rows                       (S1CU:119-142)
    Blocks at or past len_b are left untouched, as in the reference.
    Layouts: mid_o [nblk,B,Hq,D], mid_o_logexpsum [nblk,B,Hq] (S1CU:26-27).
    """
    B, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    scale = 1.0 / math.sqrt(D)
    nblk_grid = (max_len_in_batch + block_seq - 1) // block_seq  # S1CU:211
    for b in range(B):
        n = int(b_seqlen[b])
        req = int(b_req_idx[b])
        qb = q[b].to(dtype).reshape(Hkv, G, D)
        for blk in range(min(nblk_grid, mid_o.shape[0])):
            s0 = blk * block_seq
            s1 = min(s0 + block_seq, n)
            if s1 <= s0:
                break
            kr = gather_rows(k, req_to_tokens, req, s0, s1).to(dtype).permute(1, 0, 2)  # [Hkv, t, D]
            vr = gather_rows(v, req_to_tokens, req, s0, s1).to(dtype).permute(1, 0, 2)
            s = torch.bmm(qb, kr.transpose(1, 2)) * scale  # [Hkv, G, t]
            lse = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - lse[..., None])
            o = torch.bmm(p, vr)  # [Hkv, G, D]
            mid_o[blk, b] = o.reshape(Hq, D).to(mid_o.dtype)
            mid_o_logexpsum[blk, b] = lse.reshape(Hq).to(mid_o_logexpsum.dtype)


def decode_stage2(mid_o, mid_o_logexpsum, b_seqlen, o, out_logexpsum, block_seq: int) -> None:
    """LSE-weighted merge over the block axis, argument order of S2PY:53.

    n_b = 0 if len_b <= 0 else ceil(len_b / block_seq) (S2CU:30); the first n_b rows of
    mid_o[:, b, h] are merged with the recurrence of S2CU:38-48; o = acc / sum,
    out_logexpsum = max + log(sum) (S2CU:50-57).  With block_seq = 1 and
    b_seqlen = merge_len this merges per-instance partials (MODEL:514-516).
    n_b = 0 gives O = 0, LSE = -inf (the reference writes nothing there).
    """
    B = o.shape[0]
    for b in range(B):
        n = int(b_seqlen[b])
        nb = 0 if n <= 0 else (n + block_seq - 1) // block_seq
        if nb == 0:
            o[b] = 0
            out_logexpsum[b] = float("-inf")
            continue
        parts = [(mid_o[i, b].float(), mid_o_logexpsum[i, b].float()) for i in range(nb)]
        ob, lb = lse_merge(parts)
        o[b] = ob.to(o.dtype)
        out_logexpsum[b] = lb


def token_decode_attention_flash_decoding(q, req_to_token_indexs, b_req_idx, b_seq_len, mid_o,
                                          mid_o_logexpsum, batch_size, max_len_in_batch, q_head_num,
                                          head_dim, cache_k, cache_v, BLOCK_SEQ, out=None, o_logexpsum=None):
    """stage1 -> stage2 with fp32 outputs, signature and allocation rule of FDPY:3-28."""
    o_tensor = torch.empty_like(q, dtype=torch.float32) if out is None else out
    lse = torch.empty([batch_size, q_head_num], dtype=torch.float32) if o_logexpsum is None else o_logexpsum
    decode_stage1(q.view(-1, q_head_num, head_dim), cache_k, cache_v, req_to_token_indexs, b_req_idx,
                  b_seq_len, max_len_in_batch, mid_o, mid_o_logexpsum, BLOCK_SEQ)
    decode_stage2(mid_o, mid_o_logexpsum, b_seq_len, o_tensor.view(-1, q_head_num, head_dim), lse, BLOCK_SEQ)
    return o_tensor, lse


def decode_full(q, k, v, req_to_tokens, b_req_idx, b_seqlen, dtype=torch.float32):
    """One-shot decode attention over each request's whole token list -> (O [B,Hq,D], LSE [B,Hq])."""
    B, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    O = torch.zeros(B, Hq, D, dtype=dtype)
    LSE = torch.full((B, Hq), float("-inf"), dtype=dtype)
    for b in range(B):
        n = int(b_seqlen[b])
        if n <= 0:
            continue
        req = int(b_req_idx[b])
        kr = gather_rows(k, req_to_tokens, req, 0, n).to(dtype).permute(1, 0, 2)
        vr = gather_rows(v, req_to_tokens, req, 0, n).to(dtype).permute(1, 0, 2)
        s = torch.bmm(q[b].to(dtype).reshape(Hkv, G, D), kr.transpose(1, 2)) / math.sqrt(D)
        lse = torch.logsumexp(s, dim=-1)
        O[b] = torch.bmm(torch.exp(s - lse[..., None]), vr).reshape(Hq, D)
        LSE[b] = lse.reshape(Hq)
    return O, LSE


# --------------------------------------------------------------------------------------
# KV pool writes (the data format on the producing side of the path)
# --------------------------------------------------------------------------------------
def kv_scatter(src: torch.Tensor, dest_index: torch.Tensor, pool: torch.Tensor) -> None:
    """pool[dest_index[i]] = src[i], bit-exact
    (loongserve/common/basemodel/triton_kernel/destindex_copy_kv.py:21-27)."""
    pool.index_copy_(0, dest_index.to(torch.int64), src)


def register_tokens(req_to_tokens, b_req_idx, b_start_loc, b_seq_len, mem_index) -> None:
    """req_to_tokens[req_b, 0:len_b] = mem_index[start_b : start_b+len_b]
    (loongserve/common/infer_utils.py:1-13)."""
    for b in range(len(b_req_idx)):
        s, n = int(b_start_loc[b]), int(b_seq_len[b])
        req_to_tokens[int(b_req_idx[b]), 0:n] = mem_index[s:s + n].to(req_to_tokens.dtype)


def copy_kv_index_to_req(req_to_token_indexs, b_req_idx, b_seq_len, memindex) -> None:
    """req_to_token_indexs[b_req_idx[i], b_seq_len[i] - 1] = memindex[i], one entry per request
    (loongserve/common/basemodel/triton_kernel/copy_kv_index_to_req.py:12-18)."""
    for i in range(len(b_req_idx)):
        req_to_token_indexs[int(b_req_idx[i]), int(b_seq_len[i]) - 1] = int(memindex[i])


def kv_ranges(kv_cache_index_begin, kv_cache_index_end, kv_first_token_global_idx, peers: int):
    """(kv_range_begin, kv_range_end, new_kv_cache_len) of pre_copy_and_register_kv
    (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:24-31, docstring :42-48):
    ceil((index - first) / peers) written as Python floor division of x + peers - 1."""
    rb = [(int(b) - int(f) + (peers - 1)) // peers for b, f in zip(kv_cache_index_begin, kv_first_token_global_idx)]
    re = [(int(e) - int(f) + (peers - 1)) // peers for e, f in zip(kv_cache_index_end, kv_first_token_global_idx)]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    return i32(rb), i32(re), i32([e - b for b, e in zip(rb, re)])


def kv_copy_register(batch_size, new_kv_cache_len, kv_range_begin, kv_range_end, new_kv_cache_len_sum, kv, kv_b_start_loc,
                     cur_kv_cache_index, mem_index, total_kv_cache, req_to_token_indexs, b_req_idx,
                     num_used_mem_index: int, max_len_in_batch: int, should_register_kv: bool) -> None:
    """destindex_copy_and_register_kv as plain loops
    (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:92-117: skip rule :96-97, slot list offset :99-100,
    source row :106, row loop bounded by the grid :159 and BLOCK_N :157, registration :112-117)."""
    row_limit = (max_len_in_batch + 255) // 256 * 256
    for b in range(batch_size):
        n_new, begin, end = int(new_kv_cache_len[b]), int(kv_range_begin[b]), int(kv_range_end[b])
        if n_new <= 0 or begin < 0 or end < 0:
            continue
        start = (int(new_kv_cache_len_sum[b - 1]) if b > 0 else 0) + num_used_mem_index
        for n in range(min(n_new, row_limit)):
            slot = int(mem_index[start + n])
            total_kv_cache[slot] = kv[int(kv_b_start_loc[b]) + begin + n]
            if should_register_kv:
                req_to_token_indexs[int(b_req_idx[b]), int(cur_kv_cache_index[b]) + n] = slot


def decoding_stage_migration_sender(send_buf, req_to_token_indexes, mem_state, kv_cache, request_ids, num_tokens, b_seq_len) -> None:
    """_fwd_sender_kernel as loops (loongserve/models/llama/triton_kernel/decoding_stage_migration.py:44-68)."""
    off = 0
    for b in range(len(request_ids)):
        n, req = int(num_tokens[b]), int(request_ids[b])
        for j in range(n):
            slot = int(req_to_token_indexes[req, int(b_seq_len[b]) - n + j])
            mem_state[slot] = 0
            send_buf[:, off + j] = kv_cache[:, slot]
        off += n


def decoding_stage_migration_receiver(recv_buf, req_to_token_indexes, kv_cache, alloc_mem, request_ids, num_tokens, b_seq_len) -> None:
    """_fwd_receiver_kernel as loops (decoding_stage_migration.py:133-157)."""
    off = 0
    for b in range(len(request_ids)):
        n, req = int(num_tokens[b]), int(request_ids[b])
        for j in range(n):
            slot = int(alloc_mem[off + j])
            req_to_token_indexes[req, int(b_seq_len[b]) + j] = slot
            kv_cache[:, slot] = recv_buf[:, off + j]
        off += n

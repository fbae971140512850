"""Operators of the attention hot path, with the reference's Python signatures.

Each function validates its tensors, extracts raw device pointers / strides and calls the
C ABI in liblsattn.so on the current PyTorch HIP stream.  Nothing here computes on the
host and nothing falls back to PyTorch math.

Reference call sites (relative to the reference tree):
  loongserve/models/llama/layer_infer/longserve_transformer_layer_infer.py:11-14 imports
  context_attention_fwd, longserve_flash_decode_stage1/2 and
  longserve_token_decode_attention_flash_decoding; :146-160, :272-281, :293-308, :360-367
  call them.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import LSATTN_BF16, LSATTN_F16, LSATTN_F32

_DT = {torch.float16: LSATTN_F16, torch.bfloat16: LSATTN_BF16, torch.float32: LSATTN_F32}


# torch.cuda.current_stream() builds a Stream object through several Python layers (about 8 us a call, more than a small
# decode kernel runs); the raw handle of the same stream comes from one C call where this torch has it
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of the current PyTorch stream of the current device: the launches go there."""
    if _raw_current_stream is not None:
        return _raw_current_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError("%s must live on the GPU (got %s)" % (name, t.device))


def _i32vec(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    _dev(t, name)
    if t.dtype != torch.int32 or t.dim() != 1 or not t.is_contiguous():
        raise ValueError("%s must be a contiguous 1-D int32 tensor" % name)
    if n is not None and t.shape[0] != n:
        raise ValueError("%s must have %d entries" % (name, n))


def _slots(t: torch.Tensor, name: str, n: Optional[int] = None) -> torch.Tensor:
    """A vector of pool slot numbers.  The reference's allocator hands these out as int64 (torch.nonzero /
    arange, loongserve/common/longserve_mem_manager.py:21, :37) while the kernels read int32: an int64 vector is
    narrowed on the device first (pools have fewer than 2**31 slots)."""
    if t.dtype == torch.int64:
        t = t.to(torch.int32)
    _i32vec(t, name, n)
    return t


# A bfloat16 V is rewritten as fp16 before the attention launch (the kernel multiplies P and V in fp16 either way and
# converting inside it costs about 15 % of its speed).  False keeps V as it is and lets the kernel convert.
PRECONVERT_BF16_V = True


def _v_as_f16(v: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp16 copy of a [tokens, heads, head_dim] bfloat16 tensor (any token / head strides), made on the device by
    lsattn_bf16_to_f16_rows into `out` (the caller's contiguous fp16 [tokens, heads, head_dim] buffer; a new tensor if
    None); values beyond fp16's range become +-65504."""
    T, H, D = v.shape
    if out is None:
        out = torch.empty((T, H, D), dtype=torch.float16, device=v.device)
    elif out.dtype != torch.float16 or tuple(out.shape) != (T, H, D) or not out.is_contiguous() or out.device != v.device:
        raise ValueError("v_f16 must be a contiguous float16 tensor of v's shape on v's device")
    if T == 0:
        return out
    lib = _lib.load()
    if v.stride(1) == D:  # heads adjacent: one row per token
        rc = lib.lsattn_bf16_to_f16_rows(v.data_ptr(), v.stride(0), out.data_ptr(), H * D, T, H * D, _stream())
        _lib.check(rc, "lsattn_bf16_to_f16_rows")
    else:
        for hh in range(H):
            rc = lib.lsattn_bf16_to_f16_rows(v[:, hh].data_ptr(), v.stride(0), out[:, hh].data_ptr(), H * D, T, D, _stream())
            _lib.check(rc, "lsattn_bf16_to_f16_rows")
    return out


KERNEL_HEAD_DIM = 128  # the tuned kernel's head size (and the only one whose KV chunks are cut); 16, 32 and 64 take the plain kernel


def _prefill_args(q, k, v, o, q_b_start_loc, q_b_seq_len, q_first, kv_b_start_loc, kv_b_seq_len, kv_first,
                  peers: int, max_q_len: int, sm_scale: Optional[float], v_f16: Optional[torch.Tensor] = None,
                  v_f16_valid: bool = False, o_b_start_loc: Optional[torch.Tensor] = None,
                  cuts: Optional[Tuple[int, int, int]] = None, total_q_len: Optional[int] = None) -> _lib.PrefillArgs:
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (o, "o")):
        _dev(t, n)
        if t.dim() != 3:
            raise ValueError("%s must be [tokens, heads, head_dim]" % n)
        if t.stride(2) != 1:
            raise ValueError("%s must be contiguous in head_dim" % n)
    Lq, Lk, Lv = q.shape[-1], k.shape[-1], v.shape[-1]
    # RING:248-250
    assert Lq == Lk and Lk == Lv
    assert Lk in {16, 32, 64, 128}
    if q.dtype not in (torch.float16, torch.bfloat16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share dtype float16 or bfloat16")
    if k.shape[1] != v.shape[1] or q.shape[1] % k.shape[1] != 0:
        raise ValueError("bad head counts: Hq=%d Hkv=%d" % (q.shape[1], k.shape[1]))
    if o_b_start_loc is None and cuts is None and o.shape != q.shape:
        raise ValueError("o must have the shape of q")
    if cuts is not None and (o.shape[1:] != q.shape[1:] or o.shape[0] < cuts[0] * cuts[2] or cuts[2] < q.shape[0]):
        raise ValueError("o must hold kv_cuts * o_cut_rows rows of q's heads and head_dim")
    if o_b_start_loc is not None and o.shape[1:] != q.shape[1:]:
        raise ValueError("o must have q's heads and head_dim")
    B = q_b_seq_len.shape[0]
    for t, n in ((q_b_start_loc, "q_b_start_loc"), (q_b_seq_len, "q_b_seq_len"), (q_first, "q_first_token_global_idx"),
                 (kv_b_start_loc, "kv_b_start_loc"), (kv_b_seq_len, "kv_b_seq_len"), (kv_first, "kv_first_token_global_idx")):
        _i32vec(t, n, B)
    a = _lib.PrefillArgs()
    # (the kernel for head sizes below 128 converts V as it stages it, at no cost: no copy unless the caller brings one)
    if q.dtype == torch.bfloat16 and ((PRECONVERT_BF16_V and Lq == KERNEL_HEAD_DIM) or v_f16 is not None):
        if v_f16_valid:
            if v_f16 is None or v_f16.dtype != torch.float16 or v_f16.shape != v.shape or v_f16.stride(2) != 1:
                raise ValueError("v_f16_valid needs v_f16, the float16 copy of v")
            v = v_f16
        else:
            v = _v_as_f16(v, v_f16)
        a.v_is_f16 = 1
        a._v_f16 = v  # keeps the copy alive as long as the argument block
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_t, a.k_stride_h = k.stride(0), k.stride(1)
    a.v_stride_t, a.v_stride_h = v.stride(0), v.stride(1)
    a.q_b_start_loc, a.q_b_seq_len, a.q_first_token_global_idx = q_b_start_loc.data_ptr(), q_b_seq_len.data_ptr(), q_first.data_ptr()
    a.kv_b_start_loc, a.kv_b_seq_len, a.kv_first_token_global_idx = kv_b_start_loc.data_ptr(), kv_b_seq_len.data_ptr(), kv_first.data_ptr()
    a.batch, a.num_q_heads, a.num_kv_heads, a.head_dim = B, q.shape[1], k.shape[1], Lq
    a.dtype = _DT[q.dtype]
    a.sp_peers = int(peers)
    a.max_q_len = int(max_q_len)
    a.sm_scale = (1.0 / (Lq ** 0.5)) if sm_scale is None else float(sm_scale)  # RING:252
    a.o = o.data_ptr()
    a.o_stride_t, a.o_stride_h = o.stride(0), o.stride(1)
    a.o_dtype = _DT[o.dtype]
    if o_b_start_loc is not None:
        _i32vec(o_b_start_loc, "o_b_start_loc", B)
        a.o_b_start_loc = o_b_start_loc.data_ptr()
    if cuts is not None:
        a.kv_cuts, a.kv_cut_len, a.o_cut_rows = int(cuts[0]), int(cuts[1]), int(cuts[2])
    if total_q_len is not None:
        if int(total_q_len) < 0:
            raise ValueError("total_q_len must be >= 0")
        a.total_q_rows = int(total_q_len)
    return a


def _cut_workspace(workspace, S: int, Tq: int, Hq: int, D: int, device):
    """(po [S*Tq,Hq,D], pl [S*Tq,Hq]) fp32 views for the partials of S cuts: of `workspace` (one contiguous float32 tensor
    of at least S*Tq*Hq*(D+1) elements, or a pair of tensors of exactly those shapes), or new tensors if it is None."""
    n_o, n_l = S * Tq * Hq * D, S * Tq * Hq
    if workspace is None:
        return (torch.empty((S * Tq, Hq, D), dtype=torch.float32, device=device),
                torch.empty((S * Tq, Hq), dtype=torch.float32, device=device))
    if isinstance(workspace, (tuple, list)):
        po, pl = workspace
        if (po.dtype != torch.float32 or pl.dtype != torch.float32 or tuple(po.shape) != (S * Tq, Hq, D)
                or tuple(pl.shape) != (S * Tq, Hq) or not po.is_contiguous() or not pl.is_contiguous()):
            raise ValueError("workspace pair: contiguous float32 [S*Tq,Hq,D] and [S*Tq,Hq]")
        _dev(po, "workspace"); _dev(pl, "workspace")
        return po, pl
    _dev(workspace, "workspace")
    if workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.numel() < n_o + n_l:
        raise ValueError("workspace: a contiguous float32 tensor of at least S*Tq*Hq*(D+1) = %d elements" % (n_o + n_l))
    flat = workspace.view(-1)
    return flat[:n_o].view(S * Tq, Hq, D), flat[n_o:n_o + n_l].view(S * Tq, Hq)


def _workspace_cuts(workspace, Tq: int, Hq: int, D: int) -> int:
    """How many cuts' partials a single-tensor workspace holds."""
    if workspace is None or isinstance(workspace, (tuple, list)) or Tq == 0:
        return _lib.LSATTN_MAX_KV_CUTS
    return workspace.numel() // (Tq * Hq * (D + 1))


def _merge_cuts(po, pl, S: int, Tq: int, q_b_start_loc, q_b_seq_len, max_q_len: int, mode: int, o, lse=None, m=None, l=None):
    a = _lib.MergeCutsArgs()
    a.o_parts, a.lse_parts, a.part_rows, a.n_parts, a.mode = po.data_ptr(), pl.data_ptr(), Tq, S, mode
    a.batch, a.num_q_heads, a.head_dim, a.max_q_len = q_b_seq_len.shape[0], po.shape[1], po.shape[2], int(max_q_len)
    a.q_b_start_loc, a.q_b_seq_len = q_b_start_loc.data_ptr(), q_b_seq_len.data_ptr()
    a.o, a.o_stride_t, a.o_stride_h, a.o_dtype = o.data_ptr(), o.stride(0), o.stride(1), _DT[o.dtype]
    if mode == 1:
        a.m, a.l, a.ml_stride_t, a.ml_stride_h = m.data_ptr(), l.data_ptr(), m.stride(0), m.stride(1)
    else:
        a.lse = lse.data_ptr()
    _lib.check(_lib.load().lsattn_prefill_merge_cuts(C.byref(a), _stream()), "lsattn_prefill_merge_cuts")


# Launches below this many 128-row workgroups (batch x query heads x ceil(max_q / 128)) are cut along the keys when the
# KV chunks may hold at least KV_SPLIT_MIN_KEYS keys: 256 CUs run one workgroup each.
KV_SPLIT_BELOW_WORKGROUPS = 192
KV_SPLIT_ROUND = 256  # workgroups of a cut launch that run at once: one per CU
KV_SPLIT_MIN_KEYS = 8192


def kv_split_count(batch: int, num_q_heads: int, max_q_len: int, kv_rows: int, num_kv_heads: Optional[int] = None) -> int:
    """KV cuts the prefill operators use by themselves: the count that leaves the longest chain of tiles on a CU shortest
    when the launch's workgroups run in rounds of 256 (one per CU), the smaller count on ties, with cuts of at least 4096
    keys (kv_rows bounds every sequence's chunk: max_kv_len where the caller gives it, else the rows of the k buffer; the
    lengths themselves live on the device).  The launch's size without cuts is counted in 128-row workgroups as the
    kernel forms them: up to four query heads of a KV head side by side (num_kv_heads given), 128 / that many positions each."""
    pack = 1
    if num_kv_heads:
        group = num_q_heads // num_kv_heads
        while pack < 4 and group % (2 * pack) == 0:
            pack *= 2
    wgs = batch * (num_q_heads // pack) * ((max_q_len + 128 // pack - 1) // (128 // pack))
    if wgs <= 0 or wgs >= KV_SPLIT_BELOW_WORKGROUPS or kv_rows < KV_SPLIT_MIN_KEYS:
        return 1
    # rounds(S) / S of the uncut chain is what a CU walks with S cuts.  (measured, GQA 32/8 unless said: 16 rows x 131072 keys
    # 32 cuts 124 us against 134 with 16 and 160 with 64; 100 x 131072 8 cuts 252, 10 cuts 285, 16 cuts 243, 32 cuts 270, MHA 8 cuts 388
    # against 412 with 16; 128 x 32768 8 cuts 80 against 84 with 16)
    best, best_cost = 1, None
    for S in range(1, max(1, min(_lib.LSATTN_MAX_KV_CUTS, kv_rows // 4096)) + 1):
        # (and every cut adds a part to write and to merge: about a thousandth of the uncut chain each in the cases above)
        cost = (-(-wgs * S // KV_SPLIT_ROUND)) / S + 0.001 * S
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = S, cost
    return best


def _cut_len(kv_rows: int, S: int) -> int:
    """Keys per cut: kv_rows over S cuts, rounded up to the kernel's 64-key tile."""
    return -(-(-(-kv_rows // S)) // 64) * 64


@torch.inference_mode()
def context_attention_fwd(q, k, v, o, q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                          kv_b_start_loc, kv_b_seq_len, kv_first_token_global_idx,
                          logical_sp_peers_num: int, max_q_b_seq_len: int, m, l, *, v_f16: Optional[torch.Tensor] = None,
                          v_f16_valid: bool = False, workspace=None, max_kv_len: Optional[int] = None,
                          kv_splits: Optional[int] = None, total_q_len: Optional[int] = None) -> None:
    """One ring-attention step folded in place into (o, m, l); signature of RING:191-206.

    Keyword-only additions for bfloat16 inputs (the reference is fp16 only): the kernel multiplies P and V in fp16, so V is
    rewritten as fp16 first.  v_f16 is the caller's buffer for that copy (contiguous float16, v's shape): with it the call
    allocates nothing; v_f16_valid=True says it already holds the copy of this v (e.g. from an earlier step over the same
    chunk) and skips the conversion.

    Keyword-only, for short query chunks against a long KV chunk (a chunked-prefill step of a long request): the launch has
    one workgroup per 128 query rows and head, too few for the chip.  With workspace (a contiguous float32 tensor the caller
    owns, S * Tq * Hq * (D + 1) elements for S cuts; or a pair of tensors [S*Tq,Hq,D], [S*Tq,Hq]) the KV chunks are cut
    into S slices inside one launch that writes S fp32 partials per row to the workspace, and a second launch folds
    them into (o, m, l) by the same update (RING:171-188).  S follows kv_split_count (from shapes alone; max_kv_len, an
    upper bound of every chunk's length, replaces the rows of the k buffer there: in the layer k is a view of a buffer
    sized for the longest batch), capped by what the workspace holds; kv_splits forces it.  Without a workspace the call
    is the reference's: one launch, no scratch.  (m, l) stay opaque: a step folded this way enters as (its LSE, 1).

    Keyword-only, for batches that mix long and short requests: total_q_len, an upper bound of the sum of q_b_seq_len
    (q.shape[0] when q is packed and no two sequences share rows).  The launch is sized by max_q_b_seq_len times the batch
    (RING:262), all the host knows; with the bound it is sized by the query tiles that can exist when those are at most half
    as many.  A bound below the real sum leaves rows uncomputed.

    Call it repeatedly with the same local q/o/m/l and a different kv chunk each time.
    Start from m = -inf, l = 0 (o need not be zeroed).  After k calls o is the
    normalised attention output over all keys seen and ln2*(m + log2 l) their LSE.
    """
    if o.dtype != q.dtype:
        raise ValueError("o must have the dtype of q")
    D = q.shape[-1]
    for t, n in ((m, "m"), (l, "l")):
        _dev(t, n)
        if t.dtype != torch.float32 or t.dim() != 2 or tuple(t.shape) != (q.shape[0], q.shape[1]):
            raise ValueError("%s must be float32 [tokens, q_heads]" % n)
    if m.stride() != l.stride():
        raise ValueError("m and l must share strides")
    S = 1
    if workspace is not None and D == KERNEL_HEAD_DIM and q.dim() == 3:
        kv_rows = k.shape[0] if max_kv_len is None else int(max_kv_len)
        S = kv_split_count(q_b_seq_len.shape[0], q.shape[1], int(max_q_b_seq_len), kv_rows, k.shape[1]) if kv_splits is None else int(kv_splits)
        S = min(S, _workspace_cuts(workspace, q.shape[0], q.shape[1], D), _lib.LSATTN_MAX_KV_CUTS)
    if S > 1:
        Tq = q.shape[0]
        po, pl = _cut_workspace(workspace, S, Tq, q.shape[1], D, q.device)
        a = _prefill_args(q, k, v, po, q_b_start_loc, q_b_seq_len, q_first_token_global_idx, kv_b_start_loc,
                          kv_b_seq_len, kv_first_token_global_idx, logical_sp_peers_num, max_q_b_seq_len,
                          1.0 / (D ** 0.5), v_f16, v_f16_valid, cuts=(S, _cut_len(kv_rows, S), Tq))
        a.lse = pl.data_ptr()
        if o.dim() != 3 or o.stride(2) != 1:
            raise ValueError("o must be [tokens, heads, head_dim], contiguous in head_dim")
        _lib.check(_lib.load().lsattn_prefill_step(C.byref(a), _stream()), "lsattn_prefill_step")
        _merge_cuts(po, pl, S, Tq, q_b_start_loc, q_b_seq_len, max_q_b_seq_len, 1, o, m=m, l=l)
        return
    a = _prefill_args(q, k, v, o, q_b_start_loc, q_b_seq_len, q_first_token_global_idx, kv_b_start_loc,
                      kv_b_seq_len, kv_first_token_global_idx, logical_sp_peers_num, max_q_b_seq_len,
                      1.0 / (D ** 0.5), v_f16, v_f16_valid, total_q_len=total_q_len)
    a.m, a.l = m.data_ptr(), l.data_ptr()
    a.ml_stride_t, a.ml_stride_h = m.stride(0), m.stride(1)
    _lib.check(_lib.load().lsattn_prefill_step_merge(C.byref(a), _stream()), "lsattn_prefill_step_merge")


@torch.inference_mode()
def prefill_attention_step(q, k, v, q_b_start_loc, q_b_seq_len, q_first_token_global_idx,
                           kv_b_start_loc, kv_b_seq_len, kv_first_token_global_idx,
                           logical_sp_peers_num: int, max_q_b_seq_len: int,
                           out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                           sm_scale: Optional[float] = None, accumulate: bool = False, v_f16: Optional[torch.Tensor] = None,
                           v_f16_valid: bool = False, kv_splits: Optional[int] = None,
                           kv_split_workspace=None, max_kv_len: Optional[int] = None,
                           total_q_len: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """One step as a mergeable partial: (O fp32 [Tq,Hq,D] normalised, LSE fp32 [Tq,Hq]).
    v_f16 / v_f16_valid: as in context_attention_fwd (the caller's buffer for the fp16 copy of a bfloat16 v).
    kv_splits: short query chunks against a long KV chunk give the launch too few workgroups for the chip (one per 128
    query rows and head); with kv_splits = S > 1 every sequence's KV chunk is cut into S slices inside one launch, which
    computes the S partials of every row (lsattn_prefill_args.kv_cuts), and lsattn_prefill_merge_cuts joins them for the
    rows of the sequences.  None chooses S from the shapes (kv_split_count over max_kv_len, an upper bound of every
    chunk's length; the rows of the k buffer if not given), 1 switches it off.  The partials take S times the size of
    (out, lse): kv_split_workspace passes the caller's memory for them (as context_attention_fwd's workspace).

    Same inputs as context_attention_fwd; rows that see no key get O = 0, LSE = -inf.
    total_q_len: as in context_attention_fwd (an upper bound of the rows of all sequences together, for skewed batches).
    With accumulate=True the step is LSE-merged into the (out, lse) passed in (a running partial of earlier steps over
    other keys; lse = -inf marks an empty row) in the kernel's epilogue, instead of being written from the empty state;
    rows that see no key in this step keep what they hold.
    """
    if accumulate and (out is None or lse is None):
        raise ValueError("accumulate=True needs the running out and lse")
    D = q.shape[-1]
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    if lse is None:
        lse = torch.empty(q.shape[:2], dtype=torch.float32, device=q.device)
    if out.dtype != torch.float32 or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("out and lse must be float32, lse contiguous")
    kv_rows = k.shape[0] if max_kv_len is None else int(max_kv_len)
    S = kv_split_count(q_b_seq_len.shape[0], q.shape[1], int(max_q_b_seq_len), kv_rows, k.shape[1]) if kv_splits is None else int(kv_splits)
    if D != KERNEL_HEAD_DIM:
        S = 1  # (the cut along the keys is the 128-wide kernel's)
    if S > 1:
        if S > _lib.LSATTN_MAX_KV_CUTS:
            raise ValueError("at most %d KV slices" % _lib.LSATTN_MAX_KV_CUTS)
        if out.dim() != 3 or out.stride(2) != 1 or tuple(out.shape) != tuple(q.shape):
            raise ValueError("out must have q's shape and be contiguous in head_dim")
        Tq = q.shape[0]
        po, pl = _cut_workspace(kv_split_workspace, S, Tq, q.shape[1], q.shape[2], q.device)
        a = _prefill_args(q, k, v, po, q_b_start_loc, q_b_seq_len, q_first_token_global_idx, kv_b_start_loc, kv_b_seq_len,
                          kv_first_token_global_idx, logical_sp_peers_num, max_q_b_seq_len, sm_scale,
                          v_f16, v_f16_valid, cuts=(S, _cut_len(kv_rows, S), Tq))
        a.lse = pl.data_ptr()
        _lib.check(_lib.load().lsattn_prefill_step(C.byref(a), _stream()), "lsattn_prefill_step")
        _merge_cuts(po, pl, S, Tq, q_b_start_loc, q_b_seq_len, max_q_b_seq_len, 2 if accumulate else 0, out, lse=lse)
        return out, lse
    a = _prefill_args(q, k, v, out, q_b_start_loc, q_b_seq_len, q_first_token_global_idx, kv_b_start_loc,
                      kv_b_seq_len, kv_first_token_global_idx, logical_sp_peers_num, max_q_b_seq_len, sm_scale,
                      v_f16, v_f16_valid, total_q_len=total_q_len)
    a.lse = lse.data_ptr()
    if accumulate:
        _lib.check(_lib.load().lsattn_prefill_step_accumulate(C.byref(a), _stream()), "lsattn_prefill_step_accumulate")
    else:
        _lib.check(_lib.load().lsattn_prefill_step(C.byref(a), _stream()), "lsattn_prefill_step")
    return out, lse


@torch.inference_mode()
def lse_merge(parts: Sequence[Tuple[torch.Tensor, torch.Tensor]], out: Optional[torch.Tensor] = None,
              lse: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float32):
    """Merge partials [(O_i fp32 [..., D], LSE_i [...])] over disjoint key sets -> (O, LSE)."""
    n = len(parts)
    if not 1 <= n <= _lib.LSATTN_MAX_PARTS:
        raise ValueError("1..%d partials" % _lib.LSATTN_MAX_PARTS)
    o0, l0 = parts[0]
    a = _lib.MergeArgs()
    for i, (oi, li) in enumerate(parts):
        _dev(oi, "partial O")
        if oi.dtype != torch.float32 or li.dtype != torch.float32 or not oi.is_contiguous() or not li.is_contiguous():
            raise ValueError("partials must be contiguous float32")
        if oi.shape != o0.shape or li.shape != l0.shape or oi.shape[:-1] != li.shape:
            raise ValueError("partials must share shapes")
        a.o_parts[i] = oi.data_ptr()
        a.lse_parts[i] = li.data_ptr()
    if out is None:
        out = torch.empty(o0.shape, dtype=out_dtype, device=o0.device)
    if lse is None:
        lse = torch.empty(l0.shape, dtype=torch.float32, device=o0.device)
    if not out.is_contiguous() or not lse.is_contiguous() or out.shape != o0.shape or lse.dtype != torch.float32:
        raise ValueError("bad output tensors")
    a.n_parts, a.head_dim, a.rows = n, o0.shape[-1], l0.numel()
    a.o, a.o_dtype, a.lse = out.data_ptr(), _DT[out.dtype], lse.data_ptr()
    _lib.check(_lib.load().lsattn_lse_merge(C.byref(a), _stream()), "lsattn_lse_merge")
    return out, lse


@torch.inference_mode()
def kv_scatter(src: torch.Tensor, dest_index: torch.Tensor, pool: torch.Tensor) -> None:
    """pool[dest_index[i]] = src[i] (bit-exact row scatter into the token-indexed pool).

    Semantics of destindex_copy_kv
    (loongserve/common/basemodel/triton_kernel/destindex_copy_kv.py:31-51).
    """
    _dev(src, "src"); _dev(pool, "pool")
    dest_index = _slots(dest_index, "dest_index", src.shape[0])
    if src.dtype != pool.dtype or src.shape[1:] != pool.shape[1:]:
        raise ValueError("src and pool rows must match")
    if src.shape[0] == 0:
        return  # an empty chunk writes nothing
    if pool.shape[0] == 0 or not src[0].is_contiguous() or not pool[0].is_contiguous():
        raise ValueError("rows must be contiguous")
    row_bytes = src[0].numel() * src.element_size()
    rc = _lib.load().lsattn_kv_scatter(src.data_ptr(), src.stride(0) * src.element_size(), pool.data_ptr(),
                                       pool.stride(0) * pool.element_size(), dest_index.data_ptr(),
                                       src.shape[0], row_bytes, _stream())
    _lib.check(rc, "lsattn_kv_scatter")


def rmsnorm_forward(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Name and signature of the Triton operator behind the final norm
    (loongserve/models/llama/triton_kernel/rmsnorm.py:41-63, called
    loongserve/models/llama/layer_infer/longserve_post_layer_infer.py:35): a new tensor y = x / rms(x) * weight over the
    last dimension.  Runs the same kernel as longserve_cuda_kernels.rms_norm."""
    from .longserve_cuda_kernels import rms_norm
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    return rms_norm(x.view(-1, x.shape[-1]), weight, eps).view(x.shape)


def rotary_emb_fwd(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    """Name and signature of the Triton rotary operator (loongserve/models/llama/triton_kernel/rotary_emb.py:119); nothing in
    the reference calls it (the layer uses longserve_cuda_kernels.rotary_emb, which this runs)."""
    from .longserve_cuda_kernels import rotary_emb
    rotary_emb(q, k, cos, sin)


def silu_and_mul_fwd(input: torch.Tensor) -> torch.Tensor:
    """Name and signature of the Triton operator (loongserve/models/llama/triton_kernel/silu_and_mul.py:50-74): in place
    on the first half of the columns, which is returned as a view; nothing in the reference calls it (ffn_block does the
    same through longserve_cuda_kernels.silu_and_mul_inplace, which this runs)."""
    from .longserve_cuda_kernels import silu_and_mul_inplace
    silu_and_mul_inplace(input)
    return input[:, 0:(input.shape[-1] // 2)]


def destindex_copy_kv(K: torch.Tensor, DestLoc: torch.Tensor, Out: torch.Tensor) -> None:
    """Out[DestLoc[i]] = K[i]: name and argument order of the operator the layer calls to persist a step's K/V rows
    (loongserve/common/basemodel/triton_kernel/destindex_copy_kv.py:32, called
    loongserve/models/llama/layer_infer/longserve_transformer_layer_infer.py:377)."""
    kv_scatter(K, DestLoc, Out)


@torch.inference_mode()
def rotary_emb_write_kv(q: torch.Tensor, cache_kv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                        mem_index: Optional[torch.Tensor] = None, pool: Optional[torch.Tensor] = None,
                        req_to_token_indexs: Optional[torch.Tensor] = None, b_req_idx: Optional[torch.Tensor] = None,
                        b_seq_len: Optional[torch.Tensor] = None, b_start_loc: Optional[torch.Tensor] = None,
                        max_len_in_batch: Optional[int] = None, decode: bool = False) -> None:
    """A step's write-back of its new tokens in one launch (lsattn_rotary_kv_write) instead of the three operators the
    layer calls one after the other:
      longserve_cuda_kernels.rotary_emb(q, cache_kv[:, :Hkv], cos, sin)           (..._layer_infer.py:88-93), in place;
      destindex_copy_kv(cache_kv, mem_index, pool)                                (..._layer_infer.py:377), if pool is given;
      init_req_to_token_indexes(req_to_token_indexs, b_req_idx, b_seq_len, mem_index)  (prefill, decode=False) or
      copy_kv_index_to_req(req_to_token_indexs, b_req_idx, b_seq_len, mem_index)       (decode=True), if the table is given.
    q [T, Hq, D], cache_kv [T, 2*Hkv, D] (K heads then V heads), float16; the results are those of the separate
    operators bit for bit."""
    for t, n in ((q, "q"), (cache_kv, "cache_kv")):
        _dev(t, n)
        if t.dim() != 3 or t.dtype != torch.float16 or t.stride(2) != 1:
            raise ValueError("%s must be a 3-d float16 tensor with a contiguous last dimension" % n)
    T, Hq, D = q.shape
    if cache_kv.shape[0] != T or cache_kv.shape[2] != D or cache_kv.shape[1] % 2:
        raise ValueError("cache_kv must be [tokens, 2 * kv_heads, head_dim] for q's tokens and head_dim")
    for t, n in ((cos, "cos"), (sin, "sin")):
        _dev(t, n)
        if t.dtype != torch.float16 or tuple(t.shape) != (T, D // 2) or not t.is_contiguous():
            raise ValueError("%s must be a contiguous float16 [tokens, head_dim / 2] tensor" % n)
    a = _lib.RotaryKvWriteArgs()
    a.q, a.q_stride_t, a.q_stride_h, a.num_q_heads = q.data_ptr(), q.stride(0), q.stride(1), Hq
    a.kv, a.kv_stride_t, a.kv_stride_h, a.num_kv_heads = cache_kv.data_ptr(), cache_kv.stride(0), cache_kv.stride(1), cache_kv.shape[1] // 2
    a.cos, a.sin, a.num_tokens, a.head_dim = cos.data_ptr(), sin.data_ptr(), T, D
    keep = []
    if mem_index is not None:
        mem_index = _slots(mem_index, "mem_index")
        keep.append(mem_index)
        a.dest_index = mem_index.data_ptr()
    if pool is not None:
        _dev(pool, "pool")
        if mem_index is None or mem_index.shape[0] != T:
            raise ValueError("mem_index must name one slot per token")
        if pool.dtype != torch.float16 or pool.shape[1:] != cache_kv.shape[1:] or (pool.shape[0] and not pool[0].is_contiguous()):
            raise ValueError("pool must be float16 [slots, 2 * kv_heads, head_dim] with contiguous slots")
        a.pool, a.pool_slot_stride = pool.data_ptr(), pool.stride(0)
    if req_to_token_indexs is not None:
        _dev(req_to_token_indexs, "req_to_token_indexs")
        if req_to_token_indexs.dtype != torch.int32 or req_to_token_indexs.dim() != 2 or not req_to_token_indexs.is_contiguous():
            raise ValueError("req_to_token_indexs must be a contiguous [max_req, max_seq] int32 tensor")
        if mem_index is None or b_req_idx is None or b_seq_len is None:
            raise ValueError("registration needs mem_index, b_req_idx and b_seq_len")
        B = b_req_idx.shape[0]
        _i32vec(b_req_idx, "b_req_idx", B); _i32vec(b_seq_len, "b_seq_len", B)
        a.req_to_tokens, a.max_seq_len = req_to_token_indexs.data_ptr(), req_to_token_indexs.shape[1]
        a.b_req_idx, a.b_seq_len, a.batch = b_req_idx.data_ptr(), b_seq_len.data_ptr(), B
        if decode:
            if mem_index.shape[0] != B:
                raise ValueError("decode registration: one slot per request")
            a.register_mode = 2
        else:
            if b_start_loc is None:
                b_start_loc = (torch.cumsum(b_seq_len, 0, dtype=torch.int32) - b_seq_len).to(torch.int32)
            if max_len_in_batch is None:
                max_len_in_batch = int(b_seq_len.max().item()) if B else 0
            _i32vec(b_start_loc, "b_start_loc", B)
            keep.append(b_start_loc)
            a.b_start_loc, a.max_len_in_batch, a.register_mode = b_start_loc.data_ptr(), int(max_len_in_batch), 1
    _lib.check(_lib.load().lsattn_rotary_kv_write(C.byref(a), _stream()), "lsattn_rotary_kv_write")


@torch.inference_mode()
def copy_kv_index_to_req(req_to_token_indexs: torch.Tensor, b_req_idx: torch.Tensor, b_seq_len: torch.Tensor,
                         memindex: torch.Tensor) -> None:
    """req_to_token_indexs[b_req_idx[i], b_seq_len[i] - 1] = memindex[i]: registers the slot of each request's new token
    in the decoding stage (loongserve/common/basemodel/triton_kernel/copy_kv_index_to_req.py:22-40, called
    loongserve/models/llama/longserve_model.py:491, :497).  memindex is int32 or, as the allocator returns it, int64."""
    _dev(req_to_token_indexs, "req_to_token_indexs"); _dev(memindex, "memindex")
    B = b_seq_len.shape[0]
    assert b_seq_len.shape[0] == memindex.shape[0] and b_req_idx.shape[0] == b_seq_len.shape[0]  # as the reference
    _i32vec(b_req_idx, "b_req_idx", B); _i32vec(b_seq_len, "b_seq_len", B)
    if req_to_token_indexs.dtype != torch.int32 or req_to_token_indexs.dim() != 2 or not req_to_token_indexs.is_contiguous():
        raise ValueError("req_to_token_indexs must be a contiguous [max_req, max_seq] int32 tensor")
    if memindex.dtype not in (torch.int32, torch.int64) or memindex.dim() != 1 or not memindex.is_contiguous():
        raise ValueError("memindex must be a contiguous 1-D int32 or int64 tensor")
    rc = _lib.load().lsattn_register_decode_tokens(req_to_token_indexs.data_ptr(), req_to_token_indexs.shape[1],
                                                   b_req_idx.data_ptr(), b_seq_len.data_ptr(), memindex.data_ptr(),
                                                   1 if memindex.dtype == torch.int64 else 0, B, _stream())
    _lib.check(rc, "lsattn_register_decode_tokens")


@torch.inference_mode()
def init_req_to_token_indexes(req_to_token_indexs, b_req_idx, b_seq_len, alloc_mem_index,
                              b_start_loc: Optional[torch.Tensor] = None, max_len_in_batch: Optional[int] = None) -> None:
    """req_to_token_indexs[req_b, 0:len_b] = alloc_mem_index[start_b : start_b+len_b] on the device.

    Signature of loongserve/common/infer_utils.py:1 plus two optional arguments that avoid
    a host round trip (packed start offsets and the longest length)."""
    _dev(req_to_token_indexs, "req_to_token_indexs")
    if req_to_token_indexs.dtype != torch.int32 or not req_to_token_indexs.is_contiguous():
        raise ValueError("req_to_token_indexs must be contiguous int32")
    B = b_req_idx.shape[0]
    _i32vec(b_req_idx, "b_req_idx", B); _i32vec(b_seq_len, "b_seq_len", B)
    alloc_mem_index = _slots(alloc_mem_index, "alloc_mem_index")
    if b_start_loc is None:
        b_start_loc = (torch.cumsum(b_seq_len, 0, dtype=torch.int32) - b_seq_len).to(torch.int32)
    if max_len_in_batch is None:
        max_len_in_batch = int(b_seq_len.max().item()) if B else 0
    _i32vec(b_start_loc, "b_start_loc", B)
    rc = _lib.load().lsattn_register_tokens(req_to_token_indexs.data_ptr(), req_to_token_indexs.shape[1],
                                            b_req_idx.data_ptr(), b_start_loc.data_ptr(), b_seq_len.data_ptr(),
                                            alloc_mem_index.data_ptr(), B, max_len_in_batch, _stream())
    _lib.check(rc, "lsattn_register_tokens")


@torch.inference_mode()
def pre_copy_and_register_kv(kv_cache_index_begin: torch.Tensor, kv_cache_index_end: torch.Tensor,
                             kv_first_token_global_idx: torch.Tensor, num_logical_sp_peers: int):
    """(kv_range_begin, kv_range_end, new_kv_cache_len): the locally held rows of each request that fall in
    the cache-index window, with local row n holding global token first + n * peers.

    Signature and results of pre_copy_and_register_kv
    (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:34-62)."""
    B = kv_cache_index_begin.shape[0]
    _i32vec(kv_cache_index_begin, "kv_cache_index_begin", B); _i32vec(kv_cache_index_end, "kv_cache_index_end", B)
    _i32vec(kv_first_token_global_idx, "kv_first_token_global_idx", B)
    rb, re, nl = (torch.empty_like(kv_cache_index_begin) for _ in range(3))
    if B == 0:
        return rb, re, nl
    rc = _lib.load().lsattn_kv_ranges(kv_cache_index_begin.data_ptr(), kv_cache_index_end.data_ptr(),
                                      kv_first_token_global_idx.data_ptr(), int(num_logical_sp_peers), B,
                                      rb.data_ptr(), re.data_ptr(), nl.data_ptr(), _stream())
    _lib.check(rc, "lsattn_kv_ranges")
    return rb, re, nl


@torch.inference_mode()
def destindex_copy_and_register_kv(batch_size: int, new_kv_cache_len: torch.Tensor, kv_range_begin: torch.Tensor,
                                   kv_range_end: torch.Tensor, new_kv_cache_len_sum: torch.Tensor, kv: torch.Tensor,
                                   kv_b_start_loc: torch.Tensor, cur_kv_cache_index: torch.Tensor, mem_index: torch.Tensor,
                                   total_kv_cache: torch.Tensor, req_to_token_indexs: torch.Tensor, b_req_idx: torch.Tensor,
                                   num_used_mem_index: int, max_len_in_batch: int, should_register_kv: bool) -> None:
    """Copy the migrating KV rows of every request into their pool slots and, on the first layer, register
    the slots in the request table.

    Signature and semantics of destindex_copy_and_register_kv
    (loongserve/models/llama/triton_kernel/copy_and_register_kv.py:119-170)."""
    B = int(batch_size)
    if B == 0:
        return
    for t, name in ((new_kv_cache_len, "new_kv_cache_len"), (kv_range_begin, "kv_range_begin"), (kv_range_end, "kv_range_end"),
                    (kv_b_start_loc, "kv_b_start_loc"), (cur_kv_cache_index, "cur_kv_cache_index"), (b_req_idx, "b_req_idx")):
        _i32vec(t, name, B)
    mem_index = _slots(mem_index, "mem_index")
    _dev(new_kv_cache_len_sum, "new_kv_cache_len_sum")
    if new_kv_cache_len_sum.dtype != torch.int64 or new_kv_cache_len_sum.shape != (B,) or not new_kv_cache_len_sum.is_contiguous():
        raise ValueError("new_kv_cache_len_sum must be a contiguous int64 vector of length batch_size")
    _dev(kv, "kv"); _dev(total_kv_cache, "total_kv_cache"); _dev(req_to_token_indexs, "req_to_token_indexs")
    if kv.dtype != total_kv_cache.dtype or kv.shape[1:] != total_kv_cache.shape[1:]:
        raise ValueError("kv and total_kv_cache rows must match")
    if kv.shape[0] == 0:
        return  # no rows held: nothing can migrate
    if total_kv_cache.shape[0] == 0 or not kv[0].is_contiguous() or not total_kv_cache[0].is_contiguous():
        raise ValueError("rows must be contiguous")
    if req_to_token_indexs.dtype != torch.int32 or not req_to_token_indexs.is_contiguous():
        raise ValueError("req_to_token_indexs must be contiguous int32")
    a = _lib.KvCopyRegisterArgs()
    a.kv, a.kv_stride_bytes = kv.data_ptr(), kv.stride(0) * kv.element_size()
    a.pool, a.pool_stride_bytes = total_kv_cache.data_ptr(), total_kv_cache.stride(0) * total_kv_cache.element_size()
    a.row_bytes = kv[0].numel() * kv.element_size()
    a.new_kv_cache_len, a.kv_range_begin, a.kv_range_end = new_kv_cache_len.data_ptr(), kv_range_begin.data_ptr(), kv_range_end.data_ptr()
    a.new_kv_cache_len_sum, a.kv_b_start_loc = new_kv_cache_len_sum.data_ptr(), kv_b_start_loc.data_ptr()
    a.cur_kv_cache_index, a.mem_index, a.b_req_idx = cur_kv_cache_index.data_ptr(), mem_index.data_ptr(), b_req_idx.data_ptr()
    a.req_to_tokens, a.max_seq_len = req_to_token_indexs.data_ptr(), req_to_token_indexs.shape[1]
    a.batch, a.num_used_mem_index, a.max_len_in_batch = B, int(num_used_mem_index), int(max_len_in_batch)
    a.should_register = 1 if should_register_kv else 0
    rc = _lib.load().lsattn_kv_copy_register(C.byref(a), _stream())
    _lib.check(rc, "lsattn_kv_copy_register")


def _migration_args(buf, req_to_token_indexes, kv_cache, request_ids, num_tokens, b_seq_len):
    B = request_ids.shape[0]
    for t, name in ((request_ids, "request_ids"), (num_tokens, "num_tokens"), (b_seq_len, "b_seq_len")):
        _i32vec(t, name, B)
    _dev(buf, "buffer"); _dev(kv_cache, "kv_cache"); _dev(req_to_token_indexes, "req_to_token_indexes")
    if kv_cache.dim() != 4 or buf.dim() != 4 or buf.dtype != kv_cache.dtype or buf.shape[0] != kv_cache.shape[0] or \
            buf.shape[2:] != kv_cache.shape[2:]:
        raise ValueError("buffer [layers, tokens, 2*heads, head_dim] and kv_cache [layers, slots, 2*heads, head_dim] must match")
    if not buf[0, 0].is_contiguous() or not kv_cache[0, 0].is_contiguous():
        raise ValueError("rows must be contiguous")
    if req_to_token_indexes.dtype != torch.int32 or not req_to_token_indexes.is_contiguous():
        raise ValueError("req_to_token_indexes must be contiguous int32")
    a = _lib.DecodeMigrationArgs()
    es = kv_cache.element_size()
    a.staging, a.staging_layer_stride_bytes, a.staging_row_stride_bytes = buf.data_ptr(), buf.stride(0) * es, buf.stride(1) * es
    a.kv_cache, a.kv_layer_stride_bytes, a.kv_row_stride_bytes = kv_cache.data_ptr(), kv_cache.stride(0) * es, kv_cache.stride(1) * es
    a.row_bytes, a.num_layers = kv_cache[0, 0].numel() * es, kv_cache.shape[0]
    a.req_to_tokens, a.max_seq_len = req_to_token_indexes.data_ptr(), req_to_token_indexes.shape[1]
    cumsum = torch.cumsum(num_tokens, dim=0, dtype=torch.int32)
    a.request_ids, a.num_tokens, a.num_tokens_cumsum, a.b_seq_len = request_ids.data_ptr(), num_tokens.data_ptr(), cumsum.data_ptr(), b_seq_len.data_ptr()
    a.batch = B
    # the launch is sized by the longest migration, read back like the reference's torch.max(num_tokens) grid dimension
    a.max_num_tokens = int(num_tokens.max().item()) if B > 0 else 0
    return a, cumsum


@torch.inference_mode()
def decoding_stage_migration_sender_kernel(send_buf, req_to_token_indexes, mem_state, kv_cache, request_ids, num_tokens, b_seq_len) -> None:
    """Gather the last num_tokens[b] tokens of every request from every layer of kv_cache into send_buf and mark their
    slots free.  Signature of decoding_stage_migration_sender_kernel
    (loongserve/models/llama/triton_kernel/decoding_stage_migration.py:70-98)."""
    if request_ids.shape[0] == 0:
        return
    _i32vec(mem_state, "mem_state")
    a, keep = _migration_args(send_buf, req_to_token_indexes, kv_cache, request_ids, num_tokens, b_seq_len)
    a.mem_state = mem_state.data_ptr()
    _lib.check(_lib.load().lsattn_decode_migration_send(C.byref(a), _stream()), "lsattn_decode_migration_send")


@torch.inference_mode()
def decoding_stage_migration_receiver_kernel(recv_buf, req_to_token_indexes, kv_cache, alloc_mem, request_ids, num_tokens, b_seq_len) -> None:
    """Store recv_buf into the freshly allocated slots of every layer of kv_cache and append the slots to the request
    table.  Signature of decoding_stage_migration_receiver_kernel
    (loongserve/models/llama/triton_kernel/decoding_stage_migration.py:159-183)."""
    if request_ids.shape[0] == 0:
        return
    alloc_mem = _slots(alloc_mem, "alloc_mem")
    a, keep = _migration_args(recv_buf, req_to_token_indexes, kv_cache, request_ids, num_tokens, b_seq_len)
    a.alloc_mem = alloc_mem.data_ptr()
    _lib.check(_lib.load().lsattn_decode_migration_recv(C.byref(a), _stream()), "lsattn_decode_migration_recv")

"""Stand-in for the `longserve_cuda_kernels` extension module.

Exports flash_decoding_stage1 / flash_decoding_stage2 with the argument order and the
tensor checks of longserve_cuda_kernels/src/entrypoints.cpp:103-221, and rms_norm,
silu_and_mul_inplace, rotary_emb, ffn_block, hello_world (:15-101, :228-241).  A failed
check raises ValueError instead of aborting the process (the reference calls
__assert_fail, longserve_cuda_kernels/src/common.h:29-32).
Beyond the reference: q/k/v may be bfloat16, stage-2 `o` may be bfloat16, and
flash_decoding runs both decode stages from one library call.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from . import _lib
from .ops import _DT, _stream


def _req(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError("longserve_cuda_kernels: check failed: " + what)


def _stage1_args(mid_o, mid_o_logexpsum, q, k, v, req_to_tokens, b_req_idx, b_seqlen,
                 max_len_in_batch: int, seq_block_size: int, merge_blocks: int = 1,
                 partials_in_library: bool = False) -> _lib.DecodeStage1Args:
    """The checks of ENTRY:115-160 and the argument block of lsattn_decode_stage1.  partials_in_library: mid_o and
    mid_o_logexpsum only carry the shape (meta tensors) and the block names no partial buffers."""
    # ENTRY:115-122
    _req(mid_o.is_contiguous(), "mid_o.is_contiguous()")
    _req(mid_o_logexpsum.is_contiguous(), "mid_o_logexpsum.is_contiguous()")
    _req(q.is_contiguous(), "q.is_contiguous()")
    _req(k.stride(2) == 1, "k.stride(2) == 1")
    _req(v.stride(2) == 1, "v.stride(2) == 1")
    _req(req_to_tokens.is_contiguous(), "req_to_tokens.is_contiguous()")
    _req(b_req_idx.is_contiguous(), "b_req_idx.is_contiguous()")
    _req(b_seqlen.is_contiguous(), "b_seqlen.is_contiguous()")
    # ENTRY:124-131
    for t, d, n in ((mid_o, 4, "mid_o"), (mid_o_logexpsum, 3, "mid_o_logexpsum"), (q, 3, "q"), (k, 3, "k"), (v, 3, "v"),
                    (req_to_tokens, 2, "req_to_tokens"), (b_req_idx, 1, "b_req_idx"), (b_seqlen, 1, "b_seqlen")):
        on_gpu = t.is_cuda or (partials_in_library and t.is_meta)
        if t.dim() != d or not on_gpu:  # (the message is only built on failure: this runs once per decode step)
            _req(t.dim() == d, "%s.dim() == %d" % (n, d))
            _req(on_gpu, "%s on the GPU" % n)
    # ENTRY:133-140 (bfloat16 accepted in addition to half)
    _req(mid_o.dtype == torch.float32, "mid_o float32")
    _req(mid_o_logexpsum.dtype == torch.float32, "mid_o_logexpsum float32")
    _req(q.dtype in (torch.float16, torch.bfloat16), "q half or bfloat16")
    _req(k.dtype == q.dtype and v.dtype == q.dtype, "k, v dtype == q dtype")
    _req(req_to_tokens.dtype == torch.int32, "req_to_tokens int32")
    _req(b_req_idx.dtype == torch.int32, "b_req_idx int32")
    _req(b_seqlen.dtype == torch.int32, "b_seqlen int32")
    # shapes are inferred from mid_o as in ENTRY:155-160; make the implied relations explicit
    B, Hq, D = mid_o.size(1), mid_o.size(2), mid_o.size(3)
    _req(tuple(q.shape) == (B, Hq, D), "q.shape == mid_o.shape[1:]")
    _req(tuple(mid_o_logexpsum.shape) == tuple(mid_o.shape[:3]), "mid_o_logexpsum.shape == mid_o.shape[:3]")
    _req(k.size(1) == v.size(1) and k.size(2) == D and v.size(2) == D, "k/v head shapes")
    _req(b_req_idx.size(0) == B and b_seqlen.size(0) == B, "b_req_idx/b_seqlen length == batch")
    _req(seq_block_size >= 1, "seq_block_size >= 1")
    a = _lib.DecodeStage1Args()
    if not partials_in_library:
        a.mid_o, a.mid_o_logexpsum = mid_o.data_ptr(), mid_o_logexpsum.data_ptr()
    a.q, a.k, a.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    a.k_stride_0, a.k_stride_1 = k.stride(0), k.stride(1)
    a.v_stride_0, a.v_stride_1 = v.stride(0), v.stride(1)
    a.sm_scale = 1.0 / math.sqrt(q.size(2))  # ENTRY:142
    a.dtype = _DT[q.dtype]
    a.req_to_tokens, a.b_req_idx, a.b_seqlen = req_to_tokens.data_ptr(), b_req_idx.data_ptr(), b_seqlen.data_ptr()
    a.batch, a.num_q_heads, a.num_kv_heads = B, Hq, k.size(1)
    a.num_blocks, a.head_dim, a.max_seq_len = mid_o.size(0), D, req_to_tokens.size(1)
    a.seq_block_size, a.max_len_in_batch = int(seq_block_size), int(max_len_in_batch)
    _req(1 <= int(merge_blocks) <= 16, "1 <= merge_blocks <= 16")
    a.merge_blocks = int(merge_blocks)
    return a


@torch.inference_mode()
def flash_decoding_stage1(mid_o, mid_o_logexpsum, q, k, v, req_to_tokens, b_req_idx, b_seqlen,
                          max_len_in_batch: int, seq_block_size: int, merge_blocks: int = 1) -> None:
    """ENTRY:103-164, same argument order.  merge_blocks > 1 (not in the reference): one partial per that many consecutive
    blocks, in the row of the first; the rows of the others are marked empty (LSE = -inf)."""
    a = _stage1_args(mid_o, mid_o_logexpsum, q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch, seq_block_size,
                     merge_blocks)
    _lib.check(_lib.load().lsattn_decode_stage1(C.byref(a), _stream()), "lsattn_decode_stage1")


def _stage2_args(o, out_logexpsum, b_seqlen, mid_o, mid_o_logexpsum, block_seq: int,
                 partials_in_library: bool = False) -> _lib.DecodeStage2Args:
    """The checks of ENTRY:174-190 and the argument block of lsattn_decode_stage2."""
    # ENTRY:174-190
    for t, d, n in ((o, 3, "o"), (out_logexpsum, 2, "out_logexpsum"), (b_seqlen, 1, "b_seqlen"), (mid_o, 4, "mid_o"),
                    (mid_o_logexpsum, 3, "mid_o_logexpsum")):
        on_gpu = t.is_cuda or (partials_in_library and t.is_meta)
        if not t.is_contiguous() or t.dim() != d or not on_gpu:
            _req(t.is_contiguous(), "%s.is_contiguous()" % n)
            _req(t.dim() == d, "%s.dim() == %d" % (n, d))
            _req(on_gpu, "%s on the GPU" % n)
    _req(o.dtype in (torch.float16, torch.float32, torch.bfloat16), "o half, bfloat16 or float")
    _req(out_logexpsum.dtype == torch.float32, "out_logexpsum float32")
    _req(b_seqlen.dtype == torch.int32, "b_seqlen int32")
    _req(mid_o.dtype == torch.float32, "mid_o float32")
    _req(mid_o_logexpsum.dtype == torch.float32, "mid_o_logexpsum float32")
    B, H, D = mid_o.size(1), mid_o.size(2), mid_o.size(3)
    _req(tuple(o.shape) == (B, H, D), "o.shape == mid_o.shape[1:]")
    _req(tuple(out_logexpsum.shape) == (B, H), "out_logexpsum.shape == [batch, heads]")
    _req(tuple(mid_o_logexpsum.shape) == tuple(mid_o.shape[:3]), "mid_o_logexpsum.shape == mid_o.shape[:3]")
    _req(b_seqlen.size(0) == B, "b_seqlen length == batch")
    _req(block_seq >= 1, "block_seq >= 1")
    a = _lib.DecodeStage2Args()
    a.o, a.o_dtype, a.out_logexpsum, a.b_seqlen = o.data_ptr(), _DT[o.dtype], out_logexpsum.data_ptr(), b_seqlen.data_ptr()
    if not partials_in_library:
        a.mid_o, a.mid_o_logexpsum = mid_o.data_ptr(), mid_o_logexpsum.data_ptr()
    a.batch, a.num_heads, a.num_seq_blocks, a.head_dim, a.block_seq = B, H, mid_o.size(0), D, int(block_seq)
    return a


@torch.inference_mode()
def flash_decoding_stage2(o, out_logexpsum, b_seqlen, mid_o, mid_o_logexpsum, block_seq: int) -> None:
    """ENTRY:166-221, same argument order."""
    a = _stage2_args(o, out_logexpsum, b_seqlen, mid_o, mid_o_logexpsum, block_seq)
    _lib.check(_lib.load().lsattn_decode_stage2(C.byref(a), _stream()), "lsattn_decode_stage2")


# Argument blocks of the fused call, by the full metadata of its tensors.  A decode step of a serving loop calls with the
# same buffers every time (the request table, the length vector and the KV pool are updated in place), and the checks and
# the filling of the two blocks then cost more host time than a small batch's kernels run: a call whose tensors all have
# the address, shape, strides and dtype of an earlier, validated call reuses that call's blocks.
_FUSED_CACHE: dict = {}
_FUSED_CACHE_MAX = 64


def _meta(t):
    return (t.data_ptr(), t.shape, t.stride(), t.dtype, t.device.index)


# The fused call keeps the partials of a request side by side in mid_o ([batch, blocks, heads, head_dim] in the same
# memory) instead of a block of all requests after the other: mid_o is scratch there (FDPY:12-27 hands neither buffer
# out), and in a batch the reference's layout puts every partial of a request on a page of its own.
FUSED_PARTIALS_BY_REQUEST = True


def flash_decoding(mid_o, mid_o_logexpsum, q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch: int,
                   o, out_logexpsum, block_seq: int) -> None:
    """Stage 1 and stage 2 with the same block size from one library call (what FDPY:12-27 does with two): the checks of
    both, one argument pass, the two launches back to back."""
    key = (_meta(mid_o), _meta(mid_o_logexpsum), _meta(q), _meta(k), _meta(v), _meta(req_to_tokens), _meta(b_req_idx),
           _meta(b_seqlen), _meta(o), _meta(out_logexpsum), max_len_in_batch, block_seq, FUSED_PARTIALS_BY_REQUEST)
    blocks = _FUSED_CACHE.get(key)
    if blocks is None:
        a1 = _stage1_args(mid_o, mid_o_logexpsum, q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch, block_seq)
        a2 = _stage2_args(o, out_logexpsum, b_seqlen, mid_o, mid_o_logexpsum, block_seq)
        a1.partials_by_request = a2.partials_by_request = 1 if FUSED_PARTIALS_BY_REQUEST else 0
        if len(_FUSED_CACHE) >= _FUSED_CACHE_MAX:
            del _FUSED_CACHE[next(iter(_FUSED_CACHE))]  # the oldest entry (a caller that allocates new outputs every call never hits)
        blocks = _FUSED_CACHE[key] = (a1, a2, C.byref(a1), C.byref(a2), _lib.load().lsattn_decode_attention)
    rc = blocks[4](blocks[2], blocks[3], _stream())
    if rc:
        _lib.check(rc, "lsattn_decode_attention")


@torch.inference_mode()
def flash_decoding_static(q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch: int, o, out_logexpsum,
                          block_seq: int) -> None:
    """flash_decoding without mid_o / mid_o_logexpsum: the partials live in the library's per-GPU static array
    (lsattn_decode_attention_static), so the call needs no scratch tensors.  Raises if
    ceil(max_len_in_batch / block_seq) * batch * heads * (head_dim + 1) * 4 bytes exceed
    _lib.LSATTN_STATIC_SCRATCH_BYTES.  Calls that overlap on one GPU share the array and race."""
    _req(q.dim() == 3 and q.is_contiguous() and q.is_cuda, "q contiguous [batch, heads, head_dim] on the GPU")
    B, Hq, D = q.shape
    rows = max((int(max_len_in_batch) + int(block_seq) - 1) // int(block_seq), 1)
    # the argument blocks are checked as usual against tensors of the partials' shape that own no memory
    mid_o = torch.empty((rows, B, Hq, D), dtype=torch.float32, device="meta")
    mid_lse = torch.empty((rows, B, Hq), dtype=torch.float32, device="meta")
    a1 = _stage1_args(mid_o, mid_lse, q, k, v, req_to_tokens, b_req_idx, b_seqlen, max_len_in_batch, block_seq,
                      partials_in_library=True)
    a2 = _stage2_args(o, out_logexpsum, b_seqlen, mid_o, mid_lse, block_seq, partials_in_library=True)
    _lib.check(_lib.load().lsattn_decode_attention_static(C.byref(a1), C.byref(a2), _stream()),
               "lsattn_decode_attention_static")


def _half2d(t: torch.Tensor, name: str, dim: int) -> None:
    if not (t.is_cuda and t.dim() == dim and t.dtype == torch.float16 and t.is_contiguous()):
        raise ValueError("%s must be a contiguous %d-d float16 CUDA tensor" % (name, dim))


@torch.inference_mode()
def rms_norm(input: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Argument order, checks and result of ENTRY:15-39 (a new [num_tokens, hidden] fp16 tensor)."""
    _half2d(input, "input", 2); _half2d(weight, "weight", 1)
    if input.size(1) != weight.size(0):
        raise ValueError("input.size(1) must equal weight.size(0)")
    out = torch.empty_like(input)
    _lib.check(_lib.load().lsattn_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(), input.size(0), input.size(1),
                                           float(eps), _stream()), "lsattn_rms_norm")
    return out


@torch.inference_mode()
def silu_and_mul_inplace(io: torch.Tensor) -> None:
    """ENTRY:41-52: io is [num_tokens, 2 * inter]; the first half of every row becomes silu(gate) * up."""
    _half2d(io, "io", 2)
    if io.size(1) % 2:
        raise ValueError("io.size(1) must be even")
    _lib.check(_lib.load().lsattn_silu_and_mul_inplace(io.data_ptr(), io.size(0), io.size(1) // 2, _stream()),
               "lsattn_silu_and_mul_inplace")


def _rotary_single(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    if not (x.is_cuda and x.dim() == 3 and x.dtype == torch.float16 and x.stride(2) == 1):
        raise ValueError("x must be a 3-d float16 CUDA tensor with a contiguous last dimension")
    T, H, D = x.shape
    _half2d(cos, "cos", 2); _half2d(sin, "sin", 2)
    if cos.shape != sin.shape or cos.size(0) != T or cos.size(1) != D // 2:
        raise ValueError("cos and sin must be [num_tokens, head_dim/2]")
    _lib.check(_lib.load().lsattn_rotary_emb(x.data_ptr(), cos.data_ptr(), sin.data_ptr(), x.stride(0), x.stride(1), T, H, D,
                                             _stream()), "lsattn_rotary_emb")


@torch.inference_mode()
def rotary_emb(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> None:
    """ENTRY:54-89: in-place rotary embedding of q and of k (strided views are fine)."""
    _rotary_single(q, cos, sin)
    _rotary_single(k, cos, sin)


@torch.inference_mode()
def ffn_block(input_embds: torch.Tensor, norm_weight: torch.Tensor, norm_eps: float, gate_up_proj: torch.Tensor,
              down_proj: torch.Tensor) -> torch.Tensor:
    """ENTRY:91-101: rms_norm -> mm -> silu_and_mul_inplace -> mm into the normed buffer, which is returned.
    The two matrix products are plain library GEMMs (torch.mm), as in the reference."""
    normed = rms_norm(input_embds, norm_weight, norm_eps)
    up_gate = torch.mm(normed, gate_up_proj)
    silu_and_mul_inplace(up_gate)
    torch.mm(up_gate[:, :up_gate.size(-1) // 2], down_proj, out=normed)
    return normed


def hello_world() -> None:
    """Load check, as ENTRY:231-232."""
    print("Hello world from loongserve_amd.longserve_cuda_kernels (liblsattn v%d)!" % _lib.load().lsattn_version())

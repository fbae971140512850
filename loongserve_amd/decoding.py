"""Python wrappers the llama layer calls for decode; names and argument order of
loongserve/models/llama/triton_kernel/longserve_flash_decoding_stage1.py:78,
longserve_flash_decoding_stage2.py:53 and longserve_flash_decoding.py:3."""
from __future__ import annotations

import functools

import torch

from . import longserve_cuda_kernels


# The stage functions called on their own (the master path, longserve_transformer_layer_infer.py:272-281 then :360-367)
# leave the reference's buffers: one partial per block of block_seq tokens, row i of mid_out = block i.
# Opt-in (STAGE1_MERGES_BLOCKS = True; not the reference's layout): stage 1 computes one partial per group of consecutive
# blocks (the same rule as the fused call below, at most 16 blocks), writes it to the row of the group's first block and
# marks the rows of the others empty (LSE = -inf, mid_out row left as it was).  Any LSE merge over ceil(len / block_seq)
# rows per request that skips empty rows (this package's stage 2 does) gives the same result, with a quarter of the
# partial bytes at BLOCK_SEQ 256; a consumer that multiplies an empty row's mid_out by a zero weight instead must not use
# it (the stale row may hold anything).
STAGE1_MERGES_BLOCKS = False


def longserve_flash_decode_stage1(q, k, v, Req_to_tokens, B_req_idx, B_Seqlen, max_len_in_batch, mid_out,
                                  mid_out_logsumexp, block_seq):
    merge = 1
    if STAGE1_MERGES_BLOCKS:
        merge = min(16, _fused_block_seq(block_seq, q.shape[0], max_len_in_batch, k.shape[1]) // int(block_seq))
    longserve_cuda_kernels.flash_decoding_stage1(mid_out, mid_out_logsumexp, q, k, v, Req_to_tokens, B_req_idx,
                                                 B_Seqlen, max_len_in_batch, block_seq, merge)
    return


def longserve_flash_decode_stage2(mid_out, mid_out_logexpsum, B_Seqlen, O, out_logexpsum, block_seq):
    longserve_cuda_kernels.flash_decoding_stage2(O, out_logexpsum, B_Seqlen, mid_out, mid_out_logexpsum, block_seq)
    return


# Split size between the two stages of the fused call.  There mid_o / mid_o_logexpsum are scratch (FDPY:12-27 never hands
# them out, the callers at longserve_transformer_layer_infer.py:293-308 only use the returned pair), so the context may be
# cut more coarsely than BLOCK_SEQ: fewer fp32 block partials are written while the gather saturates the memory system
# (every MB of them costs about as much as 8 MB of reads).  The result is the same softmax, merged from fewer pieces.
# longserve_flash_decode_stage1 / _stage2 called on their own always split at the block_seq they are given.
# (Launches of eight and more requests with enough tokens do not use the split at all: lsattn_decode_attention deals their
# blocks in equal shares to the waves, one partial per share and request.  The split below is what smaller launches get.)
FUSED_SPLIT_TOKENS = 1024
# Do not coarsen below this many (upper-bound estimate of) stage-1 workgroups: one per CU.  Measured on 131072 tokens in
# all (1 x 131072 ... 16 x 8192, 8 KV heads): 92-95 us at 256 workgroups of 1024 tokens against 100-104 us at 1024 of 256.
FUSED_MIN_WORKGROUPS = 256


# Very long contexts go further, up to 4096 tokens, while the longest request still has this many blocks: there the last,
# partly filled block of a request and the spread of lengths in the batch (which the host does not see) weigh little, and
# the partials and their merge are what is left to save (one request of 1048576 tokens: 721 -> 675 us; four of 131072
# with 32 KV heads: 1336 -> 1313 us).  With fewer blocks per request the coarser split loses to the ragged tail
# (config 3, lengths 4096..32768: 903 us at 1024, 947 at 2048).
FUSED_LONG_SPLIT_TOKENS = 4096
FUSED_LONG_MIN_BLOCKS = 64
# ... and only in batches of at most this many requests.  What the coarser split wins is a few percent and only if the
# requests are about as long as each other (64 x 65536 tokens 2.78 ms at 1024, 2.58 at 4096; 32 x 131072 2.65 at 2048,
# 2.58 at 4096); what it loses when one long request stands among many short ones is more (131072 + 255 x 512 tokens:
# 0.181 ms at 1024, 0.198 at 2048, 0.238 at 4096; 131072 + 63 x 2048: 0.207 / 0.217 / 0.275; but 524288 + 63 x 2048, where the
# long request is four fifths of all tokens: 0.447 / 0.429 / 0.416), and the larger the batch the likelier the latter.
FUSED_LONG_MAX_BATCH = 64


@functools.lru_cache(maxsize=4096)
def _fused_block_seq(block_seq: int, batch_size: int, max_len_in_batch: int, num_kv_heads: int) -> int:
    bs = int(block_seq)
    task_groups = (int(num_kv_heads) + 3) // 4
    while bs * 2 <= FUSED_LONG_SPLIT_TOKENS and bs < int(max_len_in_batch):
        blocks = (int(max_len_in_batch) + 2 * bs - 1) // (2 * bs)
        if int(batch_size) * blocks * task_groups < FUSED_MIN_WORKGROUPS:
            break
        if bs * 2 > FUSED_SPLIT_TOKENS and (blocks < FUSED_LONG_MIN_BLOCKS or int(batch_size) > FUSED_LONG_MAX_BATCH):
            break
        bs *= 2
    return bs


def longserve_token_decode_attention_flash_decoding(q, req_to_token_indexs, b_req_idx, b_seq_len, mid_o,
                                                    mid_o_logexpsum, batch_size, max_len_in_batch, q_head_num,
                                                    head_dim, cache_k, cache_v, BLOCK_SEQ, out=None,
                                                    o_logexpsum=None):
    calcu_shape1 = (-1, q_head_num, head_dim)
    # outputs are float32 whatever q is, so that they can be merged again (FDPY:9-10)
    o_tensor = torch.empty_like(q, dtype=torch.float32) if out is None else out
    out_logexpsum = (torch.empty([batch_size, q_head_num], dtype=torch.float32, device=q.device)
                     if o_logexpsum is None else o_logexpsum)
    split = _fused_block_seq(BLOCK_SEQ, batch_size, max_len_in_batch, cache_k.shape[1])
    longserve_cuda_kernels.flash_decoding(mid_o, mid_o_logexpsum, q.view(calcu_shape1), cache_k, cache_v, req_to_token_indexs,
                                          b_req_idx, b_seq_len, max_len_in_batch, o_tensor.view(calcu_shape1), out_logexpsum,
                                          split)
    return o_tensor, out_logexpsum

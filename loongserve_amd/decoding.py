"""Python wrappers the llama layer calls for decode; names and argument order of
loongserve/models/llama/triton_kernel/longserve_flash_decoding_stage1.py:78,
longserve_flash_decoding_stage2.py:53 and longserve_flash_decoding.py:3."""
from __future__ import annotations

import torch

from . import longserve_cuda_kernels


def longserve_flash_decode_stage1(q, k, v, Req_to_tokens, B_req_idx, B_Seqlen, max_len_in_batch, mid_out,
                                  mid_out_logsumexp, block_seq):
    longserve_cuda_kernels.flash_decoding_stage1(mid_out, mid_out_logsumexp, q, k, v, Req_to_tokens, B_req_idx,
                                                 B_Seqlen, max_len_in_batch, block_seq)
    return


def longserve_flash_decode_stage2(mid_out, mid_out_logexpsum, B_Seqlen, O, out_logexpsum, block_seq):
    longserve_cuda_kernels.flash_decoding_stage2(O, out_logexpsum, B_Seqlen, mid_out, mid_out_logexpsum, block_seq)
    return


def longserve_token_decode_attention_flash_decoding(q, req_to_token_indexs, b_req_idx, b_seq_len, mid_o,
                                                    mid_o_logexpsum, batch_size, max_len_in_batch, q_head_num,
                                                    head_dim, cache_k, cache_v, BLOCK_SEQ, out=None,
                                                    o_logexpsum=None):
    calcu_shape1 = (-1, q_head_num, head_dim)
    # outputs are float32 whatever q is, so that they can be merged again (FDPY:9-10)
    o_tensor = torch.empty_like(q, dtype=torch.float32) if out is None else out
    out_logexpsum = (torch.empty([batch_size, q_head_num], dtype=torch.float32, device=q.device)
                     if o_logexpsum is None else o_logexpsum)
    longserve_flash_decode_stage1(q.view(calcu_shape1), cache_k, cache_v, req_to_token_indexs, b_req_idx, b_seq_len,
                                  max_len_in_batch, mid_o, mid_o_logexpsum, BLOCK_SEQ)
    longserve_flash_decode_stage2(mid_o, mid_o_logexpsum, b_seq_len, o_tensor.view(calcu_shape1), out_logexpsum,
                                  BLOCK_SEQ)
    return o_tensor, out_logexpsum

"""MI355X-native attention hot path with LoongServe's operator interface.

Prefill: context_attention_fwd (ring / context-parallel step, in-place (o, m, l) state),
prefill_attention_step (+ lse_merge) for mergeable fp32 partials.
Decode: longserve_flash_decode_stage1 / stage2,
longserve_token_decode_attention_flash_decoding, and the extension-module stand-in
`longserve_cuda_kernels`.  All of them run hand-written gfx950 HIP kernels from
liblsattn.so; importing this package fails if that library has not been built.
"""
import sys as _sys

from . import _lib

# `python -m loongserve_amd.build` imports this package on its way to the build recipe: the library it is
# about to (re)build may be missing or lack a new entry point, so that one invocation skips the load.
_building = len(getattr(_sys, "orig_argv", [])) >= 3 and _sys.orig_argv[1:3] == ["-m", "loongserve_amd.build"]
if not _building:
    _lib.load()  # fail loudly at import time if the HIP library is missing or stale

from ._lib import set_tuning  # noqa: E402
from . import longserve_cuda_kernels  # noqa: E402
from .kv_pool import LongServeMemoryManager, LongServeReqManager  # noqa: E402
from .decoding import (longserve_flash_decode_stage1, longserve_flash_decode_stage2,  # noqa: E402
                       longserve_token_decode_attention_flash_decoding)
from .ops import (context_attention_fwd, copy_kv_index_to_req, decoding_stage_migration_receiver_kernel,  # noqa: E402
                  decoding_stage_migration_sender_kernel, destindex_copy_and_register_kv, destindex_copy_kv,
                  init_req_to_token_indexes, kv_scatter, lse_merge, pre_copy_and_register_kv, prefill_attention_step,
                  rmsnorm_forward, rotary_emb_fwd, rotary_emb_write_kv, silu_and_mul_fwd)

__all__ = [
    "context_attention_fwd", "prefill_attention_step", "lse_merge", "kv_scatter", "init_req_to_token_indexes",
    "pre_copy_and_register_kv", "destindex_copy_and_register_kv", "destindex_copy_kv", "copy_kv_index_to_req",
    "rmsnorm_forward", "rotary_emb_fwd", "rotary_emb_write_kv", "silu_and_mul_fwd",
    "decoding_stage_migration_sender_kernel", "decoding_stage_migration_receiver_kernel",
    "longserve_flash_decode_stage1", "longserve_flash_decode_stage2",
    "longserve_token_decode_attention_flash_decoding", "longserve_cuda_kernels",
    "LongServeMemoryManager", "LongServeReqManager", "set_tuning",
]

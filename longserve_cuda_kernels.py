"""The reference's Python layer imports its extension module by this top-level name (`import longserve_cuda_kernels`,
loongserve/models/llama/triton_kernel/longserve_flash_decoding_stage1.py:4, longserve_cuda_kernels/README.md:41).
This module re-exports the stand-in of this build, loongserve_amd.longserve_cuda_kernels, under that name, so those files
resolve unedited when the repository root (or an installed copy of it) is on sys.path."""
from loongserve_amd.longserve_cuda_kernels import *  # noqa: F401,F403
from loongserve_amd.longserve_cuda_kernels import (ffn_block, flash_decoding, flash_decoding_stage1,  # noqa: F401
                                                   flash_decoding_stage2, flash_decoding_static, hello_world, rms_norm,
                                                   rotary_emb, silu_and_mul_inplace)

"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports every
symbol include/lsattn.h declares, and argument validation rejects bad input without
touching a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "lsattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lsattn_[a-z0-9_]+)\s*\(", text)))


def test_importing_the_package_first_leaves_one_hip_runtime_in_the_process():
    """PyTorch-ROCm ships its own libamdhip64; the library links the system's.  Whatever the program imports first, the
    process must end up with one runtime (two: the library's launches find no device in theirs)."""
    import subprocess
    import sys
    code = ("import loongserve_amd, torch\n"
            "print(sorted({l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l}))")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    paths = eval(out.stdout.strip().splitlines()[-1])
    assert len(paths) == 1, paths


def test_ceiling_library_exports_every_declared_symbol():
    """libls_ceiling.so (bench.py's measurement aids) exports what include/ls_ceiling.h declares."""
    import ctypes
    import torch  # noqa: F401  (first, so that this process keeps to one HIP runtime: see the test above)
    text = open(os.path.join(ROOT, "include", "ls_ceiling.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(ls_ceiling_[a-z0-9_]+)\s*\(", text)))
    assert len(names) == 5, names
    lib = ctypes.CDLL(os.path.join(ROOT, "loongserve_amd", "libls_ceiling.so"))
    for n in names:
        assert getattr(lib, n) is not None


def test_library_exports_every_declared_symbol():
    from loongserve_amd import _lib
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 9
    assert set(names) == set(_lib.EXPORTS), (names, sorted(_lib.EXPORTS))
    for n in names:
        assert getattr(lib, n) is not None
    # LSATTN_VERSION of include/lsattn.h: the argument blocks as _lib.py declares them
    header = open(os.path.join(ROOT, "include", "lsattn.h")).read()
    assert lib.lsattn_version() == _lib.LSATTN_VERSION == int(re.search(r"#define LSATTN_VERSION (\d+)", header).group(1))
    assert lib.lsattn_strerror(0) == b"ok"
    assert b"invalid" in lib.lsattn_strerror(-1)


def test_struct_layout_matches_header():
    # compile a tiny C program against the header and compare sizeof / offsetof with ctypes
    import subprocess
    import tempfile
    from loongserve_amd import _lib
    src = r'''
#include <stdio.h>
#include <stddef.h>
#include "lsattn.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu\n", sizeof(lsattn_prefill_args), sizeof(lsattn_merge_args),
         sizeof(lsattn_decode_stage1_args), sizeof(lsattn_decode_stage2_args), sizeof(lsattn_kv_copy_register_args));
  printf("%zu %zu\n", sizeof(lsattn_decode_migration_args), offsetof(lsattn_decode_migration_args, b_seq_len));
  printf("%zu %zu\n", sizeof(lsattn_rotary_kv_write_args), offsetof(lsattn_rotary_kv_write_args, register_mode));
  printf("%zu %zu\n", sizeof(lsattn_tuning), offsetof(lsattn_tuning, decode_listed));
  printf("%zu %zu %zu %zu\n", sizeof(lsattn_merge_cuts_args), offsetof(lsattn_merge_cuts_args, ml_stride_h), offsetof(lsattn_prefill_args, o_cut_rows),
         offsetof(lsattn_prefill_args, total_q_rows));
  printf("%zu %zu %zu %zu %zu %zu\n", offsetof(lsattn_prefill_args, sm_scale), offsetof(lsattn_prefill_args, ml_stride_h),
         offsetof(lsattn_decode_stage1_args, req_to_tokens), offsetof(lsattn_decode_stage2_args, block_seq),
         offsetof(lsattn_kv_copy_register_args, req_to_tokens), offsetof(lsattn_kv_copy_register_args, should_register));
  return 0;
}'''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
        out = subprocess.check_output([exe]).decode().split()
    sizes = [int(x) for x in out[:5]]
    mig = [int(x) for x in out[5:7]]
    rot = [int(x) for x in out[7:9]]
    tun = [int(x) for x in out[9:11]]
    cuts = [int(x) for x in out[11:15]]
    offs = [int(x) for x in out[15:]]
    assert cuts == [C.sizeof(_lib.MergeCutsArgs), _lib.MergeCutsArgs.ml_stride_h.offset, _lib.PrefillArgs.o_cut_rows.offset,
                    _lib.PrefillArgs.total_q_rows.offset]
    assert tun == [C.sizeof(_lib.Tuning), _lib.Tuning.decode_listed.offset]
    assert rot == [C.sizeof(_lib.RotaryKvWriteArgs), _lib.RotaryKvWriteArgs.register_mode.offset]
    assert mig == [C.sizeof(_lib.DecodeMigrationArgs), _lib.DecodeMigrationArgs.b_seq_len.offset]
    assert sizes == [C.sizeof(_lib.PrefillArgs), C.sizeof(_lib.MergeArgs), C.sizeof(_lib.DecodeStage1Args),
                     C.sizeof(_lib.DecodeStage2Args), C.sizeof(_lib.KvCopyRegisterArgs)]
    assert offs == [_lib.PrefillArgs.sm_scale.offset, _lib.PrefillArgs.ml_stride_h.offset,
                    _lib.DecodeStage1Args.req_to_tokens.offset, _lib.DecodeStage2Args.block_seq.offset,
                    _lib.KvCopyRegisterArgs.req_to_tokens.offset, _lib.KvCopyRegisterArgs.should_register.offset]


def test_validation_rejects_bad_arguments_without_gpu():
    from loongserve_amd import _lib
    lib = _lib.load()
    a = _lib.PrefillArgs()  # all null
    assert lib.lsattn_prefill_step(C.byref(a), None) == -1
    assert lib.lsattn_prefill_step(None, None) == -1
    d1 = _lib.DecodeStage1Args()
    assert lib.lsattn_decode_stage1(C.byref(d1), None) == -1
    mg = _lib.DecodeMigrationArgs()
    assert lib.lsattn_decode_migration_send(C.byref(mg), None) == -1
    assert lib.lsattn_decode_migration_recv(None, None) == -1
    rw = _lib.RotaryKvWriteArgs()
    assert lib.lsattn_rotary_kv_write(C.byref(rw), None) == -1
    assert lib.lsattn_rotary_kv_write(None, None) == -1
    cr = _lib.KvCopyRegisterArgs()
    assert lib.lsattn_kv_copy_register(C.byref(cr), None) == -1
    assert lib.lsattn_kv_ranges(None, None, None, 1, 0, None, None, None, None) == -1
    d2 = _lib.DecodeStage2Args()
    assert lib.lsattn_decode_stage2(C.byref(d2), None) == -1
    m = _lib.MergeArgs()
    assert lib.lsattn_lse_merge(C.byref(m), None) == -1
    assert lib.lsattn_kv_scatter(None, 0, None, 0, None, 0, 0, None) == -1
    assert lib.lsattn_bf16_to_f16_rows(None, 8, None, 8, 1, 8, None) == -1
    assert lib.lsattn_bf16_to_f16_rows(0x1000, 8, 0x2000, 8, 1, 16, None) == -1   # stride shorter than the row
    # slot allocator: sizes of the workspaces are host arithmetic, argument checks come before any launch
    assert lib.lsattn_pool_search_workspace_bytes(0) == 0
    assert lib.lsattn_pool_search_workspace_bytes(4096) == 16 + 28 + 4          # one workgroup of slots, padded to 16
    assert lib.lsattn_pool_search_workspace_bytes(2_500_000) >= 16 + 611 * 28
    assert lib.lsattn_pool_refs_workspace_bytes(0) == 0
    assert lib.lsattn_pool_refs_workspace_bytes(257) == 2 * 16 + 1040
    assert lib.lsattn_pool_alloc(None, 8, 1, None, None, 0, None) == -1
    assert lib.lsattn_pool_alloc(0x1000, 8192, 1, 0x2000, 0x3000, 16, None) == -4  # workspace too small
    assert lib.lsattn_pool_find_contiguous(0x1000, 8192, 0, 0x2000, 0x3000, 1 << 20, None) == -1  # need >= 1
    assert lib.lsattn_pool_find_contiguous(0x1004, 8192, 1, 0x2000, 0x3000, 1 << 20, None) == -1  # misaligned state
    assert lib.lsattn_pool_update_refs(0x1000, 8, 0x2000, 4, 2, 0x3000, 0x4000, 1 << 20, None) == -1  # delta must be +-1
    assert lib.lsattn_pool_update_refs(0x1000, 8, 0x2000, 4, 1, 0x3000, 0x4000, 8, None) == -4
    assert b"workspace" in lib.lsattn_strerror(-4)
    # unsupported head_dim is reported as such (pointers are fake but never dereferenced)
    fake = 0x1000
    for f in ("q", "k", "v", "o", "lse", "q_b_start_loc", "q_b_seq_len", "q_first_token_global_idx", "kv_b_start_loc",
              "kv_b_seq_len", "kv_first_token_global_idx"):
        setattr(a, f, fake)
    a.batch, a.num_q_heads, a.num_kv_heads, a.head_dim, a.sp_peers, a.max_q_len = 1, 4, 2, 48, 1, 8
    a.o_dtype = _lib.LSATTN_F32
    assert lib.lsattn_prefill_step(C.byref(a), None) == -2
    # head sizes 16, 32 and 64 have a kernel of their own, which does not cut the KV chunk
    a.head_dim, a.kv_cuts, a.kv_cut_len, a.o_cut_rows = 64, 2, 64, 8
    assert lib.lsattn_prefill_step(C.byref(a), None) == -2
    a.kv_cuts = a.kv_cut_len = a.o_cut_rows = 0
    a.head_dim, a.num_kv_heads = 128, 3
    assert lib.lsattn_prefill_step(C.byref(a), None) == -1
    # K/V token strides must be positive and keep a 64-row tile within a 32-bit byte offset
    a.num_kv_heads = 2
    for f in ("q_stride_t", "q_stride_h", "k_stride_h", "v_stride_h", "o_stride_t", "o_stride_h"):
        setattr(a, f, 128)
    a.dtype = _lib.LSATTN_F16
    for ks, vs in ((0, 256), (256, -256), ((1 << 24) + 8, 256), (256, 1 << 25)):
        a.k_stride_t, a.v_stride_t = ks, vs
        assert lib.lsattn_prefill_step(C.byref(a), None) == -1, (ks, vs)
    # the chunk cut along the keys: fp32 partials only, whole 64-key tiles per cut, the cuts' rows apart
    a.k_stride_t = a.v_stride_t = 256
    a.kv_cuts, a.kv_cut_len, a.o_cut_rows = 4, 100, 8
    assert lib.lsattn_prefill_step(C.byref(a), None) == -1          # not a multiple of 64 keys
    a.kv_cut_len, a.o_cut_rows = 128, 0
    assert lib.lsattn_prefill_step(C.byref(a), None) == -1          # no room between the cuts' outputs
    a.o_cut_rows, a.kv_cuts = 8, 65
    assert lib.lsattn_prefill_step(C.byref(a), None) == -1          # more cuts than LSATTN_MAX_KV_CUTS
    a.kv_cuts = 4
    assert lib.lsattn_prefill_step_accumulate(C.byref(a), None) == -1  # the folding steps take no cuts
    mc = _lib.MergeCutsArgs()
    assert lib.lsattn_prefill_merge_cuts(C.byref(mc), None) == -1
    assert lib.lsattn_prefill_merge_cuts(None, None) == -1
    for f in ("o_parts", "lse_parts", "q_b_start_loc", "q_b_seq_len", "o", "lse"):
        setattr(mc, f, fake)
    mc.n_parts, mc.batch, mc.num_q_heads, mc.head_dim, mc.max_q_len, mc.part_rows = 2, 1, 4, 64, 8, 8
    mc.o_stride_t, mc.o_stride_h, mc.o_dtype = 512, 128, _lib.LSATTN_F32
    assert lib.lsattn_prefill_merge_cuts(C.byref(mc), None) == -2   # head_dim
    mc.head_dim, mc.mode = 128, 1
    assert lib.lsattn_prefill_merge_cuts(C.byref(mc), None) == -1   # mode 1 needs m, l and a 16-bit o
    mc.mode, mc.n_parts = 0, 65
    assert lib.lsattn_prefill_merge_cuts(C.byref(mc), None) == -1
    # the fused decode call refuses argument blocks that do not describe the same partials
    s1, s2 = _lib.DecodeStage1Args(), _lib.DecodeStage2Args()
    assert lib.lsattn_decode_attention(None, C.byref(s2), None) == -1
    s1.mid_o, s2.mid_o = 0x1000, 0x2000
    assert lib.lsattn_decode_attention(C.byref(s1), C.byref(s2), None) == -1
    s2.mid_o = 0x1000
    s1.seq_block_size, s2.block_seq = 256, 128
    assert lib.lsattn_decode_attention(C.byref(s1), C.byref(s2), None) == -1
    # stage 1 merges at most 16 blocks into one partial
    s3 = _lib.DecodeStage1Args()
    for f in ("mid_o", "mid_o_logexpsum", "q", "k", "v", "req_to_tokens", "b_req_idx", "b_seqlen"):
        setattr(s3, f, 0x1000)
    s3.batch, s3.num_q_heads, s3.num_kv_heads, s3.num_blocks, s3.head_dim = 1, 4, 2, 4, 128
    s3.max_seq_len, s3.seq_block_size, s3.max_len_in_batch, s3.dtype = 1024, 256, 1024, _lib.LSATTN_F16
    s3.k_stride_0 = s3.v_stride_0 = 512
    s3.k_stride_1 = s3.v_stride_1 = 128
    for bad in (-1, 17):
        s3.merge_blocks = bad
        assert lib.lsattn_decode_stage1(C.byref(s3), None) == -1, bad


def test_tuning_block_is_validated_and_named_values_match_the_header():
    """lsattn_set_tuning takes the values include/lsattn.h names, refuses others, and NULL restores the library's choices;
    the names the Python side uses stand for the header's numbers."""
    from loongserve_amd import _lib
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "lsattn.h")).read()
    num = {k: int(v) for k, v in re.findall(r"#define (LSATTN_(?:PREFILL|DECODE)_[A-Z0-9_]+) (\d+)", header)}
    want = {("prefill_rows", "128"): "LSATTN_PREFILL_ROWS_128", ("prefill_rows", "256"): "LSATTN_PREFILL_ROWS_256",
            ("prefill_rows", "half"): "LSATTN_PREFILL_ROWS_HALF", ("prefill_order", "tile"): "LSATTN_PREFILL_ORDER_TILE",
            ("prefill_order", "head"): "LSATTN_PREFILL_ORDER_HEAD", ("prefill_pack", "off"): "LSATTN_PREFILL_PACK_OFF",
            ("decode_stage1", "lane"): "LSATTN_DECODE_STAGE1_LANE", ("decode_stage1", "mfma"): "LSATTN_DECODE_STAGE1_MFMA",
            ("decode_stage1", "split"): "LSATTN_DECODE_STAGE1_SPLIT", ("decode_listed", "off"): "LSATTN_DECODE_LISTED_OFF",
            ("decode_listed", "on"): "LSATTN_DECODE_LISTED_ON", ("decode_listed", "shares"): "LSATTN_DECODE_LISTED_SHARES"}
    assert len(num) == len(want)
    for (field, name), macro in want.items():
        assert _lib.TUNING_VALUES[field][name] == num[macro]
        assert _lib.TUNING_VALUES[field][None] == 0
    try:
        t = _lib.Tuning()
        for field, top in (("prefill_rows", 3), ("prefill_order", 2), ("prefill_pack", 1), ("decode_stage1", 3), ("decode_listed", 3)):
            for bad in (-1, top + 1):
                t = _lib.Tuning()
                setattr(t, field, bad)
                assert lib.lsattn_set_tuning(C.byref(t)) == -1, (field, bad)
            t = _lib.Tuning()
            setattr(t, field, top)
            assert lib.lsattn_set_tuning(C.byref(t)) == 0
        t = _lib.Tuning()
        t.reserved[1] = 1
        assert lib.lsattn_set_tuning(C.byref(t)) == -1
        with pytest.raises(ValueError):
            _lib.set_tuning(prefill_rows="512")
        with pytest.raises(ValueError):
            _lib.set_tuning(no_such_choice="x")
    finally:
        assert lib.lsattn_set_tuning(None) == 0


def test_library_reads_no_environment_variable():
    """The launch choices come from lsattn_set_tuning alone: no source of the library calls getenv."""
    csrc = os.path.join(ROOT, "loongserve_amd", "csrc")
    for name in os.listdir(csrc):
        if name.endswith((".hip", ".h")):
            assert "getenv" not in open(os.path.join(csrc, name)).read(), name


def test_python_wrappers_reject_cpu_tensors():
    import torch
    import loongserve_amd as lsa
    q = torch.zeros(4, 2, 128, dtype=torch.float16)
    i = torch.zeros(1, dtype=torch.int32)
    with pytest.raises(ValueError):
        lsa.prefill_attention_step(q, q, q, i, i, i, i, i, i, 1, 4, out=torch.zeros(4, 2, 128), lse=torch.zeros(4, 2))
    with pytest.raises(ValueError):
        lsa.longserve_cuda_kernels.flash_decoding_stage1(torch.zeros(1, 1, 2, 128), torch.zeros(1, 1, 2), q[:1], q, q,
                                                         torch.zeros(1, 4, dtype=torch.int32), i, i, 4, 4)


def test_fused_decode_split_rule():
    """The fused decode call may split the context more coarsely than BLOCK_SEQ, but only while the launch keeps enough
    workgroups; the stage functions called on their own never change the block size they are given."""
    from loongserve_amd.decoding import FUSED_LONG_SPLIT_TOKENS, _fused_block_seq
    assert _fused_block_seq(256, 64, 32768, 8) == 1024           # config 3: 64 x 32 blocks x 2 task groups
    assert _fused_block_seq(256, 1, 4096, 8) == 256              # a single short request: nothing to spare
    assert _fused_block_seq(256, 16, 8192, 8) == 1024            # 16 x 8 blocks x 2 task groups = one workgroup per CU
    assert _fused_block_seq(256, 1, 131072, 8) == 1024
    assert _fused_block_seq(256, 1, 32768, 8) == 256
    assert _fused_block_seq(256, 1, 1048576, 8) == 4096          # very long contexts: up to 4096 while >= 64 blocks remain
    assert _fused_block_seq(256, 4, 131072, 32) == 2048
    assert _fused_block_seq(256, 16, 32768, 8) == 1024
    assert _fused_block_seq(2048, 64, 32768, 8) == 2048          # never below what the caller asked for
    assert _fused_block_seq(256, 64, 524288, 8) == 4096          # up to 64 requests may go beyond 1024
    assert _fused_block_seq(256, 256, 131072, 8) == 1024         # larger batches stay there: the likelier to hold one long request among short ones
    assert _fused_block_seq(16, 4096, 16, 8) == 16
    for bs in (1, 16, 64, 256):
        got = _fused_block_seq(bs, 1 << 14, 1 << 20, 32)
        assert got % bs == 0 and got <= max(FUSED_LONG_SPLIT_TOKENS, bs)


def test_extension_module_resolves_by_its_reference_name():
    """`import longserve_cuda_kernels`, as loongserve/models/llama/triton_kernel/longserve_flash_decoding_stage1.py:4 does."""
    import importlib
    m = importlib.import_module("longserve_cuda_kernels")
    from loongserve_amd import longserve_cuda_kernels as real
    for name in ("flash_decoding_stage1", "flash_decoding_stage2", "rms_norm", "silu_and_mul_inplace", "rotary_emb", "ffn_block",
                 "hello_world"):
        assert getattr(m, name) is getattr(real, name)


def test_kv_split_count_from_shapes():
    """The split of a short-query step along the keys is chosen from shapes alone (no device read-back)."""
    from loongserve_amd.ops import kv_split_count
    assert kv_split_count(1, 32, 16384, 16384) == 1          # config 2: 4096 workgroups
    assert kv_split_count(1, 32, 2048, 2048) == 1            # config 1: enough workgroups, few keys
    assert kv_split_count(1, 32, 100, 131072) == 8           # one 100-row chunk against 131072 keys: 32 workgroups -> one round of 256
    assert kv_split_count(1, 32, 100, 131072, 8) == 8        # GQA 32/8: four heads side by side, 8 x 4 workgroups of 32 positions
    assert kv_split_count(1, 32, 16, 131072, 8) == 32        # 16 rows: 8 workgroups; cuts of at least 4096 keys
    assert kv_split_count(1, 32, 16, 20000, 8) == 4
    assert kv_split_count(1, 8, 100, 20000) == 4             # cuts of at least 4096 keys
    assert kv_split_count(4, 32, 128, 100000) == 2           # 128 workgroups: two cuts
    assert kv_split_count(1, 100, 128, 100000) == 5          # 100 workgroups: two rounds of five cuts walk less than one round of two
    assert kv_split_count(1, 32, 100, 4096) == 1             # short KV
    assert kv_split_count(0, 32, 100, 100000) == 1

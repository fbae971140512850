"""ctypes binding of liblsattn.so (the C ABI declared in include/lsattn.h).

The library is the only implementation of the operators in this package: there is no
CPU or PyTorch fallback.  If the shared object is missing or fails to load, importing
an operator raises; build it with `python -m loongserve_amd.build`.
"""
from __future__ import annotations

import ctypes as C
import os

# LSATTN_LIB_PATH selects another build of the same library (same C ABI), e.g. one made with
# different compile-time tuning; the default is the in-tree build next to this file.
LIB_PATH = os.environ.get("LSATTN_LIB_PATH") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "liblsattn.so")

LSATTN_F16, LSATTN_BF16, LSATTN_F32 = 0, 1, 2
LSATTN_MAX_PARTS = 16
LSATTN_MAX_KV_CUTS = 64
LSATTN_STATIC_SCRATCH_BYTES = 64 * 1024 * 1024

_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float


class PrefillArgs(C.Structure):
    _fields_ = [
        ("q", _vp), ("k", _vp), ("v", _vp),
        ("q_stride_t", _i64), ("q_stride_h", _i64),
        ("k_stride_t", _i64), ("k_stride_h", _i64),
        ("v_stride_t", _i64), ("v_stride_h", _i64),
        ("q_b_start_loc", _vp), ("q_b_seq_len", _vp), ("q_first_token_global_idx", _vp),
        ("kv_b_start_loc", _vp), ("kv_b_seq_len", _vp), ("kv_first_token_global_idx", _vp),
        ("batch", _i32), ("num_q_heads", _i32), ("num_kv_heads", _i32), ("head_dim", _i32),
        ("dtype", _i32), ("sp_peers", _i32), ("max_q_len", _i32), ("sm_scale", _f32),
        ("o", _vp), ("o_stride_t", _i64), ("o_stride_h", _i64),
        ("o_dtype", _i32), ("v_is_f16", _i32),
        ("lse", _vp), ("m", _vp), ("l", _vp),
        ("ml_stride_t", _i64), ("ml_stride_h", _i64),
        ("o_b_start_loc", _vp),
        ("kv_cuts", _i32), ("kv_cut_len", _i32), ("o_cut_rows", _i64), ("total_q_rows", _i64),
    ]


class MergeArgs(C.Structure):
    _fields_ = [
        ("n_parts", _i32), ("head_dim", _i32), ("rows", _i64),
        ("o_parts", _vp * LSATTN_MAX_PARTS), ("lse_parts", _vp * LSATTN_MAX_PARTS),
        ("o", _vp), ("o_dtype", _i32), ("reserved", _i32), ("lse", _vp),
    ]


class MergeCutsArgs(C.Structure):  # mirrors lsattn_merge_cuts_args
    _fields_ = [
        ("o_parts", _vp), ("lse_parts", _vp), ("part_rows", _i64), ("n_parts", _i32), ("mode", _i32),
        ("batch", _i32), ("num_q_heads", _i32), ("head_dim", _i32), ("max_q_len", _i32),
        ("q_b_start_loc", _vp), ("q_b_seq_len", _vp),
        ("o", _vp), ("o_stride_t", _i64), ("o_stride_h", _i64), ("o_dtype", _i32), ("reserved", _i32),
        ("lse", _vp), ("m", _vp), ("l", _vp), ("ml_stride_t", _i64), ("ml_stride_h", _i64),
    ]


class DecodeStage1Args(C.Structure):
    _fields_ = [
        ("mid_o", _vp), ("mid_o_logexpsum", _vp), ("q", _vp), ("k", _vp), ("v", _vp),
        ("k_stride_0", _i64), ("k_stride_1", _i64), ("v_stride_0", _i64), ("v_stride_1", _i64),
        ("sm_scale", _f32), ("dtype", _i32),
        ("req_to_tokens", _vp), ("b_req_idx", _vp), ("b_seqlen", _vp),
        ("batch", _i64), ("num_q_heads", _i64), ("num_kv_heads", _i64), ("num_blocks", _i64),
        ("head_dim", _i64), ("max_seq_len", _i64), ("seq_block_size", _i64), ("max_len_in_batch", _i64),
        ("merge_blocks", _i64), ("partials_by_request", _i64),
    ]


class DecodeStage2Args(C.Structure):
    _fields_ = [
        ("o", _vp), ("o_dtype", _i32), ("reserved", _i32), ("out_logexpsum", _vp), ("b_seqlen", _vp),
        ("mid_o", _vp), ("mid_o_logexpsum", _vp),
        ("batch", _i64), ("num_heads", _i64), ("num_seq_blocks", _i64), ("head_dim", _i64), ("block_seq", _i64),
        ("partials_by_request", _i64),
    ]


class Tuning(C.Structure):  # mirrors lsattn_tuning
    _fields_ = [("prefill_rows", _i32), ("prefill_order", _i32), ("prefill_pack", _i32), ("decode_stage1", _i32),
                ("decode_listed", _i32), ("reserved", _i32 * 3)]


# the values of lsattn_tuning's fields by name (0 / None = the library's own choice)
TUNING_VALUES = {
    "prefill_rows": {None: 0, "128": 1, "256": 2, "half": 3},
    "prefill_order": {None: 0, "tile": 1, "head": 2},
    "prefill_pack": {None: 0, "off": 1},
    "decode_stage1": {None: 0, "lane": 1, "mfma": 2, "split": 3},
    "decode_listed": {None: 0, "off": 1, "on": 2, "shares": 3},
}
LSATTN_VERSION = 3  # of include/lsattn.h, which the argument blocks above mirror


# every symbol include/lsattn.h declares: name -> (restype, argtypes)
class KvCopyRegisterArgs(C.Structure):  # mirrors lsattn_kv_copy_register_args
    _fields_ = [("kv", C.c_void_p), ("kv_stride_bytes", C.c_int64), ("pool", C.c_void_p), ("pool_stride_bytes", C.c_int64),
                ("row_bytes", C.c_int64), ("new_kv_cache_len", C.c_void_p), ("kv_range_begin", C.c_void_p),
                ("kv_range_end", C.c_void_p), ("new_kv_cache_len_sum", C.c_void_p), ("kv_b_start_loc", C.c_void_p),
                ("cur_kv_cache_index", C.c_void_p), ("mem_index", C.c_void_p), ("b_req_idx", C.c_void_p),
                ("req_to_tokens", C.c_void_p), ("max_seq_len", C.c_int64), ("batch", C.c_int64),
                ("num_used_mem_index", C.c_int64), ("max_len_in_batch", C.c_int64), ("should_register", C.c_int32),
                ("reserved", C.c_int32)]


class DecodeMigrationArgs(C.Structure):  # mirrors lsattn_decode_migration_args
    _fields_ = [("staging", C.c_void_p), ("staging_layer_stride_bytes", C.c_int64), ("staging_row_stride_bytes", C.c_int64),
                ("kv_cache", C.c_void_p), ("kv_layer_stride_bytes", C.c_int64), ("kv_row_stride_bytes", C.c_int64),
                ("row_bytes", C.c_int64), ("num_layers", C.c_int64), ("req_to_tokens", C.c_void_p), ("max_seq_len", C.c_int64),
                ("mem_state", C.c_void_p), ("alloc_mem", C.c_void_p), ("request_ids", C.c_void_p), ("num_tokens", C.c_void_p),
                ("num_tokens_cumsum", C.c_void_p), ("b_seq_len", C.c_void_p), ("batch", C.c_int64), ("max_num_tokens", C.c_int64)]


class RotaryKvWriteArgs(C.Structure):  # mirrors lsattn_rotary_kv_write_args
    _fields_ = [("q", _vp), ("q_stride_t", _i64), ("q_stride_h", _i64), ("num_q_heads", _i64),
                ("kv", _vp), ("kv_stride_t", _i64), ("kv_stride_h", _i64), ("num_kv_heads", _i64),
                ("cos", _vp), ("sin", _vp), ("num_tokens", _i64), ("head_dim", _i64),
                ("pool", _vp), ("pool_slot_stride", _i64), ("dest_index", _vp),
                ("req_to_tokens", _vp), ("max_seq_len", _i64), ("b_req_idx", _vp), ("b_start_loc", _vp), ("b_seq_len", _vp),
                ("batch", _i64), ("max_len_in_batch", _i64), ("register_mode", _i32), ("reserved", _i32)]


EXPORTS = {
    "lsattn_prefill_step": (C.c_int, [C.POINTER(PrefillArgs), _vp]),
    "lsattn_prefill_step_merge": (C.c_int, [C.POINTER(PrefillArgs), _vp]),
    "lsattn_prefill_step_accumulate": (C.c_int, [C.POINTER(PrefillArgs), _vp]),
    "lsattn_lse_merge": (C.c_int, [C.POINTER(MergeArgs), _vp]),
    "lsattn_prefill_merge_cuts": (C.c_int, [C.POINTER(MergeCutsArgs), _vp]),
    "lsattn_decode_stage1": (C.c_int, [C.POINTER(DecodeStage1Args), _vp]),
    "lsattn_decode_stage2": (C.c_int, [C.POINTER(DecodeStage2Args), _vp]),
    "lsattn_decode_attention": (C.c_int, [C.POINTER(DecodeStage1Args), C.POINTER(DecodeStage2Args), _vp]),
    "lsattn_decode_attention_static": (C.c_int, [C.POINTER(DecodeStage1Args), C.POINTER(DecodeStage2Args), _vp]),
    "lsattn_kv_scatter": (C.c_int, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _vp]),
    "lsattn_register_tokens": (C.c_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "lsattn_register_decode_tokens": (C.c_int, [_vp, _i64, _vp, _vp, _vp, C.c_int32, _i64, _vp]),
    "lsattn_kv_ranges": (C.c_int, [_vp, _vp, _vp, C.c_int32, _i64, _vp, _vp, _vp, _vp]),
    "lsattn_kv_copy_register": (C.c_int, [C.POINTER(KvCopyRegisterArgs), _vp]),
    "lsattn_decode_migration_send": (C.c_int, [C.POINTER(DecodeMigrationArgs), _vp]),
    "lsattn_decode_migration_recv": (C.c_int, [C.POINTER(DecodeMigrationArgs), _vp]),
    "lsattn_rms_norm": (C.c_int, [_vp, _vp, _vp, _i64, _i64, C.c_float, _vp]),
    "lsattn_silu_and_mul_inplace": (C.c_int, [_vp, _i64, _i64, _vp]),
    "lsattn_rotary_kv_write": (C.c_int, [C.POINTER(RotaryKvWriteArgs), _vp]),
    "lsattn_rotary_emb": (C.c_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    "lsattn_pool_search_workspace_bytes": (C.c_size_t, [_i64]),
    "lsattn_pool_alloc": (C.c_int, [_vp, _i64, _i64, _vp, _vp, C.c_size_t, _vp]),
    "lsattn_pool_find_contiguous": (C.c_int, [_vp, _i64, _i64, _vp, _vp, C.c_size_t, _vp]),
    "lsattn_pool_refs_workspace_bytes": (C.c_size_t, [_i64]),
    "lsattn_pool_update_refs": (C.c_int, [_vp, _i64, _vp, _i64, C.c_int, _vp, _vp, C.c_size_t, _vp]),
    "lsattn_bf16_to_f16_rows": (C.c_int, [_vp, _i64, _vp, _i64, _i64, _i64, _vp]),
    "lsattn_set_tuning": (C.c_int, [C.POINTER(Tuning)]),
    "lsattn_strerror": (C.c_char_p, [C.c_int]),
    "lsattn_version": (C.c_int, []),
}

_lib = None


def load():
    """Load liblsattn.so once and type its entry points.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    # PyTorch-ROCm ships a HIP runtime of its own.  Loaded first, it is the one this library's `libamdhip64.so.*`
    # dependency resolves to (same soname), and the process has one runtime; loaded second, the process would hold
    # two, and the library's launches would find no device in theirs (hipErrorNoDevice on the first launch).
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "loongserve_amd: %s is missing; there is no fallback implementation. "
            "Build it with `python -m loongserve_amd.build`." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in EXPORTS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    # the argument blocks carry no size field: a library of another interface version would read them wrongly
    if lib.lsattn_version() != LSATTN_VERSION:
        raise ImportError("loongserve_amd: %s has interface version %d, this package is written against %d; rebuild it with "
                          "`python -m loongserve_amd.build`" % (LIB_PATH, lib.lsattn_version(), LSATTN_VERSION))
    _lib = lib
    return lib


def set_tuning(**choices) -> None:
    """Force launch choices of the library process-wide (lsattn_set_tuning): prefill_rows "128" | "256" | "half",
    prefill_order "tile" | "head", prefill_pack "off", decode_stage1 "lane" | "mfma" | "split", decode_listed "off" | "on" | "shares";
    fields not named (or None) go back to the library's own choice, so set_tuning() restores all of them."""
    t = Tuning()
    for name, value in choices.items():
        if name not in TUNING_VALUES or value not in TUNING_VALUES[name]:
            raise ValueError("unknown tuning choice %s=%r" % (name, value))
        setattr(t, name, TUNING_VALUES[name][value])
    check(load().lsattn_set_tuning(C.byref(t)), "lsattn_set_tuning")


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().lsattn_strerror(rc).decode()
        raise RuntimeError("%s failed: %s (code %d)" % (what, msg, rc))

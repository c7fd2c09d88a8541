"""The structures and entry points of the kernel library's step program as ``ctypes`` sees them
(``csrc/step_program.h``, ``csrc/api.h``): field for field, in the header's order."""
from __future__ import annotations

import ctypes
from ctypes import CFUNCTYPE, POINTER, Structure, c_char_p, c_float, c_int, c_size_t, c_void_p

from tokenmill_amd.hip.library import library

MAX_GROUPS = 8


class TmTune(Structure):
    _fields_ = [("candidates", c_int), ("after", c_int), ("every", c_int)]


class TmLinear(Structure):
    _fields_ = [("w", c_void_p), ("packed", c_void_p), ("bias", c_void_p), ("packed_rows", c_int), ("packed_parts", c_int),
                ("bias_dtype", c_int), ("N", c_int), ("K", c_int), ("dtype", c_int), ("library_first", c_int)]


class TmNorm(Structure):
    _fields_ = [("w", c_void_p), ("w_dtype", c_int), ("eps", c_float)]


class TmEmbedOp(Structure):
    _fields_ = [("table", c_void_p), ("dtype", c_int), ("V", c_int), ("hidden", c_int)]


class TmAttentionOp(Structure):
    _fields_ = [("norm", TmNorm), ("qkv", TmLinear), ("o", TmLinear), ("cos_t", c_void_p), ("sin_t", c_void_p),
                ("k_pool", c_void_p), ("v_pool", c_void_p), ("H", c_int), ("KVH", c_int), ("D", c_int), ("scale", c_float),
                ("window", c_int), ("rot", c_int), ("max_positions", c_int), ("page", c_int), ("group", c_int),
                ("write", c_int)]


class TmFfnOp(Structure):
    _fields_ = [("norm", TmNorm), ("gate_up", TmLinear), ("down", TmLinear), ("I", c_int)]


class TmFinalOp(Structure):
    _fields_ = [("norm", TmNorm), ("head", TmLinear)]


class TmStep(Structure):
    _fields_ = [("T", c_int), ("S", c_int), ("R", c_int), ("num_decode", c_int), ("max_context_len", c_int),
                ("max_decode_context", c_int), ("n_tiles", c_int), ("num_groups", c_int), ("token_ids", c_void_p),
                ("positions", c_void_p), ("seq_of_token", c_void_p), ("context_lens", c_void_p), ("logit_rows", c_void_p),
                ("prefill_tiles", c_void_p), ("block_tables", c_void_p * MAX_GROUPS), ("slot_mapping", c_void_p * MAX_GROUPS),
                ("table_width", c_int * MAX_GROUPS)]


class TmStream(Structure):
    _fields_ = [("resid", c_void_p), ("delta", c_void_p), ("x", c_void_p), ("qkv", c_void_p), ("accumulate", c_int)]


TmHook = CFUNCTYPE(None, c_void_p, c_int, c_int, c_int)

# spans of a run, in the order of the header's TM_LABEL_* numbers
LABELS = ("embed", "qkv", "attention", "o_proj", "gate_up", "down", "norm", "head")
RUN_LABELS, RUN_TUNE_AT_ONCE = 1, 2

# how q|k|v, the feed-forward's activation and the attention of prompt portions were computed, in the order of the
# header's counters
COUNTERS = ("qkv_from_norm", "qkv_panel", "qkv_stream", "qkv_plain", "gate_up_from_norm",
            "gate_up_stream", "gate_up_plain", "prefill_split_keys", "prefill_shared_keys")


def bound():
    """The library with the program's entry points typed."""
    lib = library()
    if getattr(lib, "_tm_program_bound", False):
        return lib
    lib.tm_program_create.restype = c_void_p
    lib.tm_program_create.argtypes = [c_int, c_int]
    lib.tm_program_destroy.restype = None
    lib.tm_program_destroy.argtypes = [c_void_p]
    for name, op in (("tm_program_add_embedding", TmEmbedOp), ("tm_program_add_attention", TmAttentionOp),
                     ("tm_program_add_feed_forward", TmFfnOp), ("tm_program_add_head", TmFinalOp)):
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = [c_void_p, POINTER(op)]
    lib.tm_program_set_hook.restype = None
    lib.tm_program_set_hook.argtypes = [c_void_p, TmHook, c_void_p]
    lib.tm_program_set_tune.restype = c_int
    lib.tm_program_set_tune.argtypes = [c_void_p, c_int, c_int]
    lib.tm_program_workspace_bytes.restype = c_size_t
    lib.tm_program_workspace_bytes.argtypes = [c_void_p, c_int, c_int, c_int, c_int]
    lib.tm_program_counters.restype = None
    lib.tm_program_counters.argtypes = [c_void_p, POINTER(ctypes.c_longlong)]
    lib.tm_program_run.restype = c_int
    lib.tm_program_run.argtypes = [c_void_p, c_int, c_int, POINTER(TmStep), POINTER(TmStream), c_void_p, c_size_t, c_void_p,
                                   c_size_t, c_void_p, c_int, c_void_p]
    lib.tm_linear_accumulates.restype = c_int
    lib.tm_linear_accumulates.argtypes = [POINTER(TmLinear), c_int, c_void_p, c_int, c_int]
    lib.tm_linear_run.restype = c_int
    lib.tm_linear_run.argtypes = [POINTER(TmLinear), c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int,
                                  c_void_p, c_size_t, POINTER(TmTune), c_void_p]
    lib.tm_rule.restype = c_int
    lib.tm_rule.argtypes = [c_char_p]
    lib.tm_decode_split_chunks.restype = c_int
    lib.tm_decode_split_chunks.argtypes = [c_int, c_int, c_int]
    lib._tm_program_bound = True
    return lib

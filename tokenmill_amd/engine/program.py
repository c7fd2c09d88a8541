"""A model's step as one call into the kernel library.

``StepProgram.compile(model, pools)`` walks a ``DecoderModel`` once and describes each of its
operations to the library (``csrc/step_program.hip``): the embedding, for every run call a pre-norm
attention operation and a pre-norm feed-forward operation with their matrices, norms, rotary tables
and cache pools, the final norm and the output head. ``run(step)`` then is one workspace, one
structure with the step's metadata and one call, instead of a few hundred calls from the parts'
Python code; the library chooses the kernels by the same rules as that code, so both give the same
bits (tested). A model with a part the library has no operation for (a mixer with state, a
feed-forward or position encoding defined elsewhere, matrices of another type than the model's) is
not compiled, and its steps run through the parts' own ``forward``.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_size_t, c_void_p

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.hip.library import library
from tokenmill_amd.parts.base import KVCacheView, StepContext

MAX_GROUPS = 8


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


class NotCompilable(Exception):
    """Some part of the model has no operation in the library's step program."""


def _bind(lib) -> None:
    if getattr(lib, "_tm_program_bound", False):
        return
    lib.tm_program_create.restype = c_void_p
    lib.tm_program_create.argtypes = [c_int, c_int]
    lib.tm_program_destroy.restype = None
    lib.tm_program_destroy.argtypes = [c_void_p]
    for name, op in (("tm_program_set_embedding", TmEmbedOp), ("tm_program_add_attention", TmAttentionOp),
                     ("tm_program_add_feed_forward", TmFfnOp), ("tm_program_set_final", TmFinalOp)):
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = [c_void_p, POINTER(op)]
    lib.tm_program_workspace_bytes.restype = c_size_t
    lib.tm_program_workspace_bytes.argtypes = [c_void_p, c_int, c_int, c_int, c_int]
    lib.tm_program_counters.restype = None
    lib.tm_program_counters.argtypes = [c_void_p, POINTER(ctypes.c_longlong)]
    lib.tm_program_run.restype = c_int
    lib.tm_program_run.argtypes = [c_void_p, POINTER(TmStep), c_void_p, c_size_t, c_void_p, c_size_t, c_void_p, c_void_p]
    lib._tm_program_bound = True


def _norm(part, dtype) -> TmNorm:
    from tokenmill_amd.parts.norm import RMSNorm
    if type(part) is not RMSNorm or part.weight is None:
        raise NotCompilable(f"norm {type(part).__name__}")
    return TmNorm(part.weight.data_ptr(), ops.code(part.weight.dtype), part.eps)


def _linear(part, dtype) -> TmLinear:
    from tokenmill_amd.parts.linear import Linear
    w = part.weight
    if type(part) is not Linear or w is None or w.dtype != dtype or not w.is_contiguous():
        raise NotCompilable("a matrix of another type than the model's")
    bias = part.bias
    packed = part.packed
    return TmLinear(w.data_ptr(), packed.data.data_ptr() if packed is not None else None,
                    bias.data_ptr() if bias is not None else None, packed.rows if packed is not None else 0,
                    len(packed.parts) if packed is not None else 0, ops.code(bias.dtype) if bias is not None else -1,
                    part.out_features, part.in_features, ops.code(w.dtype), 1 if part.library_first else 0)


class StepProgram:
    def __init__(self, model, pools, handle: int, lib):
        self.model, self.pools = model, pools           # keep every tensor the program points at alive
        self._handle, self._lib = handle, lib
        self.vocab = model.head.vocab
        self.device = model.device
        self.runs = 0

    def __del__(self):
        if getattr(self, "_handle", None):
            self._lib.tm_program_destroy(self._handle)
            self._handle = None

    @classmethod
    def compile(cls, model, pools) -> "StepProgram | None":
        """The program of ``model`` over the cache ``pools``, or None if the model has a part the library's
        program has no operation for."""
        try:
            return cls._compile(model, pools)
        except NotCompilable:
            return None

    @classmethod
    def _compile(cls, model, pools) -> "StepProgram":
        from tokenmill_amd.parts.attention import GQAttention
        from tokenmill_amd.parts.block import PreNormBlock
        from tokenmill_amd.parts.embedding import OutputHead, TokenEmbedding
        from tokenmill_amd.parts.mlp import SwiGLU
        from tokenmill_amd.parts.position import NoPositionEncoding, RotaryEmbedding

        dtype = model.dtype
        if type(model.embedding) is not TokenEmbedding or type(model.head) is not OutputHead or pools.states \
                or len(pools.groups) > MAX_GROUPS:
            raise NotCompilable("embedding, head or per-request state")
        lib = library()
        _bind(lib)
        hidden = model.embedding.hidden
        handle = lib.tm_program_create(ops.code(dtype), hidden)
        if not handle:
            raise NotCompilable("the library refused the model's type")
        program = cls(model, pools, handle, lib)

        def check(rc, what):
            if rc != 0:
                raise NotCompilable(f"the library refused {what}")

        emb = model.embedding
        check(lib.tm_program_set_embedding(handle, TmEmbedOp(emb.weight.data_ptr(), ops.code(emb.weight.dtype), emb.vocab, hidden)),
              "the embedding")
        for j, call in enumerate(model.run):
            block = model.layers[call.layer]
            view = pools.views[j]
            if type(block) is not PreNormBlock or type(block.mixer) is not GQAttention or type(block.ffn) is not SwiGLU \
                    or not isinstance(view, KVCacheView):
                raise NotCompilable(f"layer {call.layer}")
            m, pos = block.mixer, block.mixer.position
            if type(pos) is RotaryEmbedding:
                cos, sin, rot, n_pos = pos.cos.data_ptr(), pos.sin.data_ptr(), pos.rotary_dim, pos.max_positions
            elif type(pos) is NoPositionEncoding:
                cos = sin = None
                rot = n_pos = 0
            else:
                raise NotCompilable(f"position encoding {type(pos).__name__}")
            att = TmAttentionOp(_norm(block.norm_in, dtype), _linear(m.qkv, dtype), _linear(m.o, dtype), cos, sin,
                                view.k.data_ptr(), view.v.data_ptr(), m.num_heads, m.num_kv_heads, m.head_dim, m.scale,
                                m.window or 0, rot, n_pos, view.k.shape[1], view.group, 1 if view.write else 0)
            check(lib.tm_program_add_attention(handle, att), f"the attention of layer {call.layer}")
            f = block.ffn
            if f.gate_up.bias is not None or f.down.bias is not None:
                raise NotCompilable("a feed-forward with biases")
            ffn = TmFfnOp(_norm(block.norm_post, dtype), _linear(f.gate_up, dtype), _linear(f.down, dtype), f.intermediate)
            check(lib.tm_program_add_feed_forward(handle, ffn), f"the feed-forward of layer {call.layer}")
        check(lib.tm_program_set_final(handle, TmFinalOp(_norm(model.final_norm, dtype), _linear(model.head.proj, dtype))),
              "the output head")
        return program

    COUNTERS = ("qkv_from_norm", "qkv_panel", "qkv_plain", "gate_up_from_norm", "gate_up_panel", "gate_up_plain")

    def counters(self) -> dict[str, int]:
        """How often each way of computing q|k|v and the feed-forward's activation has been taken."""
        out = (ctypes.c_longlong * len(self.COUNTERS))()
        self._lib.tm_program_counters(self._handle, out)
        return dict(zip(self.COUNTERS, out))

    def run(self, step: StepContext) -> torch.Tensor:
        """The step's float32 logits [R, vocab] at ``step.logit_rows``."""
        lib = self._lib
        T, R = step.num_tokens, step.num_logit_rows
        s = TmStep()
        s.T, s.S, s.R, s.num_decode = T, step.num_seqs, R, step.num_decode
        s.max_context_len, s.max_decode_context = step.max_context_len, step.max_decode_context
        tiles = step.prefill_tiles
        s.n_tiles = tiles.shape[0] if tiles is not None else 0
        s.prefill_tiles = tiles.data_ptr() if s.n_tiles else None
        s.num_groups = len(step.groups)
        s.token_ids, s.positions = step.token_ids.data_ptr(), step.positions.data_ptr()
        s.seq_of_token, s.context_lens = step.seq_of_token.data_ptr(), step.context_lens.data_ptr()
        s.logit_rows = step.logit_rows.data_ptr() if R else None
        for g, group in enumerate(step.groups):
            s.block_tables[g] = group.block_tables.data_ptr()
            s.slot_mapping[g] = group.slot_mapping.data_ptr()
            s.table_width[g] = group.block_tables.shape[1]
        need = lib.tm_program_workspace_bytes(self._handle, T, R, step.num_decode, step.max_decode_context)
        workspace = torch.empty(need, dtype=torch.uint8, device=self.device)
        logits = torch.empty((R, self.vocab), dtype=torch.float32, device=self.device)
        lib_ws = ops.library_workspace(self.device)
        rc = lib.tm_program_run(self._handle, ctypes.byref(s), workspace.data_ptr(), need, lib_ws.data_ptr(),
                                ops.LIBRARY_WORKSPACE_BYTES, logits.data_ptr() if R else None, ops._stream())
        if rc == 1:
            raise ops.KernelArgumentError("the step program refused the step (a size or position a kernel does not run)")
        if rc != 0:
            raise RuntimeError(f"the step program failed (code {rc})")
        self.runs += 1
        return logits

"""Checked calls into the HIP kernels.

Every wrapper checks on the host that the operands are on the GPU, contiguous where the kernel
assumes it, of a type the kernel has, and of shapes that fit each other and the kernel's limits,
BEFORE anything is launched; a kernel never sees a size it was not written for. Refusals raise
``KernelArgumentError`` with the offending value.
"""
from __future__ import annotations

import contextlib
import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from tokenmill_amd.hip.library import library

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def code(dtype: torch.dtype) -> int:
    _need(dtype in _CODES, f"kernels exist for float32 and bfloat16, not {dtype}")
    return _CODES[dtype]


def _gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operand is not on the GPU (there is no CPU path)")


def _p(t: torch.Tensor | None) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _stream() -> c_void_p:
    # the current stream of the current device, straight from the C layer: the Python-level
    # torch.cuda.current_stream() costs more than a launch
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _check(rc: int, name: str) -> None:
    if rc == 1:
        raise KernelArgumentError(f"{name}: the kernel refused its arguments")
    if rc != 0:
        raise RuntimeError(f"{name}: launch failed (code {rc})")


def _check_pools(k_pool: torch.Tensor, v_pool: torch.Tensor, KVH: int, D: int, dtype, who: str) -> int:
    """K pool [pages, page, KVH, D], V pool [pages, KVH, D, page]; returns the page size."""
    _need(k_pool.dim() == 4 and v_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          f"{who}: the cache pools must be contiguous 4-d tensors")
    pages, page = k_pool.shape[0], k_pool.shape[1]
    _need(tuple(k_pool.shape) == (pages, page, KVH, D), f"{who}: k_pool must be [pages, page, {KVH}, {D}]")
    _need(tuple(v_pool.shape) == (pages, KVH, D, page), f"{who}: v_pool must be [pages, {KVH}, {D}, page]")
    _need(k_pool.dtype == dtype and v_pool.dtype == dtype, f"{who}: the cache pools must have the type {dtype}")
    return page


def _ints(t: torch.Tensor, n: int, name: str) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n, f"{name} must be contiguous int32 [{n}]")


# --------------------------------------------------------------------------------------------

def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]] as 32-bit rows. table [V, hidden], ids int32 [T], out float32 [T, hidden]."""
    _gpu(table, ids, out)
    T = ids.numel()
    V, hidden = table.shape
    _need(table.is_contiguous() and out.is_contiguous(), "embed_gather: operands must be contiguous")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (T, hidden), "embed_gather: out must be float32 [T, hidden]")
    _ints(ids, T, "ids")
    _check(library().tm_embed_gather(_p(table), code(table.dtype), _p(ids), _p(out), c_int(T), c_int(hidden),
                                     c_int(V), _stream()), "embed_gather")
    return out


def add_rmsnorm(resid: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
    """rows None: resid += delta (in place, 32-bit), out = rmsnorm(resid) * weight, all rows.
    rows given: out[r] = rmsnorm(resid[rows[r]] + delta[rows[r]]) * weight; resid is not written."""
    _gpu(resid, delta, weight, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "add_rmsnorm: the residual stream is contiguous float32")
    _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"add_rmsnorm: out must be [{R}, {hidden}]")
    if delta is not None:
        _need(delta.dtype == out.dtype and tuple(delta.shape) == (T, hidden) and delta.is_contiguous(),
              "add_rmsnorm: delta must match the residual's shape and out's type")
    _need(tuple(weight.shape) == (hidden,) and weight.is_contiguous(), "add_rmsnorm: weight must be [hidden]")
    _need(out.dtype == torch.bfloat16 or weight.dtype == torch.float32, "add_rmsnorm: a float32 output needs float32 weights")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "add_rmsnorm: eps must be positive")
    _check(library().tm_add_rmsnorm(_p(resid), _p(delta), _p(rows), _p(weight), code(weight.dtype), _p(out),
                                    code(out.dtype), c_int(R), c_int(hidden), c_float(eps), _stream()), "add_rmsnorm")
    return out


def rope_kv_write(qkv: torch.Tensor, H: int, KVH: int, D: int, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  positions: torch.Tensor | None, slots: torch.Tensor | None, k_pool: torch.Tensor | None,
                  v_pool: torch.Tensor | None) -> None:
    """Rotate q and k of qkv [T, (H + 2 KVH) D] in place by each token's position and store k, v at
    the tokens' cache slots. cos/sin float32 [max_pos, rot/2] or None (store only); k_pool
    [pages, page, KVH, D] and v_pool [pages, KVH, D, page], or None (rotate only). A slot < 0 is
    not stored."""
    _gpu(qkv, cos, sin, positions, slots, k_pool, v_pool)
    T = qkv.shape[0]
    _need(qkv.is_contiguous() and qkv.shape[1] == (H + 2 * KVH) * D, "rope_kv_write: qkv must be contiguous [T, (H+2KVH)D]")
    rot = 0
    if cos is not None:
        _need(sin is not None and positions is not None, "rope_kv_write: cos needs sin and positions")
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
              and cos.shape == sin.shape and cos.dim() == 2, "rope_kv_write: cos/sin must be float32 [max_pos, rot/2]")
        rot = 2 * cos.shape[1]
        _need(0 < rot <= D, f"rope_kv_write: rotary width {rot} does not fit head size {D}")
        _ints(positions, T, "positions")
    write = k_pool is not None
    page = 0
    if write:
        _need(v_pool is not None and slots is not None, "rope_kv_write: a cache write needs both pools and slots")
        page = _check_pools(k_pool, v_pool, KVH, D, qkv.dtype, "rope_kv_write")
        _ints(slots, T, "slots")
    _check(library().tm_rope_kv_write(_p(qkv), code(qkv.dtype), c_int(T), c_int(H), c_int(KVH), c_int(D), c_int(rot),
                                      _p(cos), _p(sin), _p(positions), _p(slots), _p(k_pool), _p(v_pool),
                                      c_int(page), c_int(1 if write else 0), _stream()), "rope_kv_write")


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gu[t, i]) * gu[t, I + i]; gu [T, 2I], out [T, I]."""
    _gpu(gu, out)
    T, two_i = gu.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and gu.is_contiguous() and out.is_contiguous()
          and gu.dtype == out.dtype, "silu_mul: gu [T, 2I] and out [T, I] of one type, contiguous")
    _check(library().tm_silu_mul(_p(gu), _p(out), code(gu.dtype), c_int(T), c_int(two_i // 2), _stream()), "silu_mul")
    return out


def convert(src: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(src, out)
    _need(src.is_contiguous() and out.is_contiguous() and src.numel() == out.numel(), "convert: same size, contiguous")
    _check(library().tm_convert(_p(src), code(src.dtype), _p(out), code(out.dtype), c_longlong(src.numel()),
                                _stream()), "convert")
    return out


def gemm_nt_tiled(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]) with 32-bit multiply-adds in ascending k.
    a and out may be row-strided views (unit stride in the last dimension)."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and w.is_contiguous() and w.dtype == a.dtype, "gemm: w must be contiguous [N, K] of a's type")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and tuple(out.shape) == (M, N), "gemm: a [M, K], out [M, N], unit inner stride")
    _need(not (a.dtype == torch.float32 and out.dtype != torch.float32), "gemm: float32 inputs give float32 outputs")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm: bias must be [N]")
        _need(not (a.dtype == torch.float32 and bias.dtype != torch.float32), "gemm: float32 inputs need a float32 bias")
    _need(M <= 64 * 65535, "gemm: too many rows for one launch")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemm_nt_tiled(_p(a), c_int(lda), _p(w), _p(bias),
                                      c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                      c_int(M), c_int(N), c_int(K), code(a.dtype), code(out.dtype), _stream()),
           "gemm_nt_tiled")
    return out


LIBRARY_WORKSPACE_BYTES = 32 << 20
_library_workspace: dict[int, torch.Tensor] = {}


def library_workspace(device: torch.device) -> torch.Tensor:
    """The device memory the library products may use; made once per device (call it before any
    graph capture, so that the capture allocates nothing for it)."""
    ws = _library_workspace.get(device.index)
    if ws is None:
        ws = _library_workspace[device.index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


TUNE_AFTER_CALLS = 3        # a shape's candidates are timed when it is called this often (most shapes of a serving run come once)
_tune_now: tuple[int, int, bool] | None = None


@contextlib.contextmanager
def tuning(candidates: int, after: int = TUNE_AFTER_CALLS, every: bool = False):
    """Inside, the library products that this module's ``linear`` and ``gemm_library`` launch time up to
    ``candidates`` of the library's algorithms on their own operands when a shape is called the ``after``-th
    time with the same matrix (outside a graph capture) and keep the fastest (``every``: a shape timed at its
    first call also tries every algorithm the library holds for the operand types: about a second a shape,
    and an algorithm found that way is kept only if it gives the first choice's result). Timing is a
    property of the caller, not of the process: an engine that asks for it wraps its own steps in this, and
    the plans of timed callers are kept apart from the plans of the others."""
    global _tune_now
    _need(0 <= candidates <= 32 and after >= 1, "tuning: 0 to 32 candidates, after >= 1 calls")
    _need(not every or candidates >= 2, "tuning: every algorithm is tried beside at least 2 candidates")
    saved, _tune_now = _tune_now, (candidates, after, every)
    try:
        yield
    finally:
        _tune_now = saved


def _tune_arg(tune: tuple[int, int, bool] | None):
    """The TmTune argument of a library product: ``tune`` if given, else what an open ``tuning()`` says, else null."""
    from tokenmill_amd.hip.abi import TmTune
    t = tune if tune is not None else _tune_now
    if t is None or t[0] < 2:
        return None
    return ctypes.byref(TmTune(int(t[0]), int(t[1]), 1 if t[2] else 0))


def rule(name: str) -> int:
    """A number of the library's kernel-choosing rules (``csrc/choose.h``), for sizing a buffer or checking an
    argument: "skinny_rows", "panel_qkv_rows", "stream_rows", "skinny_max_rows", "gemv_f32_rows", "decode_chunk",
    "decode_split_pairs". The rules themselves are applied inside the library only."""
    value = _rules.get(name)
    if value is None:
        from tokenmill_amd.hip.abi import bound
        value = bound().tm_rule(name.encode())
        _need(value >= 0, f"the kernel library has no rule named {name!r}")
        _rules[name] = value
    return value


_rules: dict[str, int] = {}


def gemm_library(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                 tune: tuple[int, int, bool] | None = None) -> bool:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]) by hipBLASLt: bfloat16 inputs, 32-bit sums, out
    bfloat16 or float32. The plan for a shape is made on its first call and kept. Returns False
    (nothing written) if the library has no algorithm for this product. ``tune``: (candidates, after, every)
    as for ``tuning()``, which it overrides."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32),
          "gemm_library: bfloat16 inputs, bfloat16 or float32 output")
    _need(w.shape[1] == K and w.is_contiguous(), "gemm_library: w must be contiguous [N, K]")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and tuple(out.shape) == (M, N),
          "gemm_library: a [M, K], out [M, N], unit inner stride")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous() and bias.dtype in (torch.bfloat16, torch.float32),
              "gemm_library: bias must be contiguous [N], bfloat16 or float32")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    ws = library_workspace(a.device)
    rc = library().tm_gemm_library(_p(a), c_int(lda), _p(w), c_int(K), _p(bias),
                                   c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                   c_int(1 if out.dtype == torch.float32 else 0), c_int(M), c_int(N), c_int(K),
                                   _p(ws), ctypes.c_size_t(LIBRARY_WORKSPACE_BYTES), _tune_arg(tune), _stream())
    if rc == 3:
        return False
    _check(rc, "gemm_library")
    return True


def gemv_f32_ok(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> bool:
    M, K = a.shape
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    return (a.dtype == torch.float32 and w.dtype == torch.float32 and out.dtype == torch.float32
            and (bias is None or bias.dtype == torch.float32) and 0 < M <= rule("gemv_f32_rows") and K % 4 == 0
            and lda % 4 == 0 and a.stride(1) == 1 and out.stride(1) == 1 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemv_f32(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]), everything float32, M <= 16: 32-bit multiply-adds
    in an order that depends on K only."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(gemv_f32_ok(a, w, bias, out), "gemv_f32: float32 operands, at most 16 rows, K a multiple of 4, 16-byte aligned")
    _need(w.shape[1] == K and w.is_contiguous() and tuple(out.shape) == (M, N), "gemv_f32: w [N, K] contiguous, out [M, N]")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemv_f32: bias must be [N]")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemv_f32(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M), c_int(N),
                                 c_int(K), _stream()), "gemv_f32")
    return out


def gemm_f32_mfma_ok(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> bool:
    """Does the float32 product on the 32-bit matrix unit take these operands?"""
    if not (a.dtype == w.dtype == out.dtype == torch.float32 and (bias is None or bias.dtype == torch.float32)
            and a.dim() == 2 and a.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous()):
        return False
    M, K = a.shape
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(w.shape[0], out.stride(0))
    return bool(library().tm_gemm_f32_mfma_fits(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M),
                                                c_int(w.shape[0]), c_int(K)))


def gemm_f32_mfma(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]), everything float32, on the 32-bit matrix unit: 32-bit
    products and sums in an order that depends on K only. K must be a multiple of 16, N and the row strides of 4,
    and the operands 16-byte aligned."""
    _gpu(a, w, bias, out)
    _need(gemm_f32_mfma_ok(a, w, bias, out), "gemm_f32_mfma: float32 operands, K a multiple of 16, N and row strides of 4, 16-byte aligned")
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and tuple(out.shape) == (M, N), "gemm_f32_mfma: w [N, K], out [M, N]")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_f32_mfma: bias must be [N]")
    _need(M <= 64 * 65535, "gemm_f32_mfma: too many rows for one launch")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemm_f32_mfma(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M), c_int(N),
                                      c_int(K), _stream()), "gemm_f32_mfma")
    return out


def attn_paged_generic(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       block_tables: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                       H: int, KVH: int, D: int, scale: float, window: int = 0) -> torch.Tensor:
    """Attention of every token of the step over its request's cached keys (its own included).
    q: [T, >= H*D] view with unit inner stride (q heads first in each row); out [T, H*D];
    k_pool [pages, page, KVH, D], v_pool [pages, KVH, D, page]; block_tables int32 [S, W];
    seq_of_token, positions int32 [T]."""
    _gpu(q, out, k_pool, v_pool, block_tables, seq_of_token, positions)
    T = q.shape[0]
    _need(q.stride(1) == 1 and q.shape[1] >= H * D and out.is_contiguous() and tuple(out.shape) == (T, H * D),
          "attention: q [T, >=H*D] unit inner stride, out contiguous [T, H*D]")
    _need(q.dtype == out.dtype, "attention: q and out share one type")
    _need(H % KVH == 0 and D % 4 == 0 and 0 < D <= 256, f"attention(generic): head size {D} must be a multiple of 4 up to 256")
    _check_pools(k_pool, v_pool, KVH, D, q.dtype, "attention")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention: block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    _need(window >= 0, "attention: window must be >= 0 (0 = every key)")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    _check(library().tm_attn_paged_generic(_p(q), c_int(q_stride), _p(out), c_int(H * D), _p(k_pool), _p(v_pool),
                                           _p(block_tables), c_int(block_tables.shape[1]), _p(seq_of_token),
                                           _p(positions), c_int(T), c_int(H), c_int(KVH), c_int(D),
                                           c_int(k_pool.shape[1]), c_float(scale), c_int(window), code(q.dtype),
                                           _stream()), "attn_paged_generic")
    return out


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "argmax: logits must be contiguous float32 [R, V]")
    _ints(out, R, "out")
    nb = library().tm_argmax_work_chunks(c_int(V))
    work_v = work_i = None
    if nb > 1:                                   # a wide vocabulary: every row is cut over nb blocks
        work_v = torch.empty(R * nb, dtype=torch.float32, device=logits.device)
        work_i = torch.empty(R * nb, dtype=torch.int32, device=logits.device)
    _check(library().tm_argmax_rows(_p(logits), c_int(R), c_int(V), _p(out), _p(work_v), _p(work_i), _stream()),
           "argmax_rows")
    return out


_sample_work: dict[int, torch.Tensor] = {}


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                u: torch.Tensor, out: torch.Tensor, uses_top_k: bool = True, uses_top_p: bool = True) -> torch.Tensor:
    """One token per row: argmax where temperature <= 1e-5 or top_k == 1, else the inverse CDF at
    u of softmax(logits / temperature) after the top-k / top-p filters, in vocabulary order.
    ``uses_top_k`` / ``uses_top_p``: False if the caller knows that no row asks for that filter (its
    launches are then left out; a row that asks for none skips their work either way)."""
    _gpu(logits, temperature, top_k, top_p, u, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be contiguous float32 [R, V]")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (u, "u")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == R, f"sample: {name} must be float32 [R]")
    _ints(top_k, R, "top_k")
    _ints(out, R, "out")
    _need(V <= 1 << 20, f"sample: at most 2^20 logits a row, got {V}")
    lib = library()
    lib.tm_sample_work_bytes.restype = ctypes.c_size_t
    need = lib.tm_sample_work_bytes(c_int(R), c_int(V))
    work = _sample_work.get(logits.device.index)
    if work is None or work.numel() < need:            # kept and grown: one sampling call at a time per device
        work = _sample_work[logits.device.index] = torch.empty(need, dtype=torch.uint8, device=logits.device)
    _check(lib.tm_sample_rows(_p(logits), c_int(R), c_int(V), _p(temperature), _p(top_k), _p(top_p), _p(u), _p(out),
                              _p(work), ctypes.c_size_t(work.numel()), c_int((1 if uses_top_k else 0) | (2 if uses_top_p else 0)),
                              _stream()), "sample_rows")
    return out


class PackedWeight:
    """A bfloat16 matrix [N, K] (or several stacked parts of one K) in the strip order the decode-step
    products read: ``data[((s * KS + ks) * 4 + g) * rows + r, i] = W[s * rows + r, 32 ks + 8 g + i]`` with
    KS = ceil(K / 32), zero where the row or the k does not exist, so that a wavefront's load of a k-step
    of a strip is one run of rows * 64 bytes. Each part of ``parts`` (rows per part) starts a strip of its
    own: the strips of the second part lie behind those of the first."""

    def __init__(self, data: torch.Tensor, n: int, k: int, rows: int, parts: tuple[int, ...]):
        self.data, self.n, self.k, self.rows, self.parts = data, n, k, rows, parts


def pack_weight(w: torch.Tensor, rows: int, parts: list[int] | None = None) -> PackedWeight:
    """w bfloat16 [N, K] on the GPU -> its strip order in strips of ``rows`` (16, 8 or 4) rows."""
    _gpu(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and rows in (4, 8, 16), "pack_weight: bfloat16 [N, K], strips of 4, 8 or 16 rows")
    N, K = w.shape
    parts = [N] if parts is None else list(parts)
    _need(sum(parts) == N and all(p > 0 for p in parts), "pack_weight: the parts must add up to the matrix's rows")
    ks = -(-K // 32)
    out, row0 = [], 0
    for n in parts:
        strips = -(-n // rows)
        padded = torch.zeros((strips * rows, ks * 32), dtype=w.dtype, device=w.device)
        padded[:n, :K] = w[row0:row0 + n]
        # [s, r, ks, g, i] -> [s, ks, g, r, i]
        out.append(padded.view(strips, rows, ks, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))
        row0 += n
    data = torch.cat(out) if len(out) > 1 else out[0].contiguous()
    return PackedWeight(data, N, K, rows, tuple(parts))


def linear_desc(w: torch.Tensor, packed: "PackedWeight | None", bias: torch.Tensor | None, library_first: bool = False):
    """A matrix as the library's product rule takes it (a ``TmLinear``; the caller keeps the tensors alive)."""
    from tokenmill_amd.hip.abi import TmLinear
    _gpu(w, bias)
    _need(w.dim() == 2 and w.is_contiguous(), "linear: the matrix must be contiguous [N, K]")
    if bias is not None:
        _need(tuple(bias.shape) == (w.shape[0],) and bias.is_contiguous(), "linear: bias must be [N]")
    if packed is not None:
        _packed_operand(packed, None, "linear")
        _need((packed.n, packed.k) == tuple(w.shape), "linear: the packed copy is of another matrix")
    return TmLinear(w.data_ptr(), packed.data.data_ptr() if packed is not None else None,
                    bias.data_ptr() if bias is not None else None, packed.rows if packed is not None else 0,
                    len(packed.parts) if packed is not None else 0, code(bias.dtype) if bias is not None else -1,
                    w.shape[0], w.shape[1], code(w.dtype), 1 if library_first else 0)


def _linear_input(desc, x: torch.Tensor) -> int:
    _gpu(x)
    _need(x.dim() == 2 and x.shape[1] == desc.K and x.stride(1) == 1, f"linear: x must be [M, {desc.K}] with unit inner stride")
    _need(code(x.dtype) == desc.dtype, "linear: x must have the matrix's type (widen it for a 32-bit matrix)")
    return x.stride(0) if x.shape[0] > 1 else max(desc.K, x.stride(0))


def linear_accumulates(desc, x: torch.Tensor) -> bool:
    """Is there a kernel that adds round(x W^T + b) into a 32-bit tensor in its own epilogue, for these operands?"""
    from tokenmill_amd.hip.abi import bound
    ldx = _linear_input(desc, x)
    return bool(bound().tm_linear_accumulates(ctypes.byref(desc), code(x.dtype), _p(x), ldx, x.shape[0]))


def linear(desc, x: torch.Tensor, out: torch.Tensor | None, accum: torch.Tensor | None = None,
           tune: tuple[int, int, bool] | None = None) -> torch.Tensor:
    """out[M, N] = x[M, K] W^T (+ bias) by the kernel the library's product rule chooses for the row count and
    types (``desc``: ``linear_desc``). With ``accum`` (float32 [M, N]; only where ``linear_accumulates``) the
    result, rounded to the matrix's type, is added there instead and ``out`` stays unwritten."""
    from tokenmill_amd.hip.abi import bound
    ldx = _linear_input(desc, x)
    M = x.shape[0]
    ws = library_workspace(x.device)
    if accum is not None:
        _gpu(accum)
        _need(accum.dtype == torch.float32 and tuple(accum.shape) == (M, desc.N) and accum.stride(1) == 1,
              f"linear: accum must be float32 [{M}, {desc.N}]")
        ldacc = accum.stride(0) if M > 1 else max(desc.N, accum.stride(0))
        _check(bound().tm_linear_run(ctypes.byref(desc), code(x.dtype), _p(x), ldx, M, None, 0, 0, _p(accum), ldacc, _p(ws),
                                     LIBRARY_WORKSPACE_BYTES, _tune_arg(tune), _stream()), "linear")
        return accum
    _gpu(out)
    _need(out is not None and tuple(out.shape) == (M, desc.N) and out.stride(1) == 1, f"linear: out must be [{M}, {desc.N}]")
    _need(not (x.dtype == torch.float32 and out.dtype != torch.float32), "linear: float32 inputs give float32 outputs")
    ldc = out.stride(0) if M > 1 else max(desc.N, out.stride(0))
    _check(bound().tm_linear_run(ctypes.byref(desc), code(x.dtype), _p(x), ldx, M, _p(out), ldc, code(out.dtype), None, 0,
                                 _p(ws), LIBRARY_WORKSPACE_BYTES, _tune_arg(tune), _stream()), "linear")
    return out


def skinny_strip_rows(N: int, K: int) -> int:
    """Rows of a strip the skinny product wants an [N, K] matrix packed in."""
    return int(library().tm_skinny_strip_rows(c_int(N), c_int(K)))


def fused_qkv_strip_rows(H: int, KVH: int, D: int, K: int) -> int:
    """Rows of a strip the norm-fused q|k|v product wants its matrix packed in."""
    return int(library().tm_fused_qkv_strip_rows(c_int(H), c_int(KVH), c_int(D), c_int(K)))


def _packed_operand(w: PackedWeight, rows_expected: int | None, who: str) -> None:
    _need(isinstance(w, PackedWeight) and w.data.is_cuda and w.data.dtype == torch.bfloat16 and w.data.is_contiguous()
          and w.data.data_ptr() % 16 == 0, f"{who}: the matrix must be a PackedWeight on the GPU")
    if rows_expected is not None:
        _need(w.rows == rows_expected, f"{who}: the matrix is packed in strips of {w.rows} rows, the kernel reads {rows_expected}")


def gemm_skinny(a: torch.Tensor, w: "torch.Tensor | PackedWeight", bias: torch.Tensor | None,
                out: torch.Tensor | None, silu: bool = False, accum: torch.Tensor | None = None) -> torch.Tensor:
    """MFMA product for at most 64 rows of bfloat16 activations: out[M, N] = a @ w^T (+ bias), or with
    ``silu`` out[M, N] = silu(a @ w[:N]^T) * (a @ w[N:]^T) for a stacked [gate; up] matrix w [2N, K].
    out is bfloat16 or float32 (float32 not with silu). With ``accum`` (float32 [M, N]) nothing is
    stored to out: the result, rounded to bfloat16, is added into accum (the residual stream).
    w may be a ``PackedWeight`` (at most 16 rows of a then; with silu packed as two parts of 16-row
    strips): the same bits, read faster."""
    if isinstance(w, PackedWeight):
        return _gemm_skinny_packed(a, w, bias, out, silu, accum)
    _gpu(a, w, bias, out, accum)
    M, K = a.shape
    if accum is not None:
        _need(out is None and not silu and accum.dtype == torch.float32 and accum.dim() == 2 and accum.shape[0] == M
              and accum.stride(1) == 1, "gemm_skinny: accum must be float32 [M, N], and excludes out and silu")
        N = accum.shape[1]
        _need(tuple(w.shape) == (N, K) and w.is_contiguous() and a.dtype == w.dtype == torch.bfloat16 and 0 < M <= 64
              and a.stride(1) == 1, "gemm_skinny: bfloat16 a [M<=64, K], contiguous w [N, K]")
        lda = a.stride(0) if M > 1 else max(K, a.stride(0))
        _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
              "gemm_skinny: K and the row stride must be multiples of 8 and the operands 16-byte aligned")
        if bias is not None:
            _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N]")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        _check(library().tm_gemm_skinny(_p(a), c_int(lda), _p(w), _p(bias),
                                        c_int(code(bias.dtype) if bias is not None else -1), _p(None), c_int(N),
                                        c_int(M), c_int(N), c_int(K), c_int(BF16), c_int(0), _p(accum), c_int(ldacc),
                                        _stream()), "gemm_skinny")
        return accum
    N = out.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 inputs")
    _need(0 < M <= 64, f"gemm_skinny: at most 64 rows, got {M}")
    _need(w.is_contiguous() and tuple(w.shape) == ((2 * N if silu else N), K), "gemm_skinny: w must be contiguous [N, K]")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and out.shape[0] == M, "gemm_skinny: unit inner strides")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
          "gemm_skinny: K and the row stride must be multiples of 8 and the operands 16-byte aligned")
    _need(out.dtype in (torch.bfloat16, torch.float32) and not (silu and out.dtype != torch.bfloat16),
          "gemm_skinny: out is bfloat16, or float32 without silu")
    if bias is not None:
        _need(not silu and tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N], not with silu")
    _check(library().tm_gemm_skinny(_p(a), c_int(lda), _p(w), _p(bias),
                                    c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                    c_int(M), c_int(N), c_int(K), code(out.dtype), c_int(1 if silu else 0),
                                    _p(None), c_int(0), _stream()), "gemm_skinny")
    return out


def _gemm_skinny_packed(a, w: PackedWeight, bias, out, silu: bool, accum) -> torch.Tensor:
    _gpu(a, bias, out, accum)
    _packed_operand(w, 16 if silu else None, "gemm_skinny")
    M, K = a.shape
    N = w.n // 2 if silu else w.n
    _need(a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1 and 0 < M <= rule("skinny_rows") and K == w.k,
          f"gemm_skinny: bfloat16 a [M<={rule('skinny_rows')}, {w.k}] for a packed matrix")
    _need(w.parts == ((N, N) if silu else (w.n,)), "gemm_skinny: with silu the matrix is packed as its two halves, else as one part")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0,
          "gemm_skinny: K and the row stride must be multiples of 8 and the activations 16-byte aligned")
    if bias is not None:
        _need(not silu and tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N], not with silu")
    if accum is not None:
        _need(out is None and not silu and accum.dtype == torch.float32 and tuple(accum.shape) == (M, N)
              and accum.stride(1) == 1, "gemm_skinny: accum must be float32 [M, N], and excludes out and silu")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        c, ldc, out_code = None, N, BF16
    else:
        _need(out is not None and tuple(out.shape) == (M, N) and out.stride(1) == 1
              and out.dtype in (torch.bfloat16, torch.float32) and not (silu and out.dtype != torch.bfloat16),
              "gemm_skinny: out [M, N] bfloat16, or float32 without silu")
        ldacc = 0
        c, ldc, out_code = out, (out.stride(0) if M > 1 else max(N, out.stride(0))), code(out.dtype)
    _check(library().tm_gemm_skinny_packed(_p(a), c_int(lda), _p(w.data), c_int(w.rows), _p(bias),
                                           c_int(code(bias.dtype) if bias is not None else -1), _p(c), c_int(ldc),
                                           c_int(M), c_int(N), c_int(K), c_int(out_code), c_int(1 if silu else 0),
                                           _p(accum), c_int(ldacc), _stream()), "gemm_skinny_packed")
    return accum if accum is not None else out


def attn_decode_mfma_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.bfloat16 and D in (32, 64, 96, 128) and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0 and H // KVH <= 16)


def attn_decode_mfma(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, context_lens: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                     window: int, max_context: int, workspace: tuple[torch.Tensor, torch.Tensor] | None = None,
                     split: bool | None = None):
    """Attention of one new token per request over its cache (the token's own key included).
    q: [S, >= H*D] rows (unit inner stride), out [S, H*D] view; block_tables int32 [S, W];
    context_lens int32 [S] (new token counted); max_context >= every context length. ``split``: None runs
    the kernel the library's rule names for this many requests (contexts split over blocks and merged, or one
    block a request and kv head); True / False name it (each kernel alone, in tests)."""
    _gpu(q, out, k_pool, v_pool, block_tables, context_lens)
    S = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "attn_decode")
    _need(attn_decode_mfma_supported(q.dtype, H, KVH, D, page), "attn_decode: unsupported head size, group or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.bfloat16 and out.shape[0] == S
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_decode: q, out [S, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if S > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if S > 1 else max(out.stride(0), H * D)
    _need(q_stride % 8 == 0 and q.data_ptr() % 16 == 0, "attn_decode: q rows must be 16-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= S
          and block_tables.stride(1) == 1, "attn_decode: block_tables must be int32 [S, W]")
    W = block_tables.shape[1]
    _need(block_tables.stride(0) == W or S == 1, "attn_decode: block_tables rows must be contiguous")
    _ints(context_lens, S, "context_lens")
    _need(0 < max_context <= W * page, "attn_decode: max_context exceeds what the block tables hold")
    from tokenmill_amd.hip.abi import bound
    chunks = -(-max_context // rule("decode_chunk"))
    part_o = part_ml = None
    if split is None:                                             # few (request, kv head) pairs: contexts split over blocks
        split = bool(bound().tm_decode_split_chunks(S, KVH, max_context))
    if split and chunks > 1:
        if workspace is None:
            workspace = (torch.empty((S, H, chunks, D), dtype=torch.float32, device=q.device),
                         torch.empty((S, H, chunks, 2), dtype=torch.float32, device=q.device))
        part_o, part_ml = workspace
        _need(part_o.numel() >= S * H * chunks * D and part_ml.numel() >= S * H * chunks * 2
              and part_o.dtype == torch.float32 and part_ml.dtype == torch.float32, "attn_decode: workspace too small")
    _need(out_stride % 4 == 0 and out.data_ptr() % 8 == 0, "attn_decode: out rows must be 8-byte aligned")
    _check(library().tm_attn_decode_mfma(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                                         _p(block_tables), c_int(W), _p(context_lens), _p(part_o), _p(part_ml),
                                         c_int(chunks), c_int(S), c_int(H), c_int(KVH), c_int(D), c_int(page),
                                         c_float(scale), c_int(window), _stream()), "attn_decode_mfma")
    return out


PREFILL_TILE = 16           # query tokens per tile of the MFMA prefill attention


def attn_prefill_mfma_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.bfloat16 and D in (32, 64, 96, 128) and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0)


def attn_prefill_mfma(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      block_tables: torch.Tensor, tiles: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                      window: int, shared: bool = False) -> torch.Tensor:
    """Attention of prompt portions over the cache. q: [T, >= H*D] rows, out [T, H*D]; tiles int32
    [n, 4] = (request index, first row, tokens (1..16), position of the first token) cover the rows
    to compute; every row of a tile belongs to one request at consecutive positions. ``shared``: the kernel
    that stages a tile's keys and values through LDS for all heads of a kv head, instead of the one whose
    wavefronts split the key blocks (each kernel alone, in tests; a step's choice is the library's)."""
    _gpu(q, out, k_pool, v_pool, block_tables, tiles)
    T = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "attn_prefill")
    _need(attn_prefill_mfma_supported(q.dtype, H, KVH, D, page), "attn_prefill: unsupported head size or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.bfloat16 and out.shape[0] == T
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_prefill: q, out [T, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if T > 1 else max(out.stride(0), H * D)
    _need(q_stride % 8 == 0 and q.data_ptr() % 16 == 0 and out_stride % 2 == 0 and out.data_ptr() % 4 == 0,
          "attn_prefill: q rows must be 16-byte aligned and out rows 4-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attn_prefill: block_tables must be contiguous int32 [S, W]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "attn_prefill: tiles must be contiguous int32 [n, 4]")
    if shared:
        _need(bool(library().tm_attn_prefill_shared_takes(c_int(H), c_int(KVH), c_int(D))) and out_stride % 4 == 0
              and out.data_ptr() % 8 == 0, "attn_prefill: the shared-keys kernel takes up to 16 query heads a kv head "
              "and out rows aligned to 8 bytes")
    entry = library().tm_attn_prefill_shared if shared else library().tm_attn_prefill_mfma
    _check(entry(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                 _p(block_tables), c_int(block_tables.shape[1]), _p(tiles),
                 c_int(tiles.shape[0]), c_int(H), c_int(KVH), c_int(D), c_int(page),
                 c_float(scale), c_int(window), _stream()), "attn_prefill_shared" if shared else "attn_prefill_mfma")
    return out


def attn_prefill_f32_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.float32 and D % 16 == 0 and 16 <= D <= 128 and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0)


def attn_prefill_f32(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, tiles: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                     window: int) -> torch.Tensor:
    """Attention of prompt portions over the cache in true 32-bit (32-bit MFMA). Operands as for
    ``attn_prefill_mfma``, all float32."""
    _gpu(q, out, k_pool, v_pool, block_tables, tiles)
    T = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.float32, "attn_prefill_f32")
    _need(attn_prefill_f32_supported(q.dtype, H, KVH, D, page), "attn_prefill_f32: unsupported head size or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.float32 and out.shape[0] == T
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_prefill_f32: q, out [T, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if T > 1 else max(out.stride(0), H * D)
    _need(q_stride % 4 == 0 and out_stride % 4 == 0 and q.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0,
          "attn_prefill_f32: q and out rows must be 16-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attn_prefill_f32: block_tables must be contiguous int32 [S, W]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "attn_prefill_f32: tiles must be contiguous int32 [n, 4]")
    _check(library().tm_attn_prefill_f32(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                                         _p(block_tables), c_int(block_tables.shape[1]), _p(tiles),
                                         c_int(tiles.shape[0]), c_int(H), c_int(KVH), c_int(D), c_int(page),
                                         c_float(scale), c_int(window), _stream()), "attn_prefill_f32")
    return out


def fused_norm_qkv_rope(resid: torch.Tensor, norm_w: torch.Tensor, eps: float, w: PackedWeight,
                        bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int, D: int, cos: torch.Tensor,
                        sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                        k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(rmsnorm(resid) * norm_w @ w^T + bias) for at most 16 tokens.
    resid float32 [M, K]; w the [(H + 2 KVH) D, K] matrix packed in strips of
    ``fused_qkv_strip_rows(H, KVH, D, K)`` rows; cos/sin float32 [max_pos, D/2]."""
    _gpu(resid, norm_w, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = resid.shape
    _need(0 < M <= rule("skinny_rows"), f"fused qkv: at most {rule('skinny_rows')} tokens, got {M}")
    _need(resid.dtype == torch.float32 and resid.is_contiguous() and resid.data_ptr() % 16 == 0, "fused qkv: resid float32 [M, K]")
    _need(D % 32 == 0, f"fused qkv: head size {D} must be a multiple of 32")
    _packed_operand(w, fused_qkv_strip_rows(H, KVH, D, K), "fused qkv")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1 and K % 8 == 0,
          "fused qkv: w must be the packed [(H+2KVH)D, K] matrix, K a multiple of 8")
    _need(tuple(norm_w.shape) == (K,) and norm_w.is_contiguous() and norm_w.data_ptr() % 16 == 0, "fused qkv: norm weight [K]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D,
          "fused qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "fused qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "fused qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "fused qkv")
        _need(page & (page - 1) == 0, "fused qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous() and bias.data_ptr() % 16 == 0,
              "fused qkv: bias [rows], 16-byte aligned")
    _need(eps > 0, "fused qkv: eps must be positive")
    _check(library().tm_fused_norm_qkv_rope(_p(resid), _p(norm_w), code(norm_w.dtype), c_float(eps), c_int(M), c_int(K),
                                            _p(w.data), _p(bias), c_int(code(bias.dtype) if bias is not None else -1),
                                            _p(q_out), c_int(H), c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions),
                                            _p(slots), _p(k_pool if slots is not None else None),
                                            _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "fused_norm_qkv_rope")
    return q_out


def fused_norm_gate_up_silu(resid: torch.Tensor, norm_w: torch.Tensor, eps: float, w: PackedWeight,
                            out: torch.Tensor) -> torch.Tensor:
    """out[M, I] <- silu(x Wg^T) * (x Wu^T), x = rmsnorm(resid) * norm_w, w = [Wg; Wu] [2I, K] packed as
    its two halves in strips of 16 rows."""
    _gpu(resid, norm_w, out)
    M, K = resid.shape
    I = out.shape[1]
    _need(0 < M <= rule("skinny_rows"), f"fused gate-up: at most {rule('skinny_rows')} tokens, got {M}")
    _need(resid.dtype == torch.float32 and resid.is_contiguous() and resid.data_ptr() % 16 == 0, "fused gate-up: resid float32 [M, K]")
    _packed_operand(w, 16, "fused gate-up")
    _need((w.n, w.k) == (2 * I, K) and w.parts == (I, I) and K % 8 == 0 and I % 4 == 0,
          "fused gate-up: w must be the packed [2I, K] matrix in two parts of I rows; K % 8 == 0, I % 4 == 0")
    _need(tuple(norm_w.shape) == (K,) and norm_w.is_contiguous() and norm_w.data_ptr() % 16 == 0, "fused gate-up: norm weight [K]")
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[0] == M, "fused gate-up: out bfloat16 [M, I]")
    _need(eps > 0, "fused gate-up: eps must be positive")
    _check(library().tm_fused_norm_gate_up_silu(_p(resid), _p(norm_w), code(norm_w.dtype), c_float(eps), c_int(M),
                                                c_int(K), _p(w.data), _p(out), c_int(I), _stream()),
           "fused_norm_gate_up_silu")
    return out


def panel_fits(M: int, K: int) -> bool:
    """Do the panel products (q|k|v + rotary + cache write, gate|up + SiLU·up for up to 64 tokens behind a
    norm that ran by itself) take M tokens of width K?"""
    return bool(library().tm_gemm_panel_fits(c_int(M), c_int(K)))


def _panel_input(x: torch.Tensor, who: str) -> int:
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1 and x.data_ptr() % 16 == 0 and M > 0
          and panel_fits(M, K), f"{who}: x bfloat16 [M, K] with x and the partial sums fitting a block's LDS")
    ldx = x.stride(0) if M > 1 else max(K, x.stride(0))
    _need(ldx % 8 == 0, f"{who}: rows of x must be 16-byte aligned")
    return ldx


def panel_qkv_rope(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int,
                   D: int, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                   k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(x @ w^T + bias) for up to 64 tokens; x bfloat16 [M, K] is the normed
    input, everything else as for ``fused_norm_qkv_rope``."""
    _gpu(x, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = x.shape
    ldx = _panel_input(x, "panel qkv")
    _need(D % 32 == 0, f"panel qkv: head size {D} must be a multiple of 32")
    _packed_operand(w, fused_qkv_strip_rows(H, KVH, D, K), "panel qkv")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1, "panel qkv: w must be the packed [(H+2KVH)D, K] matrix")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D,
          "panel qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "panel qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "panel qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "panel qkv")
        _need(page & (page - 1) == 0, "panel qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous() and bias.data_ptr() % 16 == 0,
              "panel qkv: bias [rows], 16-byte aligned")
    _check(library().tm_panel_qkv_rope(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), _p(bias),
                                       c_int(code(bias.dtype) if bias is not None else -1), _p(q_out), c_int(H),
                                       c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions), _p(slots),
                                       _p(k_pool if slots is not None else None),
                                       _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "panel_qkv_rope")
    return q_out


def stream_fits(M: int, K: int) -> bool:
    """Do the products that stream a packed matrix once for up to 64 tokens take M tokens of width K?"""
    return bool(library().tm_gemm_stream_fits(c_int(M), c_int(K)))


def _stream_input(x: torch.Tensor, w: PackedWeight, who: str) -> int:
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1 and x.data_ptr() % 16 == 0 and stream_fits(M, K) and K == w.k,
          f"{who}: x bfloat16 [M<=64, {w.k}], 16-byte aligned")
    ldx = x.stride(0) if M > 1 else max(K, x.stride(0))
    _need(ldx % 8 == 0, f"{who}: rows of x must be 16-byte aligned")
    return ldx


def stream_qkv_rope(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int,
                    D: int, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                    k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(x @ w^T + bias) for up to 64 tokens of any width; x bfloat16 [M, K] is the
    normed input, w the [(H + 2 KVH) D, K] matrix packed in strips of 16, 8 or 4 rows; the rest as for
    ``fused_norm_qkv_rope``."""
    _gpu(x, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = x.shape
    _packed_operand(w, None, "stream qkv")
    ldx = _stream_input(x, w, "stream qkv")
    _need(D % 32 == 0, f"stream qkv: head size {D} must be a multiple of 32")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1, "stream qkv: w must be the packed [(H+2KVH)D, K] matrix")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D and cos.data_ptr() % 16 == 0
          and sin.data_ptr() % 16 == 0, "stream qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "stream qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "stream qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "stream qkv")
        _need(page & (page - 1) == 0, "stream qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous(), "stream qkv: bias [rows]")
    _check(library().tm_stream_qkv_rope(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), _p(bias),
                                        c_int(code(bias.dtype) if bias is not None else -1), _p(q_out), c_int(H),
                                        c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions), _p(slots),
                                        _p(k_pool if slots is not None else None),
                                        _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "stream_qkv_rope")
    return q_out


def stream_gate_up_silu(x: torch.Tensor, w: PackedWeight, out: torch.Tensor) -> torch.Tensor:
    """out[M, I] <- silu(x Wg^T) * (x Wu^T) for up to 64 tokens of any width; w as for ``fused_norm_gate_up_silu``."""
    _gpu(x, out)
    M, K = x.shape
    I = out.shape[1]
    _packed_operand(w, 16, "stream gate-up")
    ldx = _stream_input(x, w, "stream gate-up")
    _need((w.n, w.k) == (2 * I, K) and w.parts == (I, I) and I % 4 == 0,
          "stream gate-up: w must be the packed [2I, K] matrix in two parts of I rows; I % 4 == 0")
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[0] == M, "stream gate-up: out bfloat16 [M, I]")
    _check(library().tm_stream_gate_up_silu(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), _p(out), c_int(I),
                                            _stream()), "stream_gate_up_silu")
    return out


def stream_linear(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, out: torch.Tensor | None,
                  accum: torch.Tensor | None = None) -> torch.Tensor:
    """out[M, N] = x @ w^T (+ bias) for up to 64 tokens of any width, out bfloat16 or float32; or with ``accum``
    (float32 [M, N]) the result, rounded to bfloat16, is added there and out stays unwritten. w: the [N, K]
    matrix packed as one part in strips of 16, 8 or 4 rows."""
    _gpu(x, bias, out, accum)
    M, K = x.shape
    _packed_operand(w, None, "stream linear")
    ldx = _stream_input(x, w, "stream linear")
    N = w.n
    _need(len(w.parts) == 1, "stream linear: the matrix is packed as one part")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "stream linear: bias must be [N]")
    if accum is not None:
        _need(out is None and accum.dtype == torch.float32 and tuple(accum.shape) == (M, N) and accum.stride(1) == 1,
              "stream linear: accum must be float32 [M, N], and excludes out")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        c, ldc, f32 = None, N, 0
    else:
        _need(out is not None and tuple(out.shape) == (M, N) and out.stride(1) == 1
              and out.dtype in (torch.bfloat16, torch.float32), "stream linear: out [M, N] bfloat16 or float32")
        ldacc = 0
        c, ldc, f32 = out, (out.stride(0) if M > 1 else max(N, out.stride(0))), 1 if out.dtype == torch.float32 else 0
    _check(library().tm_stream_linear(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), c_int(N), _p(bias),
                                      c_int(code(bias.dtype) if bias is not None else -1), _p(c), c_int(ldc), c_int(f32),
                                      _p(accum), c_int(ldacc), _stream()), "stream_linear")
    return accum if accum is not None else out


def stream_linear_split(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None) -> torch.Tensor:
    """The plain product of up to 64 rows with K split over groups of blocks: returns float32 [parts, M, N], the
    partial sums (bias in part 0) that ``add_rmsnorm_parts`` or ``sum_parts`` add up. The number of parts follows
    from the matrix's shape alone."""
    _gpu(x, bias)
    M, K = x.shape
    _packed_operand(w, None, "stream linear")
    ldx = _stream_input(x, w, "stream linear")
    N = w.n
    _need(len(w.parts) == 1, "stream linear: the matrix is packed as one part")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "stream linear: bias must be [N]")
    n_parts = library().tm_stream_linear_parts(c_int(N), c_int(K))
    parts = torch.empty((n_parts, M, N), dtype=torch.float32, device=x.device)
    _check(library().tm_stream_linear_split(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), c_int(N),
                                            _p(bias), c_int(code(bias.dtype) if bias is not None else -1), _p(parts),
                                            _stream()), "stream_linear_split")
    return parts


def sum_parts(parts: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = round(parts[0] + parts[1] + ...) in out's type; parts float32 [P, ...]."""
    _gpu(parts, out)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and out.is_contiguous()
          and tuple(parts.shape[1:]) == tuple(out.shape), "sum_parts: parts float32 [P, *out.shape]")
    _check(library().tm_sum_parts(_p(parts), c_int(parts.shape[0]), ctypes.c_size_t(out.numel()), _p(out), code(out.dtype),
                                  ctypes.c_size_t(out.numel()), _stream()), "sum_parts")
    return out


def add_rmsnorm_parts(resid: torch.Tensor, parts: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                      rows: torch.Tensor | None = None) -> torch.Tensor:
    """``add_rmsnorm`` with what is to be added given as float32 partial sums [P, T, hidden]: added in their order and
    rounded to out's type before they meet the residual."""
    _gpu(resid, parts, weight, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "add_rmsnorm: the residual stream is contiguous float32")
    _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"add_rmsnorm: out must be [{R}, {hidden}]")
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and parts.dim() == 3 and tuple(parts.shape[1:]) == (T, hidden)
          and 1 <= parts.shape[0] <= 16, "add_rmsnorm: parts must be float32 [P <= 16, T, hidden]")
    _need(tuple(weight.shape) == (hidden,) and weight.is_contiguous(), "add_rmsnorm: weight must be [hidden]")
    _need(out.dtype == torch.bfloat16 or weight.dtype == torch.float32, "add_rmsnorm: a float32 output needs float32 weights")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "add_rmsnorm: eps must be positive")
    _check(library().tm_add_rmsnorm_parts(_p(resid), _p(parts), c_int(parts.shape[0]), ctypes.c_size_t(T * hidden), _p(rows),
                                          _p(weight), code(weight.dtype), _p(out), code(out.dtype), c_int(R), c_int(hidden),
                                          c_float(eps), _stream()), "add_rmsnorm_parts")
    return out


def fused_lds_fits(M: int, K: int) -> bool:
    """Does the normed input of M tokens (4, 8 or 16 rows of K + 8 bfloat16), beside the partial sums of
    the block's 4 (K < 2048) or 8 wavefronts, fit the 160 KB of LDS a block of the norm-fused products may use?"""
    rows = 4 if M <= 4 else (8 if M <= 8 else 16)
    waves = 8 if K >= 2048 else 4
    return rows * (K + 8) * 2 + 4 * waves * 2 * 64 * 5 + 1024 <= 160 * 1024


def argmax_rows_static(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``argmax_rows`` without any allocation: the chunk candidates go to a fixed array the library holds on
    each GPU. For callers that cannot allocate; calls that may overlap on one GPU must not be made."""
    _gpu(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "argmax: logits must be contiguous float32 [R, V]")
    _ints(out, R, "out")
    lib = library()
    pairs, most = R * lib.tm_argmax_work_chunks(c_int(V)), lib.tm_argmax_rows_static_max_pairs()
    _need(pairs <= most or lib.tm_argmax_work_chunks(c_int(V)) == 1,
          f"argmax (static): {R} rows of {V} logits need {pairs} chunk candidates; the fixed array holds {most}")
    _need(logits.device.index == torch.cuda.current_device(), "argmax (static): the logits' GPU must be the current device")
    _check(lib.tm_argmax_rows_static(_p(logits), c_int(R), c_int(V), _p(out), _stream()), "argmax_rows_static")
    return out

"""A plain, slow Qwen2 forward pass: whole sequences, no cache, one function for each part.

Written from the formulas of KoduruChandrasekhar/TokenMill (each function cites the file and lines
it was read from). It shares no code with ``tokenmill_amd``: it reads ``config.json`` and
``model.safetensors`` itself and uses only elementary torch operations on the CPU.

Two precisions. ``dt=torch.float32`` computes everything in 32-bit. ``dt=torch.bfloat16`` keeps
every accumulation in 32-bit and rounds to bfloat16 at exactly the places where the engine's
bfloat16 path stores a bfloat16 tensor:

    weights, embedding rows, the output of each norm, each projection's output (bias added in
    32-bit before rounding), rotated q and k, the softmax weights before they multiply V, the
    attention output, silu(gate)*up.  The residual stream and the logits stay in 32-bit.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# ---------------------------------------------------------------------------------------------
# precision helpers
# ---------------------------------------------------------------------------------------------

def rnd(x: torch.Tensor, dt: torch.dtype) -> torch.Tensor:
    """Round a 32-bit tensor to the storage type ``dt`` and return it as 32-bit again."""
    return x if dt == torch.float32 else x.to(dt).to(torch.float32)


# The order in which the 32-bit sums of the products are taken. 0: one sum over the whole inner
# dimension (whatever order torch's routine has). k >= 1: partial sums over pieces of 16, 24, 32, 40 or
# 48 elements, added last piece first for odd k and first piece first for even k. All are correct; in
# bfloat16 a rounding falls the other way here and there, and how far such runs of the SAME model
# drift apart is the noise floor below which no bfloat16 comparison can look (the reference measures
# its 16-bit floor the same way, with two batchings of one model, which make its library take other
# kernels: reference baselines/make_golden.py:195-217). The orders k >= 1 also round the softmax
# weights before the division by their sum instead of after it (``_weighted_values``).
_SUM_ORDER = 0
_PIECES = (16, 24, 32, 40, 48)
NUM_ORDERS = 1 + 2 * len(_PIECES)


class summation_order:
    def __init__(self, order: int):
        self.order = order

    def __enter__(self):
        global _SUM_ORDER
        self.before, _SUM_ORDER = _SUM_ORDER, self.order

    def __exit__(self, *exc):
        global _SUM_ORDER
        _SUM_ORDER = self.before


def _matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a [M, K] @ b [K, N] in 32-bit, in the current summation order."""
    piece = _PIECES[((_SUM_ORDER - 1) // 2) % len(_PIECES)]
    if _SUM_ORDER == 0 or a.shape[-1] <= piece:
        return a @ b
    starts = range(0, a.shape[-1], piece)
    total = None
    for lo in (reversed(starts) if _SUM_ORDER % 2 else starts):
        part = a[..., lo:lo + piece] @ b[lo:lo + piece]
        total = part if total is None else total + part
    return total


# ---------------------------------------------------------------------------------------------
# reading a model folder
# ---------------------------------------------------------------------------------------------

def read_config(model_dir) -> dict:
    """Keys and fall-backs of reference src/infer/config.py:41-69."""
    raw = json.loads((Path(model_dir) / "config.json").read_text())
    h = raw["num_attention_heads"]
    theta = raw.get("rope_theta")
    if theta is None:
        theta = (raw.get("rope_parameters") or {}).get("rope_theta", 10000.0)
    return {
        "vocab": raw["vocab_size"],
        "hidden": raw["hidden_size"],
        "inter": raw["intermediate_size"],
        "layers": raw["num_hidden_layers"],
        "heads": h,
        "kv_heads": raw.get("num_key_value_heads", h),
        "head_dim": raw.get("head_dim") or raw["hidden_size"] // h,     # src/infer/config.py:29-31
        "theta": float(theta),
        "eps": raw.get("rms_norm_eps", 1e-6),
        "tied": raw.get("tie_word_embeddings", False),
    }


def read_weights(model_dir) -> dict[str, torch.Tensor]:
    """Every tensor of model.safetensors under its checkpoint name, as 32-bit floats."""
    out = {}
    with safe_open(str(Path(model_dir) / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name).to(torch.float32)
    return out


# ---------------------------------------------------------------------------------------------
# the parts
# ---------------------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, dt=torch.float32) -> torch.Tensor:
    """reference src/infer/model/layers.py:41-44: normalise in 32-bit with eps inside the root,
    round to the storage type, THEN multiply by the weight (and round the product)."""
    x32 = x.to(torch.float32)
    var = (x32 * x32).mean(dim=-1, keepdim=True)
    normed = rnd(x32 * torch.rsqrt(var + eps), dt)
    return rnd(rnd(weight, dt) * normed, dt)


def rope_tables(n_pos: int, dim: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """reference src/infer/model/layers.py:47-53: inv_freq_i = theta^(-2i/dim), angle = pos *
    inv_freq, tables [n_pos, dim] holding each angle twice (first half, second half), 32-bit."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
    freqs = torch.outer(torch.arange(n_pos).float(), inv_freq)
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """reference src/infer/model/layers.py:55-57: (x1, x2) -> (-x2, x1) over the two halves."""
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
               dt=torch.float32) -> torch.Tensor:
    """reference src/infer/model/layers.py:60-64: x*cos + rotate_half(x)*sin with the rows of the
    tables picked by each token's absolute position.  x: [T, heads, D].  The angles and the
    multiply-add are 32-bit; the result is rounded once."""
    c = cos[positions][:, None, :]
    s = sin[positions][:, None, :]
    return rnd(x * c + rotate_half(x) * s, dt)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
           dt=torch.float32, out_dt=None) -> torch.Tensor:
    """y = x W^T + b with W [out, in] (torch's F.linear as used at reference
    src/infer/model/layers.py:144,150,163-164 and src/infer/model/qwen2.py:51-52)."""
    y = _matmul(rnd(x, dt), rnd(weight, dt).t())
    if bias is not None:
        y = y + rnd(bias, dt)
    return rnd(y, dt if out_dt is None else out_dt)


def _weighted_values(scores: torch.Tensor, v: torch.Tensor, dt) -> torch.Tensor:
    """softmax(scores) @ v with the softmax in 32-bit and its weights rounded to the storage type before
    they multiply the values (reference src/infer/model/layers.py:81-82). In the other summation orders the
    weights are rounded BEFORE they are divided by their sum (exp(score - max), rounded, times v, over the
    32-bit sum): the order a kernel that sees the keys block by block has to take. Both round each weight
    once, to the same relative precision."""
    if _SUM_ORDER == 0:
        return _matmul(rnd(torch.softmax(scores, dim=-1), dt), v)
    e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
    return _matmul(rnd(e, dt), v) / e.sum(dim=-1, keepdim=True)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     dt=torch.float32, window: int | None = None) -> torch.Tensor:
    """One whole sequence.  q: [L, H, D], k, v: [L, KVH, D] -> [L, H, D].

    reference src/infer/model/layers.py:72-97 (the "eager" branch): query head h reads kv head
    h // (H // KVH) (repeat_interleave, :86-87); scores = q k^T * scale; query i sees keys j <= i
    (lower triangle, :76-78); softmax in 32-bit (:81); weights rounded to the storage type before
    they multiply V (:81-82).  ``window`` (not in the reference, whose model keeps every key) adds
    the lower bound j > i - window for the engine's windowed layer groups."""
    L, H, D = q.shape
    kvh = k.shape[1]
    group = H // kvh
    out = torch.empty(L, H, D, dtype=torch.float32)
    i = torch.arange(L)[:, None]
    j = torch.arange(L)[None, :]
    allowed = j <= i
    if window is not None:
        allowed = allowed & (j > i - window)
    for h in range(H):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.t()) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = _weighted_values(scores, vh, dt)
    return rnd(out, dt)


def attention_rows(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, first_pos: int, scale: float,
                   dt=torch.float32, window: int | None = None) -> torch.Tensor:
    """The same attention for the queries at positions first_pos, first_pos + 1, ... only (what a
    portion of a long prompt, or one decoded token, computes): q [n, H, D] against all of k, v
    [L, KVH, D]; query i of them sees keys j <= first_pos + i. With first_pos = 0 and n = L it is
    ``causal_attention`` (tested), whose L x L scores a context of thousands of keys cannot afford."""
    n, H, D = q.shape
    L, kvh = k.shape[0], k.shape[1]
    group = H // kvh
    out = torch.empty(n, H, D, dtype=torch.float32)
    i = first_pos + torch.arange(n)[:, None]
    j = torch.arange(L)[None, :]
    allowed = j <= i
    if window is not None:
        allowed = allowed & (j > i - window)
    for h in range(H):
        scores = (q[:, h, :] @ k[:, h // group, :].t()) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = _weighted_values(scores, v[:, h // group, :], dt)
    return rnd(out, dt)


def silu_mul(gate: torch.Tensor, up: torch.Tensor, dt=torch.float32) -> torch.Tensor:
    """reference src/infer/model/layers.py:164: silu(gate) * up, silu(z) = z * sigmoid(z);
    computed in 32-bit and rounded once."""
    return rnd(gate * torch.sigmoid(gate) * up, dt)


def attention_block(x: torch.Tensor, w: dict, prefix: str, cfg: dict, positions: torch.Tensor,
                    cos, sin, dt=torch.float32, window=None) -> torch.Tensor:
    """reference src/infer/model/layers.py:142-150: q, k, v projections WITH bias, heads viewed
    [T, heads, D], rope on q and k (not v), attention with scale D^-0.5 (:138), o projection
    without bias."""
    T = x.shape[0]
    H, KVH, D = cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    q = linear(x, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"], dt).view(T, H, D)
    k = linear(x, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"], dt).view(T, KVH, D)
    v = linear(x, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"], dt).view(T, KVH, D)
    q = apply_rope(q, cos, sin, positions, dt)
    k = apply_rope(k, cos, sin, positions, dt)
    a = causal_attention(q, k, v, D ** -0.5, dt, window)
    return linear(a.reshape(T, H * D), w[prefix + "o_proj.weight"], None, dt)


def mlp_block(x: torch.Tensor, w: dict, prefix: str, dt=torch.float32) -> torch.Tensor:
    """reference src/infer/model/layers.py:162-164: down(silu(gate(x)) * up(x)), no biases."""
    gate = linear(x, w[prefix + "gate_proj.weight"], None, dt)
    up = linear(x, w[prefix + "up_proj.weight"], None, dt)
    return linear(silu_mul(gate, up, dt), w[prefix + "down_proj.weight"], None, dt)


def decoder_layer(x: torch.Tensor, w: dict, i: int, cfg: dict, positions, cos, sin,
                  dt=torch.float32, window=None) -> torch.Tensor:
    """reference src/infer/model/qwen2.py:21-23: x + attn(norm_in(x)), then h + mlp(norm_post(h)).
    The residual stream x is 32-bit in both precisions."""
    p = f"model.layers.{i}."
    h = rms_norm(x, w[p + "input_layernorm.weight"], cfg["eps"], dt)
    x = x + attention_block(h, w, p + "self_attn.", cfg, positions, cos, sin, dt, window)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg["eps"], dt)
    return x + mlp_block(h, w, p + "mlp.", dt)


def forward_logits(w: dict, cfg: dict, ids: list[int], dt=torch.float32,
                   windows: list | None = None, offset: int = 0) -> torch.Tensor:
    """Logits [T, vocab] (32-bit) at every position of one whole sequence.

    reference src/infer/model/qwen2.py:43-52: embedding rows (no scaling), the layers in order,
    the final norm, then hidden @ W_out^T with W_out the embedding table when tied (:39-41)."""
    T = len(ids)
    positions = torch.arange(T) + offset        # offset: only for the test that distances alone count
    cos, sin = rope_tables(T + offset, cfg["head_dim"], cfg["theta"])
    x = rnd(w["model.embed_tokens.weight"], dt)[torch.tensor(ids, dtype=torch.long)]
    for i in range(cfg["layers"]):
        x = decoder_layer(x, w, i, cfg, positions, cos, sin, dt, windows[i] if windows else None)
    h = rms_norm(x, w["model.norm.weight"], cfg["eps"], dt)
    w_out = w["model.embed_tokens.weight"] if cfg["tied"] else w["lm_head.weight"]
    return linear(h, w_out, None, dt, out_dt=torch.float32)


# ---------------------------------------------------------------------------------------------
# sampling and generation
# ---------------------------------------------------------------------------------------------

_M64 = (1 << 64) - 1


def uniform_from_counter(seed: int, index: int) -> float:
    """The engine's random stream (its own design; the reference draws from torch generators,
    src/infer/sampling.py:49-54): u in [0, 1) from (request seed, index of the generated token)
    by two rounds of the splitmix64 finaliser, top 24 bits."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xBF58476D1CE4E5B9) & _M64
    for _ in range(2):
        z = (z + 0x9E3779B97F4A7C15) & _M64
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
        z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def filter_top_k_top_p(logits: torch.Tensor, top_k: int, top_p: float) -> torch.Tensor:
    """reference src/infer/sampling.py:12-25 for one row of temperature-scaled logits: keep the k
    largest (k <= 0 or k >= V: all); then, in descending order, drop a token once the probability
    mass BEFORE it exceeds p; the largest always stays.  Dropped entries become -inf."""
    V = logits.shape[0]
    sorted_logits, order = logits.sort(descending=True, stable=True)
    k = V if top_k <= 0 else min(top_k, V)
    remove = torch.arange(V) >= k
    probs = sorted_logits.masked_fill(remove, float("-inf")).softmax(dim=-1)
    before = probs.cumsum(dim=-1) - probs
    remove |= before > top_p
    remove[0] = False
    out = torch.empty_like(logits)
    out[order] = sorted_logits.masked_fill(remove, float("-inf"))
    return out


def sample_token(logits: torch.Tensor, temperature: float, top_k: int, top_p: float,
                 seed: int, index: int) -> tuple[int, float]:
    """reference src/infer/sampling.py:28-46: argmax when temperature <= 1e-5 or top_k == 1
    (src/infer/engine/sequence.py:29-31); else logits / temperature, the filters, softmax, one
    draw.  The draw is the inverse CDF in vocabulary order at ``uniform_from_counter``.
    Returns (token, distance of u from the nearest CDF edge of that token)."""
    if temperature <= 1e-5 or top_k == 1:
        return int(logits.argmax()), 1.0
    z = logits.to(torch.float32) / temperature
    if top_k > 0 or top_p < 1.0:
        z = filter_top_k_top_p(z, top_k, top_p)
    probs = torch.softmax(z.double(), dim=-1)
    cdf = probs.cumsum(dim=-1)
    u = uniform_from_counter(seed, index)
    target = u * float(cdf[-1])
    tok = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
    tok = min(tok, logits.shape[0] - 1)
    while float(probs[tok]) == 0.0 and tok > 0:
        tok -= 1
    lo = float(cdf[tok - 1]) if tok > 0 else 0.0
    return tok, min(abs(target - lo), abs(float(cdf[tok]) - target))


def generate(w: dict, cfg: dict, prompt: list[int], max_tokens: int, dt=torch.float32,
             temperature: float = 0.0, top_k: int = -1, top_p: float = 1.0, seed: int = 0,
             eos: set | None = None) -> tuple[list[int], list[float]]:
    """reference src/infer/model/qwen2.py:85-106 without its cache: every new token is found by a
    whole forward pass over prompt + output so far.  Returns the tokens and, for each, the margin
    by which it was chosen (top-2 logit gap when greedy, distance to the CDF edge otherwise)."""
    ids = list(prompt)
    out, margins = [], []
    for n in range(max_tokens):
        logits = forward_logits(w, cfg, ids, dt)[-1]
        tok, margin = sample_token(logits, temperature, top_k, top_p, seed, n)
        if temperature <= 1e-5 or top_k == 1:
            top2 = logits.topk(2).values
            margin = float(top2[0] - top2[1])
        out.append(tok)
        margins.append(margin)
        ids.append(tok)
        if eos and tok in eos:
            break
    return out, margins

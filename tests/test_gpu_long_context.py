"""The attention kernels at the context lengths that are measured and served: 2,048, 4,096 and 16,384
keys, against the plain attention of exactly the rows a step computes.

Random keys at such lengths give nearly uniform weights, which hide a wrong key among thousands. So
each case plants what shows a fault: a far key that carries the last query of a request (it must be
found across hundreds of pages), a request whose scores rise steadily with the position over its
whole length (the running maximum of a flash-style kernel keeps moving, and the prefill kernel's
deferred rescaling is exercised to the end), and NaN in every page behind a window.
"""
from __future__ import annotations

import pytest
import torch

from plain import qwen2_plain as P
from test_gpu_kernels import DEV, paged_case, v_layout

pytestmark = pytest.mark.gpu

# (query heads, kv heads, head size, page): the published shapes' head sizes and groups, few heads
SHAPES = [(7, 1, 64, 16), (14, 2, 64, 16), (5, 1, 128, 16), (8, 2, 128, 64)]
# size of the planted query and key entries: 18 * 18 / sqrt(128) = 28.6 natural units, against 16,383 other
# keys whose scores are spread about 1.6 around 0: they share less than 1e-7 of the weight
SPIKE = 18.0


def truth64_rows(case, lens, q_lens, scale, window=None):
    """The same rows evaluated in 64-bit."""
    outs = []
    for qq, k, v, n, ql in zip(case["qfull"], case["k"], case["v"], lens, q_lens):
        outs.append(P.attention_rows(qq[n - ql:].double(), k.double(), v.double(), n - ql, scale, torch.float32, window))
    return torch.cat(outs)


def assert_as_exact_as_plain_float32(got, want32, want64, what):
    """Sums of thousands of terms and scores of a few hundred units are what 32-bit arithmetic loses digits
    on (a score of 230 is known to 1.4e-5 only, and with it its weight): the plain 32-bit evaluation itself
    is up to 1e-4 from a 64-bit one on these inputs. So both are held against the 64-bit evaluation, and
    the kernel may be as far from it as 2e-5 of the largest value plus twice the plain 32-bit's own distance."""
    scale = float(want64.abs().max())
    plain_err = float((want32.double() - want64.double()).abs().max())
    err = float((got.double() - want64.double()).abs().max())
    assert err <= 2e-5 * scale + 2 * plain_err, f"{what}: {err:.3e} from the 64-bit values; the plain 32-bit is {plain_err:.3e} from them"


def truth_rows(case, lens, q_lens, scale, dt, window=None):
    """Plain attention of the last q_len queries of every request over all its keys."""
    outs = []
    for qq, k, v, n, ql in zip(case["qfull"], case["k"], case["v"], lens, q_lens):
        outs.append(P.attention_rows(qq[n - ql:].float(), k.float(), v.float(), n - ql, scale, dt, window))
    return torch.cat(outs)


def poison_behind_window(case, lens, q_lens, window, page):
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        for i in range(max(0, n - ql - window + 1) // page):
            case["kp"][case["tables"][s, i]] = float("nan")
            case["vp"][case["tables"][s, i]] = float("nan")


def bf16_tol():
    return dict(rtol=1.6e-2, atol=1.2e-2)


def tiles_for(lens, q_lens):
    tiles, row = [], 0
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        for j in range(0, ql, 16):
            tiles.append((s, row + j, min(16, ql - j), n - ql + j))
        row += ql
    return torch.tensor(tiles, dtype=torch.int32)


def check_far_key(out, case, request, far, row, H, KVH, D, atol):
    """The planted key ``far`` of ``request`` carries the query in ``row`` of ``out`` [T, H*D]."""
    v_far = case["v"][request][far].float()
    got = out[row].view(H, D)
    for h in range(H):
        torch.testing.assert_close(got[h], v_far[h // (H // KVH)], rtol=0, atol=atol)


@pytest.mark.parametrize("H,KVH,D,page", SHAPES)
@pytest.mark.parametrize("one_block", [False, True])
@pytest.mark.parametrize("window", [0, 1000])
def test_decode_attention_at_long_contexts(monkeypatch, H, KVH, D, page, one_block, window):
    from tokenmill_amd.hip import ops
    split = False if one_block else None          # False: the kernel that walks a whole context in one block
    dt = torch.bfloat16
    lens = [2048, 4096, 16384, 2047, 4097, 1, 300]
    q_lens = [1] * len(lens)
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=31, spike=None if window else (2, 5, SPIKE), ramp=1)
    if window:
        poison_behind_window(case, lens, q_lens, window, page)
    S, scale = len(lens), D ** -0.5
    wide = torch.zeros(S, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(S, H * D).to(DEV)
    out = torch.full((S, H * D), 3.0, dtype=dt, device=DEV)
    ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    kp, vp, tables = case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV)
    ops.attn_decode_mfma(wide, out, kp, vp, tables, ctx, H, KVH, D, scale, window, max(lens), split=split)
    want = truth_rows(case, lens, q_lens, scale, dt, window or None).reshape(S, H * D)
    got = out.float().cpu()
    torch.testing.assert_close(got, want, **bf16_tol())
    if not window:
        check_far_key(got, case, 2, 5, 2, H, KVH, D, 5e-2)     # key 5 of 16,384 carries request 2
    # the same requests among others, in another order: the same bits
    sub = [2, 0, 4]
    out2 = torch.empty(len(sub), H * D, dtype=dt, device=DEV)
    ops.attn_decode_mfma(wide[sub].contiguous(), out2, kp, vp, tables[sub].contiguous(), ctx[sub].contiguous(),
                         H, KVH, D, scale, window, max(lens), split=split)
    assert torch.equal(out2, out[sub])


@pytest.mark.parametrize("H,KVH,D,page,shared", [shape + (False,) for shape in SHAPES] +
                         [(7, 1, 128, 16, True), (10, 2, 128, 64, True), (9, 1, 96, 32, True), (14, 2, 64, 16, True)])
@pytest.mark.parametrize("window", [0, 1000])
def test_prefill_attention_at_long_contexts(H, KVH, D, page, shared, window):
    """Both kernels (``shared``: the one that stages keys and values through LDS for the heads of a kv head)."""
    from tokenmill_amd.hip import ops
    dt = torch.bfloat16
    lens = [2048, 4096, 16384, 2050]
    q_lens = [2048, 100, 48, 2]                   # a whole prompt, and portions that end long contexts
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=32, spike=None if window else (2, 7, SPIKE), ramp={0, 1})
    if window:
        poison_behind_window(case, lens, q_lens, window, page)
    T, scale = sum(q_lens), D ** -0.5
    wide = torch.zeros(T, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(T, H * D).to(DEV)
    out = torch.full((T, H * D), 3.0, dtype=dt, device=DEV)
    kp, vp, tables = case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV)
    ops.attn_prefill_mfma(wide, out, kp, vp, tables, tiles_for(lens, q_lens).to(DEV), H, KVH, D, scale, window,
                          shared=shared)
    want = truth_rows(case, lens, q_lens, scale, dt, window or None).reshape(T, H * D)
    got = out.float().cpu()
    torch.testing.assert_close(got, want, **bf16_tol())
    if not window:
        check_far_key(got, case, 2, 7, sum(q_lens[:3]) - 1, H, KVH, D, 5e-2)
    # the whole prompt again as portions of 1,000 + 1,048 tokens: the same bits
    out2 = torch.empty(T, H * D, dtype=dt, device=DEV)
    t2 = torch.tensor([(0, j, min(16, 1000 - j), j) for j in range(0, 1000, 16)] +
                      [(0, 1000 + j, min(16, 1048 - j), 1000 + j) for j in range(0, 1048, 16)], dtype=torch.int32)
    ops.attn_prefill_mfma(wide, out2, kp, vp, tables, t2.to(DEV), H, KVH, D, scale, window, shared=shared)
    assert torch.equal(out2[:2048], out[:2048])


@pytest.mark.parametrize("H,KVH,D,page", [(7, 1, 64, 16), (5, 1, 128, 16), (3, 1, 48, 32)])
@pytest.mark.parametrize("window", [0, 1000])
def test_float32_attention_at_long_contexts(H, KVH, D, page, window):
    """The 32-bit path's two kernels: the 32-bit MFMA kernel for portions and the generic kernel for single
    tokens, at 32-bit tolerance."""
    from tokenmill_amd.hip import ops
    dt = torch.float32
    lens = [2048, 4096, 16384, 2050]
    q_lens = [2048, 100, 48, 2]
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=33, spike=None if window else (2, 7, SPIKE), ramp={0, 1})
    if window:
        poison_behind_window(case, lens, q_lens, window, page)
    T, scale = sum(q_lens), D ** -0.5
    wide = torch.zeros(T, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(T, H * D).to(DEV)
    out = torch.full((T, H * D), 3.0, dtype=dt, device=DEV)
    kp, vp, tables = case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV)
    if ops.attn_prefill_f32_supported(dt, H, KVH, D, page):
        ops.attn_prefill_f32(wide, out, kp, vp, tables, tiles_for(lens, q_lens).to(DEV), H, KVH, D, scale, window)
        want = truth_rows(case, lens, q_lens, scale, dt, window or None).reshape(T, H * D)
        want64 = truth64_rows(case, lens, q_lens, scale, window or None).reshape(T, H * D)
        assert_as_exact_as_plain_float32(out.cpu(), want, want64, "portions")
        if not window:
            check_far_key(out.cpu(), case, 2, 7, sum(q_lens[:3]) - 1, H, KVH, D, 2e-2)
    # single tokens (and the rows of short portions) through the generic kernel
    rows = [sum(q_lens[:s + 1]) - 1 for s in range(len(lens))]          # the last query of every request
    q1 = wide[rows].contiguous()
    out1 = torch.full((len(rows), H * D), 3.0, dtype=dt, device=DEV)
    seq_of = torch.arange(len(rows), dtype=torch.int32, device=DEV)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV)
    ops.attn_paged_generic(q1, out1, kp, vp, tables, seq_of, pos, H, KVH, D, scale, window)
    want1 = truth_rows(case, lens, [1] * len(lens), scale, dt, window or None).reshape(len(rows), H * D)
    want1_64 = truth64_rows(case, lens, [1] * len(lens), scale, window or None).reshape(len(rows), H * D)
    assert_as_exact_as_plain_float32(out1.cpu(), want1, want1_64, "single tokens")

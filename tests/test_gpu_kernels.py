"""Each HIP kernel alone against a plain torch reference on the CPU, at sizes other than the tiny
models': widths and vocabularies that are no powers of two, head sizes in steps of 16, odd numbers
of heads and groups, row counts that do not fill a tile."""
from __future__ import annotations

import math

import pytest
import torch

from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTS = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=1e-5, atol=1e-5) if dt == torch.float32 else dict(rtol=1.6e-2, atol=1e-2)


@pytest.fixture(scope="module")
def ops():
    from tokenmill_amd.hip import ops as o
    from tokenmill_amd.hip.library import library
    library()
    return o


def q(x, dt):
    """values representable in dt, as float32"""
    return x.to(dt).float()


def v_layout(vp):
    """[pages, page, KVH, D] (how the tests fill it) -> the engine's V pool [pages, KVH, D, page]."""
    return vp.permute(0, 2, 3, 1).contiguous()


@pytest.mark.parametrize("dt", DTS)
def test_embed_gather(ops, dt):
    torch.manual_seed(0)
    table = q(torch.randn(307, 120), dt)
    ids = torch.randint(0, 307, (33,), dtype=torch.int32)
    out = torch.empty(33, 120, dtype=torch.float32, device=DEV)
    ops.embed_gather(table.to(dt).to(DEV), ids.to(DEV), out)
    assert torch.equal(out.cpu(), table[ids.long()])


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("hidden", [64, 120, 896, 2048, 3584, 5000, 16384, 16388])
def test_add_rmsnorm(ops, dt, hidden):
    torch.manual_seed(1)
    T, eps = 7, 1e-5
    resid, delta, w = torch.randn(T, hidden) * 3, q(torch.randn(T, hidden), dt), q(torch.rand(hidden) + 0.5, dt)
    want_resid = resid + delta
    want = P.rms_norm(want_resid, w, eps, dt)
    r = resid.to(DEV)
    out = torch.empty(T, hidden, dtype=dt, device=DEV)
    ops.add_rmsnorm(r, delta.to(dt).to(DEV), w.to(dt).to(DEV), eps, out)
    torch.testing.assert_close(r.cpu(), want_resid, rtol=0, atol=0)            # the 32-bit sum is exact
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))
    # no delta; and rows picked (the residual is then left alone)
    r2 = resid.to(DEV)
    ops.add_rmsnorm(r2, None, w.to(dt).to(DEV), eps, out)
    torch.testing.assert_close(out.float().cpu(), P.rms_norm(resid, w, eps, dt), **tol(dt))
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    out_r = torch.empty(4, hidden, dtype=dt, device=DEV)
    ops.add_rmsnorm(r2, delta.to(dt).to(DEV), w.to(dt).to(DEV), eps, out_r, rows.to(DEV))
    torch.testing.assert_close(out_r.float().cpu(), want[rows.long()], **tol(dt))
    assert torch.equal(r2.cpu(), resid)
    if dt == torch.bfloat16:                                                    # a weight stored in 32-bit stays so
        w32 = torch.rand(hidden) + 0.5
        ops.add_rmsnorm(resid.to(DEV), None, w32.to(DEV), eps, out)
        normed = q(resid * torch.rsqrt((resid * resid).mean(-1, keepdim=True) + eps), dt)
        torch.testing.assert_close(out.float().cpu(), q(w32 * normed, dt), **tol(dt))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,KVH,D,rot", [(5, 1, 16, 16), (6, 3, 48, 48), (4, 2, 128, 64), (3, 3, 80, 80)])
def test_rope_and_cache_write(ops, dt, H, KVH, D, rot):
    torch.manual_seed(2)
    T, max_pos, pages, page = 9, 700, 12, 4
    qkv = q(torch.randn(T, (H + 2 * KVH) * D), dt)
    positions = torch.tensor([0, 1, 5, 17, 300, 699, 2, 3, 4], dtype=torch.int32)   # absolute, not contiguous
    slots = torch.randperm(pages * page)[:T].to(torch.int32)
    slots[3] = -1                                                               # a padding row: not stored
    theta = 1e6
    inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.int64).float() / rot))
    fr = torch.outer(torch.arange(max_pos).float(), inv)
    cos_h, sin_h = fr.cos(), fr.sin()
    cos, sin = P.rope_tables(max_pos, rot, theta)
    qq = qkv[:, :H * D].view(T, H, D).clone()
    kk = qkv[:, H * D:(H + KVH) * D].view(T, KVH, D).clone()
    vv = qkv[:, (H + KVH) * D:].view(T, KVH, D)
    qq[..., :rot] = P.apply_rope(qq[..., :rot], cos, sin, positions.long(), dt)
    kk[..., :rot] = P.apply_rope(kk[..., :rot], cos, sin, positions.long(), dt)
    dq = qkv.to(dt).to(DEV)
    kp = torch.full((pages, page, KVH, D), 7.0, dtype=dt, device=DEV)
    vp = torch.full((pages, KVH, D, page), 7.0, dtype=dt, device=DEV)
    ops.rope_kv_write(dq, H, KVH, D, cos_h.to(DEV), sin_h.to(DEV), positions.to(DEV), slots.to(DEV), kp, vp)
    got = dq.float().cpu()
    torch.testing.assert_close(got[:, :H * D].view(T, H, D), qq, **tol(dt))
    torch.testing.assert_close(got[:, H * D:(H + KVH) * D].view(T, KVH, D), kk, **tol(dt))
    assert torch.equal(got[:, (H + KVH) * D:].view(T, KVH, D), vv)              # v is not rotated
    kflat = kp.float().cpu().view(-1, KVH, D)
    vflat = vp.float().cpu().permute(0, 3, 1, 2).reshape(-1, KVH, D)
    written = torch.zeros(pages * page, dtype=torch.bool)
    for t in range(T):
        if slots[t] >= 0:
            written[slots[t]] = True
            assert torch.equal(kflat[slots[t]], got[t, H * D:(H + KVH) * D].view(KVH, D))
            assert torch.equal(vflat[slots[t]], vv[t])
    assert (kflat[~written] == 7.0).all() and (vflat[~written] == 7.0).all()   # nothing else is touched


@pytest.mark.parametrize("dt", DTS)
def test_silu_mul(ops, dt):
    torch.manual_seed(3)
    gu = q(torch.randn(5, 2 * 203) * 4, dt)
    out = torch.empty(5, 203, dtype=dt, device=DEV)
    ops.silu_mul(gu.to(dt).to(DEV), out)
    torch.testing.assert_close(out.float().cpu(), P.silu_mul(gu[:, :203], gu[:, 203:], dt), **tol(dt))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("M,N,K", [(1, 307, 120), (7, 64, 64), (65, 130, 17), (130, 96, 300), (3, 1152, 896)])
def test_gemm_tiled(ops, dt, M, N, K):
    torch.manual_seed(4)
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * 0.1, dt), q(torch.randn(N), dt)
    want = a @ w.t() + b
    out = torch.empty(M, N, dtype=dt, device=DEV)
    ops.gemm_nt_tiled(a.to(dt).to(DEV), w.to(dt).to(DEV), b.to(dt).to(DEV), out)
    torch.testing.assert_close(out.float().cpu(), q(want, dt), **tol(dt))
    out32 = torch.empty(M, N, dtype=torch.float32, device=DEV)                  # 32-bit result, no bias
    ops.gemm_nt_tiled(a.to(dt).to(DEV), w.to(dt).to(DEV), None, out32)
    torch.testing.assert_close(out32.cpu(), a @ w.t(), rtol=1e-5, atol=2e-5)
    # a row-strided input (the q part of a qkv row) and a row's result that does not depend on the other rows
    wide = torch.zeros(M, K + 13, dtype=dt, device=DEV)
    wide[:, :K] = a.to(dt).to(DEV)
    out_s = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.gemm_nt_tiled(wide[:, :K], w.to(dt).to(DEV), None, out_s)
    assert torch.equal(out_s, out32)
    one = torch.empty(1, N, dtype=torch.float32, device=DEV)
    ops.gemm_nt_tiled(a[M - 1:].to(dt).to(DEV), w.to(dt).to(DEV), None, one)
    assert torch.equal(one[0], out32[M - 1])


@pytest.mark.parametrize("M,N,K", [(17, 896, 896), (300, 1152, 896), (2048, 9728, 896), (130, 896, 4864), (70, 308, 112),
                                   (1, 64, 32), (129, 132, 16), (40, 512, 7680), (24, 256, 18944)])
def test_gemm_f32_on_the_matrix_unit(ops, M, N, K):
    """The float32 products of prompt-sized steps (the matrix-unit kernel and the vector-unit kernel it stands in for
    where it refuses a shape), held against a 64-bit product: each may be as far from it as torch's own float32
    product on the CPU is, half as much again, plus one rounding of the largest value. Both sum K in blocks of 128;
    one chain of additions over all of K is 3 to 10 times further off at these K and fails this. Bias added,
    row-strided operands, and a row's bits do not depend on the other rows of the call or on the tile shape they
    put it in."""
    torch.manual_seed(41)
    a, w, b = torch.randn(M, K), torch.randn(N, K) * 0.1, torch.randn(N)
    want = (a.double() @ w.double().t())
    library_err = float(((a @ w.t()).double() - want).abs().max())
    bound = 1.5 * library_err + 2.0 ** -23 * float(want.abs().max())
    out = torch.empty(M, N, device=DEV)
    ops.gemm_f32_mfma(a.to(DEV), w.to(DEV), None, out)
    err = float((out.cpu().double() - want).abs().max())
    assert err <= bound, (err, bound)
    blocked = torch.empty(M, N, device=DEV)
    ops.gemm_nt_tiled(a.to(DEV), w.to(DEV), None, blocked)
    err_tiled = float((blocked.cpu().double() - want).abs().max())
    assert err_tiled <= bound, (err_tiled, bound)
    ops.gemm_f32_mfma(a.to(DEV), w.to(DEV), b.to(DEV), out)
    assert float((out.cpu().double() - (want + b.double())).abs().max()) <= bound + 2.0 ** -22
    wide = torch.zeros(M, K + 12, device=DEV)
    wide[:, :K] = a.to(DEV)
    out_w = torch.zeros(M, N + 8, device=DEV)
    ops.gemm_f32_mfma(wide[:, :K], w.to(DEV), b.to(DEV), out_w[:, :N])
    assert torch.equal(out_w[:, :N], out) and float(out_w[:, N:].abs().max()) == 0
    rows = [M - 1] if M < 40 else [0, 37, M - 1]
    few = torch.empty(len(rows), N, device=DEV)
    ops.gemm_f32_mfma(a[rows].contiguous().to(DEV), w.to(DEV), b.to(DEV), few)
    assert torch.equal(few, out[rows])
    with pytest.raises(ops.KernelArgumentError):
        ops.gemm_f32_mfma(torch.zeros(4, 18, device=DEV), torch.zeros(8, 18, device=DEV), None, torch.empty(4, 8, device=DEV))


def paged_case(dt, lens, q_lens, H, KVH, D, page, seed, spike=None, ramp=None, ramp_slope=1.0):
    """Random requests laid out in shuffled pages. Returns device operands and the CPU truth.
    spike = (request, key[, size]): one far key that carries the request's last query. ramp: a request (or
    a set of them) whose scores rise steadily with the key's position (about 5 * ramp_slope units of log2
    per 32 keys), so that the running maximum of a flash-style kernel keeps moving."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    n_pages = sum(-(-n // page) for n in lens) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    W = max(-(-n // page) for n in lens)
    tables = torch.zeros(S, W, dtype=torch.int32)
    kp = torch.randn(n_pages, page, KVH, D, generator=g).to(dt)        # stale values everywhere
    vp = torch.randn(n_pages, page, KVH, D, generator=g).to(dt)
    qs, ks, vs, seq_of, pos = [], [], [], [], []
    used = 0
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        k = torch.randn(n, KVH, D, generator=g).to(dt)
        v = torch.randn(n, KVH, D, generator=g).to(dt)
        qq = torch.randn(n, H, D, generator=g).to(dt)
        if spike and spike[0] == s:                                  # one far key that must dominate the last query
            far, size = spike[1], (spike[2] if len(spike) > 2 else 12.0)
            k[far] *= 0.0
            k[far, :, 0] = size
            qq[n - 1] *= 0.0
            qq[n - 1, :, 0] = size
        if ramp is not None and (s in ramp if isinstance(ramp, (set, tuple)) else ramp == s):
            k[:, :, 1] = (torch.arange(n, dtype=torch.float32)[:, None] * (0.15 * ramp_slope * (64 / D) ** 0.5)).to(dt)
            qq[:, :, 1] = 6.0
        for i in range(-(-n // page)):
            tables[s, i] = perm[used]
            lo, hi = i * page, min(n, (i + 1) * page)
            kp[perm[used], :hi - lo] = k[lo:hi]
            vp[perm[used], :hi - lo] = v[lo:hi]
            used += 1
        qs.append(qq)
        ks.append(k)
        vs.append(v)
        seq_of += [s] * ql
        pos += list(range(n - ql, n))
    q_rows = torch.cat([qq[n - ql:] for qq, n, ql in zip(qs, lens, q_lens)])   # [T, H, D]
    return dict(q=q_rows, k=ks, v=vs, qfull=qs, tables=tables, kp=kp, vp=vp,
                seq_of=torch.tensor(seq_of, dtype=torch.int32), pos=torch.tensor(pos, dtype=torch.int32))


def paged_truth(case, lens, q_lens, scale, dt, window=None):
    outs = []
    for qq, k, v, n, ql in zip(case["qfull"], case["k"], case["v"], lens, q_lens):
        full = P.causal_attention(qq.float(), k.float(), v.float(), scale, dt, window)
        outs.append(full[n - ql:])
    return torch.cat(outs)


@pytest.mark.parametrize("M,N,K", [(1, 307, 120), (8, 896, 4864), (16, 1153, 896), (5, 6, 4), (3, 9728, 896)])
def test_gemv_f32(ops, M, N, K):
    """The 32-bit matrix-vector kernel of decode steps: against a 64-bit product, with and without
    bias, a strided input, and a row alone giving the same bits as among others."""
    torch.manual_seed(13)
    a, w, b = torch.randn(M, K), torch.randn(N, K) * 0.1, torch.randn(N)
    want = (a.double() @ w.double().t()).float()
    da, dw, db = a.to(DEV), w.to(DEV), b.to(DEV)
    out = torch.full((M, N), 7.0, device=DEV)
    ops.gemv_f32(da, dw, db, out)
    torch.testing.assert_close(out.cpu(), want + b, rtol=1e-5, atol=1e-5 * K ** 0.5)
    ops.gemv_f32(da, dw, None, out)
    torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=1e-5 * K ** 0.5)
    one = torch.empty(1, N, device=DEV)
    ops.gemv_f32(da[M - 1:], dw, None, one)
    assert torch.equal(one[0], out[M - 1])
    wide = torch.zeros(M, K + 12, device=DEV)
    wide[:, :K] = da
    out_s = torch.empty(M, N, device=DEV)
    ops.gemv_f32(wide[:, :K], dw, None, out_s)
    assert torch.equal(out_s, out)
    assert not ops.gemv_f32_ok(torch.zeros(17, K, device=DEV), dw, None, torch.zeros(17, N, device=DEV))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,KVH,D,page", [(4, 2, 16, 16), (6, 1, 32, 8), (14, 2, 64, 16), (5, 5, 48, 4), (3, 1, 128, 16),
                                           (8, 2, 80, 16)])
def test_paged_attention_generic(ops, dt, H, KVH, D, page):
    lens = [1, 37, 130, 64, 5, 200]
    q_lens = [1, 37, 2, 1, 3, 1]                 # whole prompts, portions that start mid-page, single tokens
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=5, spike=(5, 3))
    scale = D ** -0.5
    T = case["q"].shape[0]
    out = torch.empty(T, H * D, dtype=dt, device=DEV)
    # q sits in the first H*D columns of a wider row, as in a fused qkv product
    wide = torch.zeros(T, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(T, H * D).to(DEV)
    ops.attn_paged_generic(wide, out, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV),
                           case["seq_of"].to(DEV), case["pos"].to(DEV), H, KVH, D, scale, 0)
    want = paged_truth(case, lens, q_lens, scale, dt).reshape(T, H * D)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))
    # the spiked far key carries the last query's output: it equals that key's value almost exactly
    v_far = case["v"][5][3].float()
    got_last = out.float().cpu()[-1].view(H, D)
    for h in range(H):
        torch.testing.assert_close(got_last[h], v_far[h // (H // KVH)], rtol=0, atol=5e-2)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("window", [0, 40])
def test_paged_attention_generic_many_tokens(ops, dt, window):
    """A step with many (token, head) pairs runs one wavefront a pair, a small one lets the
    wavefronts of a block share a pair's keys: both against the plain attention, and against each
    other (the same rows computed in a large and in a small call differ by rounding only)."""
    H, KVH, D, page = 4, 2, 32, 16
    lens, q_lens = [300, 210], [300, 210]
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=14)
    scale = D ** -0.5
    T = case["q"].shape[0]
    assert T * H >= 1024
    dev = {k: (v_layout(case[k]) if k == "vp" else case[k]).to(DEV) for k in ("kp", "vp", "tables", "seq_of", "pos")}
    q = case["q"].reshape(T, H * D).to(DEV)
    out = torch.empty(T, H * D, dtype=dt, device=DEV)
    ops.attn_paged_generic(q, out, dev["kp"], dev["vp"], dev["tables"], dev["seq_of"], dev["pos"], H, KVH, D, scale, window)
    want = paged_truth(case, lens, q_lens, scale, dt, window or None).reshape(T, H * D)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))
    few = slice(280, 300)                        # the last rows of the first request, alone
    out_few = torch.empty(20, H * D, dtype=dt, device=DEV)
    ops.attn_paged_generic(q[few], out_few, dev["kp"], dev["vp"], dev["tables"], dev["seq_of"][few], dev["pos"][few],
                           H, KVH, D, scale, window)
    torch.testing.assert_close(out_few.float().cpu(), want[few], **tol(dt))
    torch.testing.assert_close(out_few.float(), out[few].float(), **tol(dt))


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("window", [1, 7, 16, 50])
def test_paged_attention_generic_window(ops, dt, window):
    H, KVH, D, page = 6, 2, 32, 8
    lens, q_lens = [60, 9, 33], [60, 1, 5]
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=6)
    # poison every page wholly behind the window of the queries run here: it must never be read
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        first_query = n - ql
        for i in range(max(0, first_query - window + 1) // page):
            case["kp"][case["tables"][s, i]] = float("nan")
            case["vp"][case["tables"][s, i]] = float("nan")
    T = case["q"].shape[0]
    out = torch.empty(T, H * D, dtype=dt, device=DEV)
    ops.attn_paged_generic(case["q"].reshape(T, H * D).to(DEV), out, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV),
                           case["tables"].to(DEV), case["seq_of"].to(DEV), case["pos"].to(DEV), H, KVH, D,
                           D ** -0.5, window)
    want = paged_truth(case, lens, q_lens, D ** -0.5, dt, window).reshape(T, H * D)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))


def test_kernels_refuse_what_they_cannot_run(ops):
    from tokenmill_amd.hip.ops import KernelArgumentError
    x = torch.zeros(4, 8, device=DEV)
    with pytest.raises(KernelArgumentError):
        ops.silu_mul(x.cpu(), torch.zeros(4, 4))                      # no CPU path
    with pytest.raises(KernelArgumentError):
        ops.silu_mul(x.double(), torch.zeros(4, 4, device=DEV).double())
    with pytest.raises(KernelArgumentError):
        ops.attn_paged_generic(torch.zeros(1, 6, device=DEV), torch.zeros(1, 6, device=DEV),
                               torch.zeros(1, 4, 1, 6, device=DEV), torch.zeros(1, 4, 1, 6, device=DEV),
                               torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                               torch.zeros(1, dtype=torch.int32, device=DEV),
                               torch.zeros(1, dtype=torch.int32, device=DEV), 1, 1, 6, 1.0)   # head size 6
    with pytest.raises(KernelArgumentError):
        ops.gemm_nt_tiled(torch.zeros(2, 8, device=DEV), torch.zeros(4, 9, device=DEV), None,
                          torch.zeros(2, 4, device=DEV))


# ----------------------------------------------------------------------------------------------- sampling

def test_argmax_rows(ops):
    torch.manual_seed(7)
    logits = torch.randn(9, 151936 // 8 + 5)
    logits[3, 100] = logits[3, 7000] = 50.0                           # a tie: the first maximum wins
    out = torch.empty(9, dtype=torch.int32, device=DEV)
    ops.argmax_rows(logits.to(DEV), out)
    assert out.cpu().tolist() == logits.argmax(-1).tolist() and out[3].item() == 100
    two = torch.tensor([[0.1, 3.0, 2.0], [5.0, -1.0, 4.9]])          # reference tests/test_sampling.py:11-13
    out = torch.empty(2, dtype=torch.int32, device=DEV)
    ops.argmax_rows(two.to(DEV), out)
    assert out.cpu().tolist() == [1, 0]


def sample(ops, logits, temps, ks, ps, us):
    R = logits.shape[0]
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    f = lambda x: torch.tensor(x, dtype=torch.float32, device=DEV)    # noqa: E731
    ops.sample_rows(logits.to(DEV), f(temps), torch.tensor(ks, dtype=torch.int32, device=DEV), f(ps), f(us), out)
    return out.cpu().tolist()


def test_sample_rows_against_the_plain_sampler(ops):
    torch.manual_seed(8)
    V = 1000
    logits = torch.randn(64, V) * 2
    cases = [(0.8, -1, 1.0), (1.0, 20, 1.0), (0.7, -1, 0.9), (1.3, 50, 0.8), (0.0, -1, 1.0), (0.9, 1, 1.0),
             (1.0, 5000, 0.999), (0.5, 3, 0.5)]
    temps, ks, ps, us, want, margins = [], [], [], [], [], []
    for r in range(64):
        t, k, p = cases[r % len(cases)]
        temps.append(t), ks.append(k), ps.append(p)
        u = P.uniform_from_counter(99, r)
        us.append(u)
        # the plain sampler draws from (seed, index); index r here
        tok, margin = P.sample_token(logits[r], t, k, p, 99, r)
        want.append(tok), margins.append(margin)
    got = sample(ops, logits, temps, ks, ps, us)
    for r in range(64):
        assert got[r] == want[r] or margins[r] < 1e-4, f"row {r} {cases[r % len(cases)]}: {got[r]} != {want[r]}"
    assert sum(g == w for g, w in zip(got, want)) >= 62


def test_sample_rows_wide_vocabulary_against_the_plain_sampler(ops):
    """A vocabulary of several chunks (no power of two, a short last chunk): every stage of the
    sampler works over (row, chunk) blocks. Rows with and without each filter in one call, and the same
    rows alone or with the filters' launches left out give the same tokens."""
    torch.manual_seed(18)
    V = 4 * 4096 + 3731
    R = 40
    logits = torch.randn(R, V) * 2.5
    logits[5, 17000:17040] += 6.0                                     # a nucleus inside the last chunks
    cases = [(0.8, -1, 1.0), (1.0, 20, 1.0), (0.7, -1, 0.9), (1.3, 50, 0.8), (0.0, -1, 1.0), (0.9, 1, 1.0),
             (1.0, V + 5, 0.999), (0.5, 3, 0.5), (1.5, 3000, 1.0), (2.0, -1, 0.97)]
    temps, ks, ps, us, want, margins = [], [], [], [], [], []
    for r in range(R):
        t, k, p = cases[r % len(cases)]
        temps.append(t), ks.append(k), ps.append(p)
        us.append(P.uniform_from_counter(7, r))
        tok, margin = P.sample_token(logits[r], t, k, p, 7, r)
        want.append(tok), margins.append(margin)
    got = sample(ops, logits, temps, ks, ps, us)
    for r in range(R):
        assert got[r] == want[r] or margins[r] < 1e-4, f"row {r} {cases[r % len(cases)]}: {got[r]} != {want[r]}"
    assert sum(g == w for g, w in zip(got, want)) >= R - 2
    # a row's token does not depend on the rows beside it
    for r in (2, 3, 7, 8, 19):
        assert sample(ops, logits[r:r + 1], temps[r:r + 1], ks[r:r + 1], ps[r:r + 1], us[r:r + 1]) == [got[r]]
    # rows that use no filter: the same with the filters' launches left out
    plain_rows = [r for r in range(R) if r % len(cases) in (0, 4, 5)]
    out = torch.empty(len(plain_rows), dtype=torch.int32, device=DEV)
    f = lambda x: torch.tensor(x, dtype=torch.float32, device=DEV)    # noqa: E731
    ops.sample_rows(logits[plain_rows].to(DEV), f([temps[r] for r in plain_rows]),
                    torch.tensor([ks[r] for r in plain_rows], dtype=torch.int32, device=DEV),
                    f([ps[r] for r in plain_rows]), f([us[r] for r in plain_rows]), out,
                    uses_top_k=False, uses_top_p=False)
    assert out.cpu().tolist() == [got[r] for r in plain_rows]


def test_sample_rows_keeps_ties_at_the_kth_value_in_vocabulary_order(ops):
    """Five entries share the k-th largest value, spread over three chunks; top_k = 4 keeps the two larger
    entries and the first two of the ties, whatever u is; with top_p on top the nucleus is cut inside them."""
    V = 3 * 4096 + 100
    row = torch.full((V,), -4.0)
    row[9000], row[300] = 3.0, 2.5
    ties = [120, 4095, 4096, 8200, 12300]
    row[ties] = 1.0
    n = 256
    draws = [(i + 0.5) / n for i in range(n)]
    got = sample(ops, row.repeat(n, 1), [1.0] * n, [4] * n, [1.0] * n, draws)
    assert set(got) == {9000, 300, 120, 4095}
    want = torch.softmax(torch.tensor([1.0, 2.5, 1.0, 3.0]), -1)      # tokens 120, 300, 4095, 9000 in vocabulary order
    for tok, w in zip((120, 300, 4095, 9000), want.tolist()):
        assert abs(got.count(tok) / n - w) < 1.5 / n + 1e-3
    got = sample(ops, row.repeat(n, 1), [1.0] * n, [6] * n, [1.0] * n, draws)
    assert set(got) == {9000, 300, 120, 4095, 4096, 8200}
    got = sample(ops, row.repeat(n, 1), [1.0] * n, [4] * n, [0.6] * n, draws)    # 3.0 and 2.5 hold 0.84 of the mass
    assert set(got) == {9000, 300}


def kept_by_kernel(ops, row, t, k, p, n=8192):
    """The tokens the sampler can return for one row: a fine grid of u over the kept distribution."""
    us = [(i + 0.5) / n for i in range(n)]
    return sorted(set(sample(ops, row.repeat(n, 1), [t] * n, [k] * n, [p] * n, us)))


def test_sample_rows_cuts_the_nucleus_inside_ties_in_vocabulary_order(ops):
    """Logits on a grid of 0.5, so that hundreds of entries share each value. The nucleus ends inside a run
    of equal entries: they stay in vocabulary order while the mass before them is at most p (reference
    src/infer/sampling.py:20-23 in sorted order; the plain implementation's stable sort makes that vocabulary
    order), not all of them; with p near 0 exactly one of the entries that share the maximum stays; with top-k
    cutting inside a run as well, the nucleus is taken over what top-k kept. -0.0 and +0.0 are one value."""
    torch.manual_seed(5)
    V = 4097
    row = (torch.randn(V) * 2).round() / 2
    for t, k, p in ((0.3, 2048, 0.5), (1.7, -1, 0.5), (0.8, -1, 0.5), (1.7, 5, 1e-6), (5.0, -1, 1e-6), (1.0, 7, 1.0),
                    (1.0, 40, 0.95), (0.6, 12, 0.7), (2.5, 300, 0.33)):
        want = torch.isfinite(P.filter_top_k_top_p(row / t, k, p)).nonzero().flatten().tolist()
        got = kept_by_kernel(ops, row, t, k, p)
        # a grid of 8,192 draws reaches every kept token whose share is above 1/8192: compare where that holds
        probs = torch.softmax(P.filter_top_k_top_p(row / t, k, p).double(), -1)
        reachable = [i for i in want if probs[i] > 2.0 / 8192]
        assert set(got) <= set(want), f"t {t} k {k} p {p}: the kernel keeps {sorted(set(got) - set(want))[:8]} beyond the plain filter"
        assert set(reachable) <= set(got), f"t {t} k {k} p {p}: the kernel drops {sorted(set(reachable) - set(got))[:8]}"
    # the ties at the maximum with p near 0: the first of them in vocabulary order, whatever u is
    top = (row == row.max()).nonzero().flatten().tolist()
    assert len(top) > 1 and kept_by_kernel(ops, row, 1.7, -1, 1e-6, n=64) == [top[0]]
    # signed zeros: a row of +0.0 and -0.0 is a row of equal entries
    zeros = torch.zeros(100)
    zeros[::3] = -0.0
    assert kept_by_kernel(ops, zeros, 1.0, 7, 1.0, n=256) == list(range(7))
    got = kept_by_kernel(ops, zeros, 1.0, -1, 0.305, n=1024)                  # mass before entry j is j / 100
    assert got == list(range(len(got))) and len(got) in (31, 32)              # (j = 30 sits on the edge up to rounding)
    out = torch.empty(1, dtype=torch.int32, device=DEV)
    ops.argmax_rows(zeros[None].to(DEV), out)
    assert out.item() == 0                                                    # the first of equal maxima, as torch.argmax


def test_sample_rows_filters_on_the_references_vectors(ops):
    """reference tests/test_sampling.py:16-31: what top-k and top-p keep."""
    draws = [i / 64 + 1 / 128 for i in range(64)]
    row = torch.tensor([1.0, 4.0, 3.0, 2.0]).repeat(64, 1)
    got = set(sample(ops, row, [1.0] * 64, [2] * 64, [1.0] * 64, draws))
    assert got == {1, 2}
    row = torch.tensor([0.5, 0.3, 0.15, 0.05]).log().repeat(64, 1)
    assert set(sample(ops, row, [1.0] * 64, [-1] * 64, [0.7] * 64, draws)) == {0, 1}
    row = torch.tensor([10.0, 0.0]).repeat(64, 1)
    assert set(sample(ops, row, [1.0] * 64, [-1] * 64, [1e-6] * 64, draws)) == {0}
    # temperature row = softmax(logits / t): frequencies over a fine grid of u
    n = 4096
    row = torch.tensor([2.0, 1.0, 0.0]).repeat(n, 1)
    grid = [(i + 0.5) / n for i in range(n)]
    for t in (1.0, 0.3):
        got = sample(ops, row, [t] * n, [-1] * n, [1.0] * n, grid)
        want = torch.softmax(torch.tensor([2.0, 1.0, 0.0]) / t, -1)
        for tok in range(3):
            assert abs(got.count(tok) / n - want[tok].item()) < 2e-3


# ----------------------------------------------------------------------------------------------- MFMA kernels

@pytest.mark.parametrize("M,N,K", [(1, 307, 120), (8, 1152, 896), (8, 896, 4864), (17, 1000, 64), (64, 896, 896),
                                   (33, 16 * 2048 + 5, 72), (48, 130, 2056), (5, 16, 8)])
def test_gemm_skinny(ops, M, N, K):
    torch.manual_seed(9)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * 0.1, dt), q(torch.randn(N), dt)
    want = a @ w.t()
    da, dw = a.to(dt).to(DEV), w.to(dt).to(DEV)
    out = torch.empty(M, N, dtype=dt, device=DEV)
    ops.gemm_skinny(da, dw, b.to(dt).to(DEV), out)
    torch.testing.assert_close(out.float().cpu(), q(want + b, dt), **tol(dt))
    out32 = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.gemm_skinny(da, dw, b.to(DEV), out32)                                   # a bias stored in 32-bit
    torch.testing.assert_close(out32.cpu(), want + b, rtol=1e-4, atol=1e-4 * K ** 0.5)
    ops.gemm_skinny(da, dw, None, out32)
    torch.testing.assert_close(out32.cpu(), want, rtol=1e-4, atol=1e-4 * K ** 0.5)
    # a row's result does not depend on the other rows of the call, nor on a strided input
    one = torch.empty(1, N, dtype=torch.float32, device=DEV)
    ops.gemm_skinny(da[M - 1:], dw, None, one)
    assert torch.equal(one[0], out32[M - 1])
    wide = torch.zeros(M, K + 24, dtype=dt, device=DEV)
    wide[:, :K] = da
    out_s = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops.gemm_skinny(wide[:, :K], dw, None, out_s)
    assert torch.equal(out_s, out32)


@pytest.mark.parametrize("rows", [4, 8, 16])
@pytest.mark.parametrize("N,K", [(896, 4864), (50, 72), (1153, 40), (16, 32)])
def test_pack_weight_layout(ops, rows, N, K):
    """The strip order, element by element from its definition; rows and k that do not exist are zeros."""
    torch.manual_seed(18)
    w = torch.randn(N, K).to(torch.bfloat16)
    pw = ops.pack_weight(w.to(DEV), rows)
    ks, strips = -(-K // 32), -(-N // rows)
    data = pw.data.cpu().view(strips, ks, 4, rows, 8)
    assert (pw.n, pw.k, pw.rows, pw.parts) == (N, K, rows, (N,))
    idx = torch.randint(0, strips * ks * 4 * rows * 8, (2000,))
    for flat in idx.tolist() + [0, data.numel() - 1]:
        i = flat % 8
        r = (flat // 8) % rows
        g = (flat // (8 * rows)) % 4
        k_step = (flat // (32 * rows)) % ks
        s_ = flat // (32 * rows * ks)
        n, k = s_ * rows + r, 32 * k_step + 8 * g + i
        want = w[n, k] if n < N and k < K else torch.tensor(0.0, dtype=torch.bfloat16)
        assert data.reshape(-1)[flat] == want, (flat, n, k)
    two = ops.pack_weight(torch.cat([w, w]).to(DEV), rows, [N, N])     # two parts: each starts a strip of its own
    assert torch.equal(two.data.cpu().view(2, -1)[0], pw.data.cpu()) and torch.equal(two.data.cpu().view(2, -1)[1], pw.data.cpu())


@pytest.mark.parametrize("M,N,K", [(8, 896, 4864), (16, 896, 896), (1, 307, 120), (8, 1152, 896), (5, 16 * 2048 + 5, 72),
                                   (3, 3584, 2056), (16, 50, 4864)])
def test_gemm_skinny_over_a_packed_matrix_gives_the_same_bits(ops, M, N, K):
    torch.manual_seed(19)
    dt = torch.bfloat16
    a = torch.randn(M, K).to(dt).to(DEV)
    w = (torch.randn(N, K) * 0.1).to(dt).to(DEV)
    b = torch.randn(N).to(dt).to(DEV)
    for rows in (4, 8, 16):
        pw = ops.pack_weight(w, rows)
        for out_dt in (dt, torch.float32):
            plain, packed = torch.empty(M, N, dtype=out_dt, device=DEV), torch.full((M, N), 7.0, dtype=out_dt, device=DEV)
            ops.gemm_skinny(a, w, b, plain)
            ops.gemm_skinny(a, pw, b, packed)
            if rows == ops.skinny_strip_rows(N, K):                      # the same strips, the same split of K: the same bits
                assert torch.equal(plain, packed)
            else:
                torch.testing.assert_close(packed.float(), plain.float(), **tol(dt))
        resid = torch.randn(M, N, device=DEV) * 5
        acc_plain, acc_packed = resid.clone(), resid.clone()
        ops.gemm_skinny(a, w, b, None, accum=acc_plain)
        ops.gemm_skinny(a, pw, b, None, accum=acc_packed)
        if rows == ops.skinny_strip_rows(N, K):
            assert torch.equal(acc_plain, acc_packed)
        else:
            torch.testing.assert_close(acc_packed, acc_plain, rtol=1.6e-2, atol=1e-2 + 1e-5)
    if N % 2 == 0:                                                       # the stacked [gate; up] matrix
        I = N // 2
        pw = ops.pack_weight(w, 16, [I, I])
        plain, packed = torch.empty(M, I, dtype=dt, device=DEV), torch.full((M, I), 7.0, dtype=dt, device=DEV)
        ops.gemm_skinny(a, w, None, plain, silu=True)
        ops.gemm_skinny(a, pw, None, packed, silu=True)
        assert torch.equal(plain, packed)
    with pytest.raises(ops.KernelArgumentError):                         # more rows than the packed kernels take
        ops.gemm_skinny(torch.zeros(17, K, dtype=dt, device=DEV), ops.pack_weight(w, 16), None,
                        torch.empty(17, N, dtype=dt, device=DEV))


@pytest.mark.parametrize("tune,after", [(0, 3), (6, 1), (6, 3)])
@pytest.mark.parametrize("M,N,K", [(300, 1152, 896), (17, 896, 4864), (2048, 200, 120), (1, 5000, 64), (70, 307, 72)])
def test_gemm_library(ops, M, N, K, tune, after):
    """The library product behind the cached plan: with and without bias, bfloat16 and float32 out,
    a strided input, the same bits on the second call (the kept plan); untimed, with the candidates
    timed at the first call, and timed when the shape comes the third time (every call before and
    after gives the product). A shape the library refuses comes back as False and `linear` takes
    another kernel. Plans of timed callers live apart from the plans of the others: a call without
    timing gives the same bits before and after a timed caller has had its algorithm chosen."""
    torch.manual_seed(12)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * 0.1, dt), q(torch.randn(N), dt)
    want = a @ w.t()
    da, dw, db = a.to(dt).to(DEV), w.to(dt).to(DEV), b.to(dt).to(DEV)
    untimed = torch.full((M, N), 7.0, dtype=dt, device=DEV)
    taken = ops.gemm_library(da, dw, db, untimed)
    with ops.tuning(tune, after):
        out = torch.full((M, N), 7.0, dtype=dt, device=DEV)
        if ops.gemm_library(da, dw, db, out):
            torch.testing.assert_close(out.float().cpu(), q(want + b, dt), **tol(dt))
            again = torch.empty_like(out)
            assert ops.gemm_library(da, dw, db, again) and torch.equal(again, out)
            for _ in range(after):                          # past the call that times the candidates
                later = torch.full((M, N), 7.0, dtype=dt, device=DEV)
                assert ops.gemm_library(da, dw, db, later)
                torch.testing.assert_close(later.float().cpu(), q(want + b, dt), **tol(dt))
        out32 = torch.full((M, N), 7.0, dtype=torch.float32, device=DEV)
        if ops.gemm_library(da, dw, None, out32):
            torch.testing.assert_close(out32.cpu(), want, rtol=1e-4, atol=1e-4 * K ** 0.5)
        wide = torch.zeros(M, K + 24, dtype=dt, device=DEV)
        wide[:, :K] = da
        out_s = torch.full((M, N), 7.0, dtype=dt, device=DEV)
        if ops.gemm_library(wide[:, :K], dw, None, out_s):
            torch.testing.assert_close(out_s.float().cpu(), q(want, dt), **tol(dt))
        # whatever the library takes, the rule above it gives the product
        out_l = torch.full((M, N), 7.0, dtype=dt, device=DEV)
        ops.linear(ops.linear_desc(dw, None, db), da, out_l)
        torch.testing.assert_close(out_l.float().cpu(), q(want + b, dt), **tol(dt))
    if taken:                                               # ... and nothing of the timing reached the untimed plan
        again = torch.empty_like(untimed)
        assert ops.gemm_library(da, dw, db, again) and torch.equal(again, untimed)


@pytest.mark.parametrize("M,N,K", [(64, 896, 4864), (333, 1152, 896)])
def test_gemm_library_tries_every_algorithm(ops, M, N, K):
    """With `every`, a shape timed at its first call also runs each algorithm the library holds for the
    operand types once and times the fastest few; whichever is kept, the product is the product:
    with a bias, with float32 out, at a shape whose matrix comes from memory (timed with flushed
    caches) and at one whose rows dominate."""
    torch.manual_seed(14)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * 0.1, dt), q(torch.randn(N), dt)
    want = a @ w.t()
    da, dw, db = a.to(dt).to(DEV), w.to(dt).to(DEV), b.to(dt).to(DEV)
    with ops.tuning(8, 1, every=True):
        for bias, add in ((db, b), (None, 0.0)):
            out = torch.full((M, N), 7.0, dtype=dt, device=DEV)
            assert ops.gemm_library(da, dw, bias, out)
            torch.testing.assert_close(out.float().cpu(), q(want + add, dt), **tol(dt))
            again = torch.empty_like(out)
            assert ops.gemm_library(da, dw, bias, again) and torch.equal(again, out)
        out32 = torch.full((M, N), 7.0, dtype=torch.float32, device=DEV)
        assert ops.gemm_library(da, dw, None, out32)
        torch.testing.assert_close(out32.cpu(), want, rtol=1e-4, atol=1e-4 * K ** 0.5)
    with pytest.raises(ops.KernelArgumentError):
        with ops.tuning(0, 1, every=True):
            pass


def test_gemm_library_takes_a_candidate_whose_workspace_fits(ops):
    """At 8,192 rows of the gate|up product the library's first choice asks for more workspace than it is
    given: the plan takes the first candidate that fits instead of refusing the shape (a refused shape
    runs 64 rows at a time through the skinny kernel, ten times slower)."""
    torch.manual_seed(13)
    dt = torch.bfloat16
    M, N, K = 8192, 9728, 896
    da = torch.randn(M, K, device=DEV).to(dt)
    dw = (torch.randn(N, K, device=DEV) * 0.1).to(dt)
    out = torch.full((M, N), 7.0, dtype=dt, device=DEV)
    assert ops.gemm_library(da, dw, None, out)
    rows = torch.arange(0, M, 257)
    want = da[rows].float().cpu() @ dw.float().cpu().t()
    torch.testing.assert_close(out[rows].float().cpu(), q(want, dt), **tol(dt))


@pytest.mark.parametrize("M,I,K", [(1, 128, 64), (8, 4864, 896), (40, 200, 120), (64, 320, 192)])
def test_gemm_skinny_with_silu_epilogue(ops, M, I, K):
    torch.manual_seed(10)
    dt = torch.bfloat16
    a, w = q(torch.randn(M, K), dt), q(torch.randn(2 * I, K) * 0.2, dt)
    gu = q(a @ w.t(), dt)
    want = P.silu_mul(gu[:, :I], gu[:, I:], dt)
    out = torch.empty(M, I, dtype=dt, device=DEV)
    ops.gemm_skinny(a.to(dt).to(DEV), w.to(dt).to(DEV), None, out, silu=True)
    torch.testing.assert_close(out.float().cpu(), want, rtol=2e-2, atol=2e-2)
    assert ((out.float().cpu() - want).abs() > 1e-2).float().mean() < 0.01      # a rounding flip of gate or up now and then


@pytest.mark.parametrize("H,KVH,D,page", [(14, 2, 64, 16), (6, 1, 32, 16), (5, 5, 128, 32), (16, 1, 64, 16),
                                           (8, 2, 96, 16), (4, 2, 64, 64)])
@pytest.mark.parametrize("window", [0, 40])
@pytest.mark.parametrize("one_block", [False, True])
def test_paged_attention_decode_mfma(ops, monkeypatch, H, KVH, D, page, window, one_block):
    """one_block: the kernel for many requests (one block walks a request's whole context), which the
    dispatcher would only take from 192 (request, kv head) pairs on."""
    split = False if one_block else None
    dt = torch.bfloat16
    lens = [1, 2, 16, 17, 255, 256, 257, 700, 64, 1000]
    q_lens = [1] * len(lens)
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=11, spike=(7, 2) if not window else None)
    if window:                                   # pages wholly behind the window must never be read
        for s, n in enumerate(lens):
            for i in range(max(0, n - 1 - window + 1) // page):
                case["kp"][case["tables"][s, i]] = float("nan")
                case["vp"][case["tables"][s, i]] = float("nan")
    S = len(lens)
    scale = D ** -0.5
    wide = torch.zeros(S, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(S, H * D).to(DEV)
    out = torch.full((S, H * D), 3.0, dtype=dt, device=DEV)
    ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    ops.attn_decode_mfma(wide, out, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV), ctx,
                         H, KVH, D, scale, window, max(lens), split=split)
    want = paged_truth(case, lens, q_lens, scale, dt, window or None).reshape(S, H * D)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))
    if not window:                               # the spiked far key (position 2 of 700) carries its request's output
        v_far = case["v"][7][2].float()
        got = out.float().cpu()[7].view(H, D)
        for h in range(H):
            torch.testing.assert_close(got[h], v_far[h // (H // KVH)], rtol=0, atol=5e-2)
    # the same requests in another batch composition give the same bits
    sub = [7, 3]
    out2 = torch.empty(2, H * D, dtype=dt, device=DEV)
    ops.attn_decode_mfma(wide[sub].contiguous(), out2, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV),
                         case["tables"][sub].contiguous().to(DEV), ctx[sub].contiguous(), H, KVH, D, scale, window,
                         max(lens), split=split)
    assert torch.equal(out2, out[sub])
    # block tables wider than any context (the shape a captured graph has), scratch memory full of NaN
    # beyond what the step writes: up to 64 chunks the merge reads ahead of the context length, beyond
    # that another merge kernel runs
    for max_context in () if one_block else (4096, 20000):
        width = -(-max_context // page)
        tables = torch.zeros(S, width, dtype=torch.int32)
        tables[:, :case["tables"].shape[1]] = case["tables"]
        chunks = -(-max_context // ops.rule("decode_chunk"))
        ws = (torch.full((S, H, chunks, D), float("nan"), device=DEV), torch.full((S, H, chunks, 2), float("nan"), device=DEV))
        out3 = torch.full((S, H * D), 3.0, dtype=dt, device=DEV)
        ops.attn_decode_mfma(wide, out3, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), tables.to(DEV), ctx,
                             H, KVH, D, scale, window, max_context, workspace=ws)
        torch.testing.assert_close(out3.float().cpu(), want, **tol(dt))
        if not window:
            assert torch.equal(out3, out)


def tiles_for(lens, q_lens):
    tiles, row = [], 0
    for s, (n, ql) in enumerate(zip(lens, q_lens)):
        for j in range(0, ql, 16):
            tiles.append((s, row + j, min(16, ql - j), n - ql + j))
        row += ql
    return torch.tensor(tiles, dtype=torch.int32)


# the two kernels: wavefronts that split a tile's key blocks (any group), and a tile's keys and values staged through
# LDS for all heads of a kv head (groups up to 16: 2, 4 or 8 wavefronts a block, the last with a copy loop whose
# trip count does not divide at head size 96)
@pytest.mark.parametrize("H,KVH,D,page,shared", [
    (14, 2, 64, 16, False), (6, 1, 32, 16, False), (5, 5, 128, 32, False), (20, 1, 64, 16, False), (8, 2, 96, 16, False),
    (4, 2, 64, 64, False),
    (14, 2, 128, 16, True), (10, 2, 128, 32, True), (24, 2, 96, 16, True), (12, 1, 128, 64, True), (14, 2, 64, 16, True),
    (6, 1, 32, 16, True), (4, 2, 64, 64, True), (3, 3, 96, 32, True)])
@pytest.mark.parametrize("window", [0, 40])
def test_paged_attention_prefill_mfma(ops, H, KVH, D, page, shared, window):
    dt = torch.bfloat16
    lens = [2, 37, 130, 64, 5, 300, 33, 200]
    q_lens = [2, 37, 2, 64, 3, 45, 17, 200]      # whole prompts and portions that start and end mid-page
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=12, spike=(5, 3) if not window else None, ramp=7)
    if window:
        for s, (n, ql) in enumerate(zip(lens, q_lens)):
            for i in range(max(0, n - ql - window + 1) // page):
                case["kp"][case["tables"][s, i]] = float("nan")
                case["vp"][case["tables"][s, i]] = float("nan")
    T = case["q"].shape[0]
    scale = D ** -0.5
    wide = torch.zeros(T, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(T, H * D).to(DEV)
    out = torch.full((T, H * D), 3.0, dtype=dt, device=DEV)
    ops.attn_prefill_mfma(wide, out, case["kp"].to(DEV), v_layout(case["vp"]).to(DEV), case["tables"].to(DEV),
                          tiles_for(lens, q_lens).to(DEV), H, KVH, D, scale, window, shared=shared)
    want = paged_truth(case, lens, q_lens, scale, dt, window or None).reshape(T, H * D)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dt))
    if not window:                               # the last query of request 5 is carried by its far key 3
        row = sum(q_lens[:6]) - 1
        v_far = case["v"][5][3].float()
        got = out.float().cpu()[row].view(H, D)
        for h in range(H):
            torch.testing.assert_close(got[h], v_far[h // (H // KVH)], rtol=0, atol=5e-2)
    # cut differently (one request alone, in two portions): the same bits
    s = 7
    k_dev, v_dev = case["kp"].to(DEV), v_layout(case["vp"]).to(DEV)
    first = sum(q_lens[:s])
    out2 = torch.empty(T, H * D, dtype=dt, device=DEV)
    t2 = torch.tensor([(s, first + j, min(16, 77 - j), j) for j in range(0, 77, 16)] +
                      [(s, first + 77 + j, min(16, 123 - j), 77 + j) for j in range(0, 123, 16)], dtype=torch.int32)
    ops.attn_prefill_mfma(wide, out2, k_dev, v_dev, case["tables"].to(DEV), t2.to(DEV), H, KVH, D, scale, window,
                          shared=shared)
    assert torch.equal(out2[first:first + 200], out[first:first + 200])
    # a launch of many tiles (the same ones again and again, as a padded step's table holds them): at head sizes up to
    # 64 a wavefront of the split-keys kernel then takes four heads instead of two, and a head's bits stay
    out3 = torch.empty(T, H * D, dtype=dt, device=DEV)
    ops.attn_prefill_mfma(wide, out3, k_dev, v_dev, case["tables"].to(DEV), t2.repeat(40, 1).to(DEV), H, KVH, D, scale,
                          window, shared=shared)
    assert torch.equal(out3[first:first + 200], out2[first:first + 200])


@pytest.mark.parametrize("H,KVH,D,page", [(14, 2, 64, 16), (6, 1, 32, 16), (5, 5, 128, 32), (3, 1, 48, 16), (8, 2, 80, 64),
                                           (4, 2, 16, 16)])
@pytest.mark.parametrize("window", [0, 40])
def test_paged_attention_prefill_f32(ops, H, KVH, D, page, window):
    """The 32-bit MFMA attention of prompt portions, at 32-bit tolerance: whole prompts, portions that
    start and end mid-page, a far key that carries a query, pages behind the window never read, and
    the same bits when a request is cut into other portions."""
    dt = torch.float32
    lens = [2, 37, 130, 64, 5, 300, 33, 200]
    q_lens = [2, 37, 2, 64, 3, 45, 17, 200]
    case = paged_case(dt, lens, q_lens, H, KVH, D, page, seed=15, spike=(5, 3) if not window else None)
    if window:
        for s, (n, ql) in enumerate(zip(lens, q_lens)):
            for i in range(max(0, n - ql - window + 1) // page):
                case["kp"][case["tables"][s, i]] = float("nan")
                case["vp"][case["tables"][s, i]] = float("nan")
    T = case["q"].shape[0]
    scale = D ** -0.5
    wide = torch.zeros(T, (H + 2 * KVH) * D, dtype=dt, device=DEV)
    wide[:, :H * D] = case["q"].reshape(T, H * D).to(DEV)
    out = torch.full((T, H * D), 3.0, dtype=dt, device=DEV)
    k_dev, v_dev = case["kp"].to(DEV), v_layout(case["vp"]).to(DEV)
    ops.attn_prefill_f32(wide, out, k_dev, v_dev, case["tables"].to(DEV), tiles_for(lens, q_lens).to(DEV), H, KVH, D,
                         scale, window)
    want = paged_truth(case, lens, q_lens, scale, dt, window or None).reshape(T, H * D)
    torch.testing.assert_close(out.cpu(), want, rtol=2e-5, atol=2e-5)
    if not window:
        row = sum(q_lens[:6]) - 1
        v_far = case["v"][5][3].float()
        got = out.cpu()[row].view(H, D)
        for h in range(H):
            torch.testing.assert_close(got[h], v_far[h // (H // KVH)], rtol=0, atol=2e-2)
    s = 7
    first = sum(q_lens[:s])
    out2 = torch.empty(T, H * D, dtype=dt, device=DEV)
    t2 = torch.tensor([(s, first + j, min(16, 77 - j), j) for j in range(0, 77, 16)] +
                      [(s, first + 77 + j, min(16, 123 - j), 77 + j) for j in range(0, 123, 16)], dtype=torch.int32)
    ops.attn_prefill_f32(wide, out2, k_dev, v_dev, case["tables"].to(DEV), t2.to(DEV), H, KVH, D, scale, window)
    assert torch.equal(out2[first:first + 200], out[first:first + 200])


# ----------------------------------------------------------------------------------------------- fused decode kernels

@pytest.mark.parametrize("M,K,H,KVH,D,page", [(8, 896, 14, 2, 64, 16), (1, 192, 6, 1, 32, 16), (16, 3584, 4, 4, 128, 32),
                                               (5, 120, 3, 1, 96, 64)])
def test_fused_norm_qkv_rope(ops, M, K, H, KVH, D, page):
    torch.manual_seed(13)
    dt = torch.bfloat16
    eps, theta, max_pos, pages = 1e-5, 1e6, 500, 9
    rows = (H + 2 * KVH) * D
    resid = torch.randn(M, K) * 2
    nw, W, b = q(torch.rand(K) + 0.5, dt), q(torch.randn(rows, K) * 0.05, dt), q(torch.randn(rows) * 0.5, dt)
    positions = torch.randint(0, max_pos, (M,), dtype=torch.int32)
    slots = torch.randperm(pages * page)[:M].to(torch.int32)
    if M > 2:
        slots[1] = -1
    # the unfused chain on the CPU
    h = P.rms_norm(resid, nw, eps, dt)
    qkv = P.linear(h, W, b, dt)
    cos, sin = P.rope_tables(max_pos, D, theta)
    qq = P.apply_rope(qkv[:, :H * D].view(M, H, D), cos, sin, positions.long(), dt)
    kk = P.apply_rope(qkv[:, H * D:(H + KVH) * D].view(M, KVH, D), cos, sin, positions.long(), dt)
    vv = qkv[:, (H + KVH) * D:].view(M, KVH, D)
    half = cos[:, :D // 2].contiguous(), sin[:, :D // 2].contiguous()
    kp = torch.full((pages, page, KVH, D), 7.0, dtype=dt, device=DEV)
    vp = torch.full((pages, KVH, D, page), 7.0, dtype=dt, device=DEV)
    q_out = torch.empty(M, H * D, dtype=dt, device=DEV)
    r_dev = resid.to(DEV)
    Wp = ops.pack_weight(W.to(dt).to(DEV), ops.fused_qkv_strip_rows(H, KVH, D, K))
    ops.fused_norm_qkv_rope(r_dev, nw.to(dt).to(DEV), eps, Wp, b.to(dt).to(DEV), q_out, H, KVH, D,
                            half[0].to(DEV), half[1].to(DEV), positions.to(DEV), slots.to(DEV), kp, vp)
    assert torch.equal(r_dev.cpu(), resid)                              # the residual is only read
    torch.testing.assert_close(q_out.float().cpu().view(M, H, D), qq, **tol(dt))
    kflat = kp.float().cpu().view(-1, KVH, D)
    vflat = vp.float().cpu().permute(0, 3, 1, 2).reshape(-1, KVH, D)
    written = torch.zeros(pages * page, dtype=torch.bool)
    for t in range(M):
        if slots[t] >= 0:
            written[slots[t]] = True
            torch.testing.assert_close(kflat[slots[t]], kk[t], **tol(dt))
            torch.testing.assert_close(vflat[slots[t]], vv[t], **tol(dt))
    assert (kflat[~written] == 7.0).all() and (vflat[~written] == 7.0).all()
    # a norm weight stored in 32-bit
    nw32 = torch.rand(K) + 0.5
    ops.fused_norm_qkv_rope(r_dev, nw32.to(DEV), eps, Wp, None, q_out, H, KVH, D, half[0].to(DEV),
                            half[1].to(DEV), positions.to(DEV), None, None, None)
    with pytest.raises(ops.KernelArgumentError):                        # a matrix packed for another kernel
        wrong = ops.pack_weight(W.to(dt).to(DEV), 4)
        ops.fused_norm_qkv_rope(r_dev, nw32.to(DEV), eps, wrong, None, q_out, H, KVH, D, half[0].to(DEV),
                                half[1].to(DEV), positions.to(DEV), None, None, None)
    normed = q(resid * torch.rsqrt((resid * resid).mean(-1, keepdim=True) + eps), dt)
    qkv2 = P.linear(q(nw32 * normed, dt), W, None, dt)
    qq2 = P.apply_rope(qkv2[:, :H * D].view(M, H, D), cos, sin, positions.long(), dt)
    torch.testing.assert_close(q_out.float().cpu().view(M, H, D), qq2, **tol(dt))


@pytest.mark.parametrize("M,K,I", [(8, 896, 4864), (1, 64, 128), (16, 192, 320), (3, 120, 200),
                                   (8, 2048, 5000), (5, 256, 8300)])      # the last two: more units than blocks
def test_fused_norm_gate_up_silu(ops, M, K, I):
    torch.manual_seed(14)
    dt = torch.bfloat16
    eps = 1e-6
    resid = torch.randn(M, K) * 3
    nw, W = q(torch.rand(K) + 0.5, dt), q(torch.randn(2 * I, K) * 0.1, dt)
    h = P.rms_norm(resid, nw, eps, dt)
    gu = P.linear(h, W, None, dt)
    want = P.silu_mul(gu[:, :I], gu[:, I:], dt)
    out = torch.empty(M, I, dtype=dt, device=DEV)
    Wp = ops.pack_weight(W.to(dt).to(DEV), 16, [I, I])
    ops.fused_norm_gate_up_silu(resid.to(DEV), nw.to(dt).to(DEV), eps, Wp, out)
    torch.testing.assert_close(out.float().cpu(), want, rtol=2e-2, atol=2e-2)
    assert ((out.float().cpu() - want).abs() > 1e-2).float().mean() < 0.01


@pytest.mark.parametrize("M,K,H,KVH,D,page", [(64, 896, 14, 2, 64, 16), (17, 192, 6, 1, 32, 16), (40, 1024, 4, 4, 128, 32),
                                               (33, 120, 3, 1, 96, 64), (5, 896, 14, 2, 64, 16)])
def test_panel_qkv_rope(ops, M, K, H, KVH, D, page):
    """q|k|v + bias + rotary + cache write for up to 64 tokens from the normed input kept in LDS."""
    torch.manual_seed(21)
    dt = torch.bfloat16
    theta, max_pos, pages = 1e6, 500, 12
    rows = (H + 2 * KVH) * D
    x = q(torch.randn(M, K), dt)
    W, b = q(torch.randn(rows, K) * 0.05, dt), q(torch.randn(rows) * 0.5, dt)
    positions = torch.randint(0, max_pos, (M,), dtype=torch.int32)
    slots = torch.randperm(pages * page)[:M].to(torch.int32)
    slots[1] = -1
    qkv = P.linear(x, W, b, dt)
    cos, sin = P.rope_tables(max_pos, D, theta)
    qq = P.apply_rope(qkv[:, :H * D].view(M, H, D), cos, sin, positions.long(), dt)
    kk = P.apply_rope(qkv[:, H * D:(H + KVH) * D].view(M, KVH, D), cos, sin, positions.long(), dt)
    vv = qkv[:, (H + KVH) * D:].view(M, KVH, D)
    half = cos[:, :D // 2].contiguous(), sin[:, :D // 2].contiguous()
    kp = torch.full((pages, page, KVH, D), 7.0, dtype=dt, device=DEV)
    vp = torch.full((pages, KVH, D, page), 7.0, dtype=dt, device=DEV)
    q_out = torch.empty(M, H * D, dtype=dt, device=DEV)
    assert ops.panel_fits(M, K)
    Wp = ops.pack_weight(W.to(dt).to(DEV), ops.fused_qkv_strip_rows(H, KVH, D, K))
    wide = torch.zeros(M, K + 16, dtype=dt, device=DEV)                 # a strided input
    wide[:, :K] = x.to(dt).to(DEV)
    ops.panel_qkv_rope(wide[:, :K], Wp, b.to(dt).to(DEV), q_out, H, KVH, D, half[0].to(DEV), half[1].to(DEV),
                       positions.to(DEV), slots.to(DEV), kp, vp)
    torch.testing.assert_close(q_out.float().cpu().view(M, H, D), qq, **tol(dt))
    kflat = kp.float().cpu().view(-1, KVH, D)
    vflat = vp.float().cpu().permute(0, 3, 1, 2).reshape(-1, KVH, D)
    written = torch.zeros(pages * page, dtype=torch.bool)
    for t in range(M):
        if slots[t] >= 0:
            written[slots[t]] = True
            torch.testing.assert_close(kflat[slots[t]], kk[t], **tol(dt))
            torch.testing.assert_close(vflat[slots[t]], vv[t], **tol(dt))
    assert (kflat[~written] == 7.0).all() and (vflat[~written] == 7.0).all()
    # a token's result does not depend on the other tokens of the call; no bias, no cache write
    q_all = torch.empty(M, H * D, dtype=dt, device=DEV)
    ops.panel_qkv_rope(wide[:, :K], Wp, None, q_all, H, KVH, D, half[0].to(DEV), half[1].to(DEV), positions.to(DEV),
                       None, None, None)
    q_one = torch.empty(1, H * D, dtype=dt, device=DEV)
    ops.panel_qkv_rope(wide[M - 1:, :K], Wp, None, q_one, H, KVH, D, half[0].to(DEV), half[1].to(DEV),
                       positions[M - 1:].to(DEV), None, None, None)
    assert torch.equal(q_one[0], q_all[M - 1])
    assert not ops.panel_fits(65, K) and not ops.panel_fits(M, 1032) and not ops.panel_fits(64, 1024)


@pytest.mark.parametrize("M,K,H,KVH,D,page,rows", [(64, 896, 14, 2, 64, 16, 8), (17, 192, 6, 1, 32, 16, 16), (40, 3584, 4, 4, 128, 32, 16),
                                                    (33, 120, 3, 1, 96, 64, 4), (5, 1096, 14, 2, 64, 16, 8), (64, 5120, 5, 1, 128, 16, 16),
                                                    (40, 72, 130, 2, 128, 16, 16), (64, 64, 260, 4, 128, 16, 8), (9, 72, 80, 5, 64, 16, 16)])
def test_stream_qkv_rope(ops, M, K, H, KVH, D, page, rows):
    """q|k|v + bias + rotary + cache write for up to 64 tokens at any width (K no multiple of 32 or of the k-steps a
    wavefront asks for at once; beyond what a block's LDS holds), the matrix streamed from its packed copy whatever
    the height of its strips."""
    torch.manual_seed(23)
    dt = torch.bfloat16
    theta, max_pos, pages = 1e6, 500, 12
    n = (H + 2 * KVH) * D
    x = q(torch.randn(M, K), dt)
    W, b = q(torch.randn(n, K) * 0.05, dt), q(torch.randn(n) * 0.5, dt)
    positions = torch.randint(0, max_pos, (M,), dtype=torch.int32)
    slots = torch.randperm(pages * page)[:M].to(torch.int32)
    slots[1] = -1
    qkv = P.linear(x, W, b, dt)
    cos, sin = P.rope_tables(max_pos, D, theta)
    qq = P.apply_rope(qkv[:, :H * D].view(M, H, D), cos, sin, positions.long(), dt)
    kk = P.apply_rope(qkv[:, H * D:(H + KVH) * D].view(M, KVH, D), cos, sin, positions.long(), dt)
    vv = qkv[:, (H + KVH) * D:].view(M, KVH, D)
    half = cos[:, :D // 2].contiguous().to(DEV), sin[:, :D // 2].contiguous().to(DEV)
    kp = torch.full((pages, page, KVH, D), 7.0, dtype=dt, device=DEV)
    vp = torch.full((pages, KVH, D, page), 7.0, dtype=dt, device=DEV)
    q_out = torch.empty(M, H * D, dtype=dt, device=DEV)
    assert ops.stream_fits(M, K) and not ops.stream_fits(65, K) and not ops.stream_fits(M, K + 4)
    Wp = ops.pack_weight(W.to(dt).to(DEV), rows)
    wide = torch.zeros(M, K + 16, dtype=dt, device=DEV)                 # a strided input
    wide[:, :K] = x.to(dt).to(DEV)
    ops.stream_qkv_rope(wide[:, :K], Wp, b.to(dt).to(DEV), q_out, H, KVH, D, half[0], half[1], positions.to(DEV),
                        slots.to(DEV), kp, vp)
    torch.testing.assert_close(q_out.float().cpu().view(M, H, D), qq, **tol(dt))
    kflat = kp.float().cpu().view(-1, KVH, D)
    vflat = vp.float().cpu().permute(0, 3, 1, 2).reshape(-1, KVH, D)
    written = torch.zeros(pages * page, dtype=torch.bool)
    for t in range(M):
        if slots[t] >= 0:
            written[slots[t]] = True
            torch.testing.assert_close(kflat[slots[t]], kk[t], **tol(dt))
            torch.testing.assert_close(vflat[slots[t]], vv[t], **tol(dt))
    assert (kflat[~written] == 7.0).all() and (vflat[~written] == 7.0).all()
    # a token's result does not depend on the other tokens of the call, nor on the strips' height; a 32-bit bias
    q_all = torch.empty(M, H * D, dtype=dt, device=DEV)
    ops.stream_qkv_rope(wide[:, :K], Wp, b.to(DEV), q_all, H, KVH, D, half[0], half[1], positions.to(DEV), None, None, None)
    assert torch.equal(q_all, q_out)
    q_one = torch.empty(1, H * D, dtype=dt, device=DEV)
    ops.stream_qkv_rope(wide[M - 1:, :K], ops.pack_weight(W.to(dt).to(DEV), 16), b.to(dt).to(DEV), q_one, H, KVH, D, half[0],
                        half[1], positions[M - 1:].to(DEV), None, None, None)
    assert torch.equal(q_one[0], q_all[M - 1])


@pytest.mark.parametrize("M,K,I", [(64, 896, 4864), (17, 64, 128), (48, 3584, 1000), (33, 120, 200), (9, 1048, 100),
                                   (64, 264, 16400), (20, 3584, 18944), (40, 72, 10000), (64, 72, 22000), (33, 72, 30000),
                                   (8, 136, 4864)])
def test_stream_gate_up_silu(ops, M, K, I):
    torch.manual_seed(24)
    dt = torch.bfloat16
    x, W = q(torch.randn(M, K), dt), q(torch.randn(2 * I, K) * (0.1 if K < 2000 else 0.03), dt)
    gu = P.linear(x, W, None, dt)
    want = P.silu_mul(gu[:, :I], gu[:, I:], dt)
    out = torch.full((M, I), 7.0, dtype=dt, device=DEV)
    Wp = ops.pack_weight(W.to(dt).to(DEV), 16, [I, I])
    xd = x.to(dt).to(DEV)
    ops.stream_gate_up_silu(xd, Wp, out)
    torch.testing.assert_close(out.float().cpu(), want, rtol=2e-2, atol=2e-2)
    assert ((out.float().cpu() - want).abs() > 1e-2).float().mean() < 0.01      # a rounding flip of gate or up now and then
    one = torch.empty(1, I, dtype=dt, device=DEV)
    ops.stream_gate_up_silu(xd[M - 1:], Wp, one)
    assert torch.equal(one[0], out[M - 1])


@pytest.mark.parametrize("M,N,K,rows", [(64, 896, 4864, 4), (17, 64, 128, 16), (40, 200, 120, 8), (64, 3584, 18944, 16),
                                        (33, 1001, 1096, 16), (48, 50, 72, 4)])
def test_stream_linear_stores_or_adds_into_the_residual(ops, M, N, K, rows):
    """The plain product of 17 to 64 rows over a packed matrix: bfloat16 and float32 out, with and without bias, and
    the rounded result added into a 32-bit tensor; N no multiple of 32, of 16 or of 4."""
    torch.manual_seed(25)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * (0.1 if K < 2000 else 0.02), dt), q(torch.randn(N), dt)
    want = a @ w.t()
    da, db = a.to(dt).to(DEV), b.to(dt).to(DEV)
    Wp = ops.pack_weight(w.to(dt).to(DEV), rows)
    out = torch.full((M, N), 7.0, dtype=dt, device=DEV)
    ops.stream_linear(da, Wp, db, out)
    torch.testing.assert_close(out.float().cpu(), q(want + b, dt), **tol(dt))
    out32 = torch.full((M, N), 7.0, dtype=torch.float32, device=DEV)
    ops.stream_linear(da, Wp, None, out32)
    torch.testing.assert_close(out32.cpu(), want, rtol=1e-4, atol=1e-4 * K ** 0.5)
    resid = torch.randn(M, N) * 5
    acc = resid.to(DEV)
    ops.stream_linear(da, Wp, db, None, accum=acc)
    assert torch.equal(acc.cpu(), resid + out.float().cpu())            # the rounded product, added in 32-bit
    one = torch.empty(1, N, dtype=dt, device=DEV)                       # a row does not depend on its batch-mates
    ops.stream_linear(da[M - 1:], Wp, db, one)
    assert torch.equal(one[0], out[M - 1])
    other = torch.empty(M, N, dtype=dt, device=DEV)                     # ... nor on the height of the packed strips
    ops.stream_linear(da, ops.pack_weight(w.to(dt).to(DEV), 16 if rows != 16 else 8), db, other)
    assert torch.equal(other, out)


@pytest.mark.parametrize("M,N,K,rows,groups", [(64, 896, 4864, 4, 8), (33, 3584, 18944, 16, 8), (20, 200, 120, 8, 1),
                                               (48, 1001, 9000, 16, 8), (64, 5120, 27648, 16, 8), (17, 3584, 3584, 8, 8),
                                               (40, 512, 1024, 16, 2), (20, 3072, 2048, 16, 8), (5, 6144, 2048, 8, 8),
                                               (33, 8192, 2048, 16, 8)])
def test_stream_linear_with_k_split_over_blocks_and_the_norm_that_adds_the_parts(ops, M, N, K, rows, groups):
    """A plain product with few rows of output and a long K splits K over groups of blocks, which leave 32-bit partial
    sums; the norm that follows adds them up in their order, rounds the sum as the product's own epilogue would have,
    and goes on as if it had been handed that tensor: the same bits as the two steps one after the other."""
    torch.manual_seed(26)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * (0.1 if K < 2000 else 0.02), dt), q(torch.randn(N), dt)
    want = a @ w.t() + b
    da, db = a.to(dt).to(DEV), b.to(dt).to(DEV)
    Wp = ops.pack_weight(w.to(dt).to(DEV), rows)
    parts = ops.stream_linear_split(da, Wp, db)
    n_parts = parts.shape[0]
    assert n_parts == groups and tuple(parts.shape[1:]) == (M, N)
    delta = ops.sum_parts(parts, torch.empty(M, N, dtype=dt, device=DEV))
    torch.testing.assert_close(delta.float().cpu(), q(want, dt), **tol(dt))
    assert torch.equal(delta.float().cpu(), q(parts.sum(0).cpu(), dt)) or n_parts > 2   # (two parts: one order only)
    one = ops.stream_linear_split(da[M - 1:], Wp, db)                   # a row's parts do not depend on its batch-mates
    assert torch.equal(one[:, 0], parts[:, M - 1])
    # the norm over the parts = the norm over the rounded sum
    nw = q(torch.rand(N) + 0.5, dt).to(dt).to(DEV)
    resid = torch.randn(M, N) * 3
    r1, r2 = resid.to(DEV), resid.to(DEV)
    o1 = ops.add_rmsnorm_parts(r1, parts, nw, 1e-6, torch.empty(M, N, dtype=dt, device=DEV))
    o2 = ops.add_rmsnorm(r2, delta, nw, 1e-6, torch.empty(M, N, dtype=dt, device=DEV))
    assert torch.equal(o1, o2) and torch.equal(r1, r2)
    assert torch.equal(r1.cpu(), resid + delta.float().cpu())
    pick = torch.tensor([M - 1, 0, 3], dtype=torch.int32, device=DEV)    # only some rows (the final norm): resid untouched
    r3 = resid.to(DEV)
    o3 = ops.add_rmsnorm_parts(r3, parts, nw, 1e-6, torch.empty(3, N, dtype=dt, device=DEV), rows=pick)
    assert torch.equal(o3, o1[pick.long()]) and torch.equal(r3.cpu(), resid)


@pytest.mark.parametrize("M,N,K", [(8, 896, 4864), (1, 64, 128), (40, 200, 120), (64, 896, 896)])
def test_gemm_skinny_adds_into_the_residual(ops, M, N, K):
    torch.manual_seed(15)
    dt = torch.bfloat16
    a, w, b = q(torch.randn(M, K), dt), q(torch.randn(N, K) * 0.1, dt), q(torch.randn(N), dt)
    resid = torch.randn(M, N) * 5
    acc = resid.to(DEV)
    ops.gemm_skinny(a.to(dt).to(DEV), w.to(dt).to(DEV), b.to(dt).to(DEV), None, accum=acc)
    out = torch.empty(M, N, dtype=dt, device=DEV)
    ops.gemm_skinny(a.to(dt).to(DEV), w.to(dt).to(DEV), b.to(dt).to(DEV), out)
    assert torch.equal(acc.cpu(), resid + out.float().cpu())            # the rounded product, added in 32-bit


def test_argmax_over_a_wide_vocabulary(ops):
    torch.manual_seed(16)
    logits = torch.randn(70, 151936)
    logits[5, 150000] = logits[5, 20] = 60.0                            # a tie across chunks: the first maximum
    logits[6, :] = float("-inf")
    logits[6, 151935] = -3.0
    out = torch.empty(70, dtype=torch.int32, device=DEV)
    ops.argmax_rows(logits.to(DEV), out)
    assert out.cpu().tolist() == logits.argmax(-1).tolist() and out[5].item() == 20 and out[6].item() == 151935

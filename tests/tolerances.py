"""How close the engine must be to the plain implementation.

float32: both sides compute in 32-bit and differ only in the order of their sums: 2e-5 of the
logits' own largest magnitude (no floor: tiny models have logits well below 1).

bfloat16: both sides round to bfloat16 at the same places, so they differ by the order of their
32-bit sums and by the roundings that fall the other way because of it. How much that is, is
measured for each model: the plain implementation runs it in bfloat16 with several summation orders
(``Plain.bf16_noise``, the way the reference measures its 16-bit floor with two batchings of one
model, reference baselines/make_golden.py:195-217), and the engine may be twice as far from the
plain implementation as the plain implementation's orders are from each other (in a small model the
flipped roundings are few, so their largest effect over a few sequences is a coarse estimate; the
tests compare many more rows, and the engine differs in more 32-bit steps than its sums). A wrong key, mask, page or position moves logits by tens of per cent of their spread,
far beyond it.

Tokens: a generated token must be the first choice of the plain implementation (in the engine's
precision) at that place, unless the plain logit of the token lies within twice the bound of the
maximum: each of the two logits may be off by the bound, so only then can an engine within the bound
prefer the other token (a near-tie, reference tests/test_gpu.py:59-71). Such exemptions are counted.
"""
import torch

F32_REL = 2e-5
BF16_NOISE_FACTOR = 2.0


def logits_bound(want: torch.Tensor, dt, noise: float | None = None) -> float:
    """Largest |difference| allowed between the engine's logits and ``want`` (the plain implementation's, in
    the precision ``dt``). ``noise``: the model's measured bfloat16 floor (needed for bfloat16)."""
    if dt == torch.float32:
        return F32_REL * float(want.abs().max())
    assert noise is not None and noise > 0, "a bfloat16 comparison needs the model's measured noise floor"
    return BF16_NOISE_FACTOR * noise


def assert_logits_close(got: torch.Tensor, want: torch.Tensor, dt, what: str = "", noise: float | None = None) -> float:
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    bound = logits_bound(want, dt, noise)
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: max |diff| {err:.3e} > {bound:.3e} (largest logit {float(want.abs().max()):.3g})"
    return err


def check_greedy_token(row: torch.Tensor, tok: int, dt, noise: float | None, what: str = "") -> bool:
    """``tok`` was chosen greedily where the plain logits (in the precision ``dt``) are ``row``. Returns True
    if it is not the plain first choice but a near-tie with it (exempted); raises if it is further away."""
    best = int(row.argmax())
    if tok == best:
        return False
    allowed = 2 * logits_bound(row, dt, noise)
    gap = float(row[best] - row[tok])
    assert gap <= allowed, f"{what}: token {tok} chosen, the plain pick {best} is {gap:.3e} ahead (near-tie: {allowed:.3e})"
    return True


def near_ties(rows: torch.Tensor, dt, noise: float | None) -> int:
    """Rows whose two largest logits are a near-tie: the most exemptions a run over these rows can have."""
    top2 = rows.topk(2, dim=-1).values
    return int(sum(float(t[0] - t[1]) <= 2 * logits_bound(r, dt, noise) for t, r in zip(top2, rows)))


def measured_noise(bf16_logits, sequences) -> float:
    """The bfloat16 floor of any model given as a function ids -> bfloat16 logits built from the plain
    implementation's parts: the largest difference between its two summation orders over ``sequences``."""
    from plain import qwen2_plain as P
    worst = 0.0
    for ids in sequences:
        a = bf16_logits(ids)
        for k in range(1, P.NUM_ORDERS):
            with P.summation_order(k):
                b = bf16_logits(ids)
            worst = max(worst, float((a - b).abs().max()))
    return worst


def assert_part_close(got: torch.Tensor, want: torch.Tensor, dt, what: str = "") -> float:
    """One part alone (a mixer, a feed-forward). float32 as for logits. bfloat16: the output's own rounding is
    up to 2^-9 of its magnitude and each rounded tensor inside the part (softmax weights, attention output,
    silu(gate)*up) can add as much again, so four roundings of the largest magnitude bound what differing
    sum orders can do; a wrong element is off by its whole size."""
    assert got.shape == want.shape and torch.isfinite(got).all(), f"{what}: shape or non-finite values"
    scale = float(want.abs().max())
    bound = (F32_REL if dt == torch.float32 else 2.0 ** -7) * scale
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: max |diff| {err:.3e} > {bound:.3e} (largest value {scale:.3g})"
    return err

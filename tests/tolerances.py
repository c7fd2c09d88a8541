"""How close the engine must be to the plain implementation. Fixed before the first GPU run.

float32: both sides compute in 32-bit and differ only in the order of their sums; a few layers of
that stay below 2e-5 of the logits' scale. bfloat16: both sides round at the same places, so they
differ by the order of 32-bit sums AND by the one-unit flips of bfloat16 roundings those cause
(2^-8 relative each); 2 % of the logits' scale bounds what such flips add up to over a few
layers, while a wrong key, mask, page or position moves logits by tens of per cent.
"""
import torch

REL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


def assert_logits_close(got: torch.Tensor, want: torch.Tensor, dt, what: str = "") -> float:
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= REL[dt] * scale, f"{what}: max |diff| {err:.3e} > {REL[dt] * scale:.3e} (scale {scale:.3g})"
    return err

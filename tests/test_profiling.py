"""The per-operation accounting behind `bench.py`'s kernel tables: labels are free when nothing collects,
count calls, bytes and flops when something does, nest into the outer operation, and, on the GPU, get
the device time of the kernels launched inside them."""
from __future__ import annotations

import pytest
import torch

from tokenmill_amd import profiling


def test_labels_cost_nothing_until_something_collects():
    called = []
    with profiling.label("idle", lambda: called.append(1) or (1, 1)) as r:
        assert r is profiling._OFF
    assert not called and not profiling.on()


def test_calls_bytes_and_flops_add_up_and_inner_labels_belong_to_the_outer_one():
    with profiling.collect(trace=False) as got:
        assert profiling.on()
        for _ in range(3):
            with profiling.label("product", lambda: (100, 2000)):
                with profiling.label("norm", lambda: (7, 7)):          # inside a product: part of it
                    pass
        with profiling.label("norm", lambda: (8, 16)):                   # by itself: an operation of its own
            pass
        with profiling.label("bare"):
            pass
        with pytest.raises(RuntimeError):
            with profiling.collect(trace=False):
                pass
    assert not profiling.on()
    ops = got["ops"]
    assert (ops["product"].calls, ops["product"].bytes, ops["product"].flops) == (3, 300, 6000)
    assert (ops["norm"].calls, ops["norm"].bytes, ops["norm"].flops) == (1, 8, 16)
    assert (ops["bare"].calls, ops["bare"].bytes) == (1, 0)
    assert "kernel_us" not in got


def test_an_error_inside_leaves_nothing_switched_on():
    with pytest.raises(ValueError):
        with profiling.collect(trace=False):
            with profiling.label("x"):
                raise ValueError("inside")
    assert not profiling.on()
    with profiling.collect(trace=False) as got:                          # and a label opened after it is a top-level one
        with profiling.label("y", lambda: (1, 2)):
            pass
    assert got["ops"]["y"].calls == 1


def test_the_floor_is_the_longer_of_bytes_and_flops():
    op = profiling.OpCost(calls=1, bytes=8.0e6, flops=2.5e9)            # 1 us of HBM, 1 us of bfloat16 MFMA
    assert profiling.floor_us(op, "bfloat16") == pytest.approx(1.0)
    assert profiling.floor_us(op, "float32") == pytest.approx(2.5e9 / 157.3e12 * 1e6)
    assert profiling.nbytes(torch.zeros(3, 4), None, torch.zeros(5, dtype=torch.bfloat16)) == 48 + 10


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["bfloat16", "float32"])
def test_a_step_under_collect_names_every_operation_with_its_cost_and_device_time(model_dirs, dtype_name):
    """One prompt step and one decode step of the first tiny configuration: every operation of a layer
    appears with the calls it must have, the product's bytes and flops follow from the sizes, each got
    device time (the span of its kernels on the GPU's timeline), and the logits are those of the same
    steps without the profile."""
    from tokenmill_amd.replay import ReplaySession
    from conftest import TINY_A, random_ids
    ids = random_ids(20, TINY_A["vocab_size"], 5)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:19], "want": [18]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": ids[19:], "want": [0]}], "end": ["a"]}]
    unprofiled = ReplaySession(model_dirs["A"], dtype_name, 64)
    want = [unprofiled.run_step(s) for s in steps]
    session = ReplaySession(model_dirs["A"], dtype_name, 64)
    with profiling.collect() as got:
        logits = [session.run_step(s) for s in steps]
    for a, b in zip(logits, want):
        assert (a == b).all()
    ops = got["ops"]
    L, hidden, H, KVH = (TINY_A[k] for k in ("num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads"))
    D, I, V = hidden // H, TINY_A["intermediate_size"], TINY_A["vocab_size"]
    for name in ("embed", "qkv", "attention", "o_proj", "gate_up", "down", "head"):
        assert name in ops, sorted(ops)
        assert ops[name].device_us > 0, name
    assert ops["qkv"].calls == ops["attention"].calls == ops["down"].calls == 2 * L and ops["head"].calls == 2
    es = 2 if dtype_name == "bfloat16" else 4
    n_qkv = (H + 2 * KVH) * D
    assert ops["qkv"].flops == 2 * L * 20 * hidden * n_qkv                 # 19 + 1 rows through every layer
    assert ops["qkv"].bytes >= 2 * L * hidden * n_qkv * es                 # the matrix at least, once a call
    assert ops["down"].flops == 2 * L * 20 * I * hidden and ops["head"].flops == 2 * 2 * hidden * V
    assert got["kernel_us"] > 0 and any("attn" in k for k in got["kernels"])      # the kernels by their own names too

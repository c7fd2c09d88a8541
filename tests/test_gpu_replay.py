"""Replay on the GPU against the plain implementation: whole, prefill + decode, portions, mixed."""
from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import ROOT, TINY, random_ids
from tolerances import assert_logits_close

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def sessions(model_dirs):
    """(config name, dtype name, max_tokens) -> ReplaySession, built once for the module."""
    from tokenmill_amd.replay import ReplaySession

    cache = {}

    def get(name, dtype_name, max_tokens=512, page=16):
        key = (name, dtype_name, max_tokens, page)
        if key not in cache:
            cache[key] = ReplaySession(model_dirs[name], dtype_name, max_tokens, page_size=page)
        return cache[key]

    return get


def run_trace(session, steps):
    """Runs steps; returns {(request, position): logits row} for every wanted place."""
    got = {}
    pos = dict(session.lengths)
    for rec in steps:
        out = session.run_step(rec)
        r = 0
        for ent in rec["entries"]:
            base = pos.get(ent["id"], 0)
            for w in ent.get("want", []):
                got[(ent["id"], base + w)] = torch.from_numpy(out[r].copy())
                r += 1
            pos[ent["id"]] = base + len(ent["tokens"])
        for rid in rec.get("end", []):
            pos.pop(rid, None)
        assert out is None or r == out.shape[0]
    return got


def check(got, plain, requests, dt, what):
    """Every row against the plain implementation's row for the same (request, position); returns the
    largest difference seen."""
    noise = plain.bf16_noise() if dt == torch.bfloat16 else None
    worst = 0.0
    for (rid, p), row in sorted(got.items()):
        want = plain.logits(requests[rid], dt)[p]
        worst = max(worst, assert_logits_close(row, want, dt, f"{what} request {rid} position {p}", noise))
    return worst


def poison_freed_pages(session):
    """From now on a page that goes back to the free list has its keys and values filled with NaN in every
    layer: whatever reads a slot that its request has not written since (a stale key behind a context's end,
    the rest of a page that is used again, a padding row) then shows in the logits as NaN."""
    import math
    pools = session.pools
    for g, alloc in enumerate(session.manager.allocators):
        plain_release = alloc.release

        def release(pages, g=g, plain_release=plain_release):
            pages = list(pages)
            if pages:
                idx = torch.tensor(pages, dtype=torch.long, device=pools.k[g].device)
                pools.k[g].index_fill_(1, idx, math.nan)
                pools.v[g].index_fill_(1, idx, math.nan)
            return plain_release(pages)

        alloc.release = release


def assert_all_given_back(session):
    session.manager.check_invariants()
    assert not session.manager.live and session.manager.num_free_pages == session.num_pages


def whole(requests):
    return [{"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], "end": [rid]}
            for i, (rid, ids) in enumerate(requests.items())]


def prefill_then_decode(requests, tail=32):
    steps, n = [], 0
    for rid, ids in requests.items():
        head = max(1, len(ids) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[:head], "want": [head - 1]}], "end": []})
        n += 1
        for p in range(head, len(ids)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [ids[p]], "want": [0]}],
                          "end": [rid] if p == len(ids) - 1 else []})
            n += 1
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(7, 2, 12, 3, 2, 5, 16, 2, 9, 4)):
    steps, n = [], 0
    for rid, ids in requests.items():
        p, k = 0, 0
        while p < len(ids):
            size = min(sizes[k % len(sizes)], len(ids) - p)
            if len(ids) - p - size == 1:          # never leave a single token: portions are >= 2 here
                size += 1
            steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[p:p + size],
                                                  "want": list(range(size))}],
                          "end": [rid] if p + size == len(ids) else []})
            p, k, n = p + size, k + 1, n + 1
    return steps


def mixed(requests, seed, live=4, max_portion=11):
    """Up to ``live`` requests at a time; each step gives some of them a portion of their prompt and
    the others one token; requests enter as others end."""
    g = torch.Generator().manual_seed(seed)
    waiting = list(requests.items())
    running: dict[str, int] = {}
    steps, n = [], 0
    while waiting or running:
        while waiting and len(running) < live:
            rid, _ = waiting.pop(0)
            running[rid] = 0
        entries, ended = [], []
        for rid in list(running):
            ids, p = requests[rid], running[rid]
            if int(torch.randint(0, 5, (1,), generator=g)) == 0 and len(running) > 1:
                continue                              # left out of this step; goes on later
            left = len(ids) - p
            prompt_part = p < (2 * len(ids)) // 3      # first two thirds in portions, the rest token by token
            size = min(left, int(torch.randint(2, max_portion + 1, (1,), generator=g))) if prompt_part else 1
            if left - size == 1 and prompt_part:
                size += 1
            entries.append({"id": rid, "tokens": ids[p:p + size], "want": list(range(size))})
            running[rid] = p + size
            if p + size == len(ids):
                ended.append(rid)
        for rid in ended:
            del running[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": ended})
            n += 1
    return steps


def make_requests(name, lengths, seed):
    vocab = TINY[name][0]["vocab_size"]
    return {f"r{i}": random_ids(L, vocab, seed * 100 + i) for i, L in enumerate(lengths)}


LENGTHS = {"A": [5, 17, 33, 70], "B": [1, 9, 24, 40, 81], "C": [3, 50, 95], "D": [2, 31, 64, 100]}
# (configuration, page size): B at its own page of 8 (the generic attention) and at 16 (the matrix-unit attention)
CASES = [("A", 16), ("B", 8), ("B", 16), ("C", 16), ("D", 16), ("D", 32)]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_each_request_alone_and_whole(sessions, plains, name, page, dtype_name):
    s = sessions(name, dtype_name, page=page)
    reqs = make_requests(name, LENGTHS[name], 1)
    got = run_trace(s, whole(reqs))
    assert len(got) == sum(LENGTHS[name])
    check(got, plains[name], reqs, DTYPES[dtype_name], "whole")
    assert_all_given_back(s)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_prefill_then_last_32_tokens_one_by_one(sessions, plains, name, page, dtype_name):
    s = sessions(name, dtype_name, page=page)
    reqs = make_requests(name, LENGTHS[name], 2)
    got = run_trace(s, prefill_then_decode(reqs))
    check(got, plains[name], reqs, DTYPES[dtype_name], "prefill+decode")
    assert_all_given_back(s)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_portions_of_changing_size(sessions, plains, name, page, dtype_name):
    s = sessions(name, dtype_name, page=page)
    reqs = make_requests(name, [n for n in LENGTHS[name] if n >= 2], 3)
    steps = portions(reqs)
    assert min(len(e["tokens"]) for st in steps for e in st["entries"]) == 2
    got = run_trace(s, steps)
    check(got, plains[name], reqs, DTYPES[dtype_name], "portions")
    assert_all_given_back(s)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", CASES)
def test_mixed_batches_with_pages_used_again(model_dirs, plains, name, page, dtype_name):
    from tokenmill_amd.replay import ReplaySession
    lengths = [37, 64, 21, 90, 48, 33, 75, 18, 59, 44, 96, 27, 70, 52, 85, 40, 113, 66, 31, 101, 58, 79, 45, 120, 88, 62]
    # The pool holds what four live requests of the longest kind need and no more (each counted rounded up to 64
    # tokens, as the replay program counts): the free list wraps several times, so most pages are handed out three
    # or four times. A page that goes back is filled with NaN: a read of anything its next owner has not written shows.
    most = 4 * 128
    s = ReplaySession(model_dirs[name], dtype_name, most, page_size=page)
    poison_freed_pages(s)
    reqs = make_requests(name, lengths, 4)
    steps = mixed(reqs, seed=5)
    assert max(len(st["entries"]) for st in steps) == 4
    assert any(len(e["tokens"]) == 1 for st in steps for e in st["entries"] if len(st["entries"]) > 1)
    got = run_trace(s, steps)
    assert sum(-(-n // page) for n in lengths) >= 3 * s.num_pages, "the free list must wrap several times"
    assert len(got) == sum(lengths)
    check(got, plains[name], reqs, DTYPES[dtype_name], "mixed")
    assert_all_given_back(s)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, plains, tmp_path, dtype_name):
    """The program itself: JSON lines on stdin, <step>.f32 files, 'done <step>' lines, exit 0."""
    reqs = make_requests("A", [19, 6], 6)
    steps = [
        {"step": 0, "entries": [{"id": "r0", "tokens": reqs["r0"][:10], "want": [0, 9]}], "end": []},
        {"step": 1, "entries": [{"id": "r0", "tokens": reqs["r0"][10:12], "want": []},
                                {"id": "r1", "tokens": reqs["r1"], "want": [5]}], "end": ["r1"]},
        {"step": 2, "entries": [{"id": "r0", "tokens": reqs["r0"][12:], "want": [6]}], "end": ["r0"]},
    ]
    out = tmp_path / "out"
    env = dict(os.environ)
    page = ["--block-size", "8"] if dtype_name == "bfloat16" else []          # the default page, and another one
    r = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(model_dirs["A"]), "--dtype", dtype_name,
                        "--out", str(out), "--max-tokens", "128", *page],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    done = [ln for ln in r.stdout.splitlines() if ln.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2"]
    assert f"pages of {8 if page else 16}" in r.stdout
    dt = DTYPES[dtype_name]
    vocab = TINY["A"][0]["vocab_size"]
    f0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, vocab))
    f1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, vocab))
    f2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, vocab))
    assert f0.shape[0] == 2 and f1.shape[0] == 1 and f2.shape[0] == 1
    p = plains["A"]
    noise = p.bf16_noise()
    assert_logits_close(f0[0], p.logits(reqs["r0"], dt)[0], dt, "step 0 place 0", noise)
    assert_logits_close(f0[1], p.logits(reqs["r0"], dt)[9], dt, "step 0 place 9", noise)
    assert_logits_close(f1[0], p.logits(reqs["r1"], dt)[5], dt, "step 1 r1", noise)
    assert_logits_close(f2[0], p.logits(reqs["r0"], dt)[18], dt, "step 2 r0", noise)

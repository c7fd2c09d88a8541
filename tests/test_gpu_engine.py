"""Generation through the engine's entry points on the GPU, checked against the plain
implementation: every token the engine produced must be the plain implementation's choice at that
place of the engine's own sequence (or lie within the tolerance of a near-tie)."""
from __future__ import annotations

import json
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, TINY, random_ids
from plain import qwen2_plain as P
from tolerances import check_greedy_token, logits_bound, near_ties

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def make_engine(model_dir, dtype_name, **kw):
    from tokenmill_amd import EngineConfig, LLMEngine
    base = dict(model=str(model_dir), dtype=dtype_name, block_size=16, kv_cache_mb=8, max_model_len=256,
                max_num_seqs=32, max_num_batched_tokens=512, watermark=0.0)
    base.update(kw)
    return LLMEngine(EngineConfig(**base))


def verify(plain, prompt, out, dt, params=None, seed=0):
    """Every generated token is what the plain implementation (in the same precision) picks after the same
    tokens, or a near-tie with it under the measured bound. Returns the number of such exemptions; they can
    never be more than the near-ties among the rows (asserted)."""
    logits = plain.logits(list(prompt) + list(out), dt)[len(prompt) - 1:-1]
    noise = plain.bf16_noise() if dt == torch.bfloat16 else None
    exempt = 0
    for n, (row, tok) in enumerate(zip(logits, out)):
        if params is None or params.greedy:
            exempt += check_greedy_token(row, tok, dt, noise, f"token {n}")
        else:
            want, margin = P.sample_token(row, params.temperature, params.top_k, params.top_p, seed, n)
            if tok != want:
                # logits off by at most the bound move every probability, and so the point where the random
                # number falls in the cumulative distribution, by at most 2 * bound / temperature
                allowed = 2 * logits_bound(row, dt, noise) / params.temperature
                assert margin <= allowed, f"token {n}: sampled {tok}, plain {want} (margin {margin:.3e} > {allowed:.3e})"
                exempt += 1
    if params is None or params.greedy:
        assert exempt <= near_ties(logits, dt, noise)
    return exempt


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_greedy_generation_whole_prompts(model_dirs, plains, dtype_name):
    """The first tiny configuration: prompts of 5 / 17 / 33 ids, whole-prompt prefill, 16 greedy tokens."""
    from tokenmill_amd import SamplingParams
    eng = make_engine(model_dirs["A"], dtype_name)
    prompts = [random_ids(n, 256, 20 + i) for i, n in enumerate((5, 17, 33))]
    outs = eng.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [len(o) for o in outs] == [16, 16, 16]
    flips = sum(verify(plains["A"], p, o, DTYPES[dtype_name]) for p, o in zip(prompts, outs))
    assert flips == 0 or dtype_name == "bfloat16"       # (bfloat16: never more than the near-ties, checked by verify)
    assert not eng.scheduler.live and eng.cache.num_free_pages == eng.cache.num_pages
    assert eng.stats["prompt_steps"] == 1 and eng.stats["decode_steps"] == 15 and eng.stats["tokens_out"] == 48


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_sampled_generation_chunked_and_mixed(model_dirs, plains, dtype_name):
    """The second tiny configuration: page size 8, prefill in portions of 12 mixed with decodes,
    temperature 0.8 with a fixed seed, prompts of 1 / 9 / 24 / 40 ids, 20 tokens."""
    from tokenmill_amd import SamplingParams
    eng = make_engine(model_dirs["B"], dtype_name, block_size=8, enable_chunked_prefill=True,
                      max_num_batched_tokens=12)
    prompts = [random_ids(n, 384, 30 + i) for i, n in enumerate((1, 9, 24, 40))]
    params = [SamplingParams(max_tokens=20, temperature=0.8, seed=100 + i, ignore_eos=True) for i in range(4)]
    outs = eng.generate(prompts, params)
    assert [len(o) for o in outs] == [20] * 4
    for i, (p, o) in enumerate(zip(prompts, outs)):
        verify(plains["B"], p, o, DTYPES[dtype_name], params[i], seed=100 + i)
    assert len({tuple(o) for o in outs}) == 4
    assert eng.cache.num_free_pages == eng.cache.num_pages
    # the same request alone gives the same tokens: a request's draws do not depend on its batch-mates
    alone = make_engine(model_dirs["B"], dtype_name, block_size=8).generate([prompts[2]], params[2])[0]
    if dtype_name == "float32":
        assert alone == outs[2]
    else:                                               # a rounding may fall the other way in another batch: near-ties only
        verify(plains["B"], prompts[2], alone, torch.bfloat16, params[2], seed=102)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_top_k_and_top_p_through_the_engine(model_dirs, plains, dtype_name):
    """Temperature sampling with top-k and with top-p, prompts in portions beside decodes (the kernels alone
    are compared with the plain sampler on equal logits in tests/test_gpu_kernels.py). In float32 every token
    is the plain implementation's. In bfloat16 the logits differ by up to the measured bound b, which can move
    a token across the edge of the kept set, so what is asserted is membership in the widest set that logits
    within b of the plain ones could keep: for top-k a scaled logit within 2b/T of the k-th largest; for top-p
    the least mass that can stand before the token (the tokens more than 2b/T above it, each probability
    lowered by e^(-2b/T)) at most p."""
    import math
    from tokenmill_amd import SamplingParams
    eng = make_engine(model_dirs["B"], dtype_name, block_size=8, enable_chunked_prefill=True, max_num_batched_tokens=20)
    dt = DTYPES[dtype_name]
    prompts = [random_ids(n, 384, 130 + i) for i, n in enumerate((9, 40, 24, 3, 33, 17))]
    temp = 0.8
    params = [SamplingParams(max_tokens=20, temperature=temp, seed=300 + i, ignore_eos=True,
                             **({"top_k": 5} if i % 2 == 0 else {"top_p": 0.9})) for i in range(len(prompts))]
    outs = eng.generate(prompts, params)
    assert eng.cache.num_free_pages == eng.cache.num_pages
    noise = plains["B"].bf16_noise() if dt == torch.bfloat16 else None
    moved = 0
    for i, (p, o, sp) in enumerate(zip(prompts, outs, params)):
        assert len(o) == 20
        logits = plains["B"].logits(p + o, dt)[len(p) - 1:-1]
        for n, (row, tok) in enumerate(zip(logits, o)):
            want, _ = P.sample_token(row, sp.temperature, sp.top_k, sp.top_p, 300 + i, n)
            if dt == torch.float32:
                assert tok == want, f"request {i} token {n}: {tok}, plain {want}"
                continue
            moved += tok != want
            slack = 2 * logits_bound(row, dt, noise) / temp
            z = row.double() / temp
            if sp.top_k > 0:
                kth = z.sort(descending=True).values[sp.top_k - 1]
                assert z[tok] >= kth - slack, f"request {i} token {n}: {tok} is not among the {sp.top_k} largest, near-ties counted"
            else:
                probs = torch.softmax(z, dim=-1)
                before = float(probs[z > z[tok] + slack].sum()) * math.exp(-slack)
                assert before <= sp.top_p, f"request {i} token {n}: a mass of at least {before:.3f} stands before {tok}"
    print(f"{dtype_name}: {moved} of 120 sampled tokens differ from the plain implementation's")
    # a shift of b moves each probability by up to 2b/T = 3%: a few draws in a hundred fall that close to an edge
    assert moved <= 24


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunked", [False, True])
def test_same_tokens_under_every_cutting_and_a_starved_pool(model_dirs, plains, dtype_name, chunked):
    """16 prompts at once (reference tests/test_engine_greedy.py:25-88): small pages, small budgets,
    and so few pages that requests are preempted and recomputed."""
    from tokenmill_amd import SamplingParams
    lengths = [1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 17, 31, 40, 64, 3, 11]
    prompts = [random_ids(n, 307, 50 + i) for i, n in enumerate(lengths)]
    sp = SamplingParams(max_tokens=24, ignore_eos=True)
    dt = DTYPES[dtype_name]
    roomy = make_engine(model_dirs["C"], dtype_name, block_size=16, enable_chunked_prefill=chunked,
                        max_num_batched_tokens=16 if chunked else 40)
    base = roomy.generate(prompts, sp)
    for p, o in zip(prompts, base):
        verify(plains["C"], p, o, dt)
    starved = make_engine(model_dirs["C"], dtype_name, block_size=4, kv_cache_mb=None, num_blocks=40,
                          enable_chunked_prefill=chunked, max_num_batched_tokens=12 if chunked else 512)
    outs = starved.generate(prompts, sp)
    assert starved.scheduler.evictions > 0
    assert starved.cache.num_free_pages == starved.cache.num_pages and not starved.scheduler.live
    starved.cache.check_invariants()
    for p, o in zip(prompts, outs):
        assert len(o) == 24
        verify(plains["C"], p, o, dt)
    if dtype_name == "float32":
        assert outs == base


def test_steps_of_17_to_48_tokens_take_the_panel_and_stream_products(model_dirs, plains):
    """24 requests decoding together, and prompt steps of 20 to 40 tokens: the q|k|v product that keeps the normed
    input in LDS and the gate|up product that streams its matrix run (counted by the step program), and every token
    is the plain implementation's."""
    from tokenmill_amd import SamplingParams
    prompts = [random_ids(1 + (7 * i) % 19, 384, 300 + i) for i in range(24)]
    layers = 3
    eng = make_engine(model_dirs["B"], "bfloat16", max_num_batched_tokens=40)
    assert not eng.runner.program.foreign_parts               # every part of this model is an operation of the library's
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 10
        verify(plains["B"], p, o, torch.bfloat16)
    took = eng.runner.program.counters()
    assert took["qkv_panel"] >= 9 * layers and took["gate_up_stream"] == took["qkv_panel"]     # the decode steps of 24 tokens at least
    assert eng.cache.num_free_pages == eng.cache.num_pages


def test_without_the_packed_copy_of_the_matrices(model_dirs, plains):
    """`pack_weights=False` keeps one copy of each matrix: the decode steps then take the kernels that
    read it row-major, and the tokens are still the plain implementation's."""
    from tokenmill_amd import SamplingParams
    eng = make_engine(model_dirs["B"], "bfloat16", pack_weights=False)
    layer = eng.model.layers[0]
    assert layer.mixer.qkv.packed is None and layer.ffn.down.packed is None
    packed = make_engine(model_dirs["B"], "bfloat16")
    assert packed.model.layers[0].mixer.qkv.packed is not None and packed.model.layers[0].ffn.gate_up.packed.parts == (320, 320)
    prompts = [random_ids(n, 384, 400 + i) for i, n in enumerate((3, 20, 33))]
    sp = SamplingParams(max_tokens=12, ignore_eos=True)
    for e in (eng, packed):
        for p, o in zip(prompts, e.generate(prompts, sp)):
            verify(plains["B"], p, o, torch.bfloat16)


def test_stop_rules_abort_and_rejections(model_dirs):
    from tokenmill_amd import RequestRejected, SamplingParams
    eng = make_engine(model_dirs["A"], "float32", max_model_len=40)
    prompt = random_ids(10, 256, 70)
    free_run = eng.generate([prompt], SamplingParams(max_tokens=12, ignore_eos=True))[0]
    # max_model_len stops generation with "length" (reference tests/test_engine_greedy.py:203-208)
    s = eng.add_request("long", random_ids(35, 256, 71), SamplingParams(max_tokens=100, ignore_eos=True))
    while eng.has_unfinished():
        eng.step()
    assert s.why_done == "length" and s.n_tokens == 40
    # an end-of-sequence token stops with "stop" and stays in the output
    eng.eos_ids = {free_run[4]}
    stopped = eng.generate([prompt], SamplingParams(max_tokens=12))[0]
    first = free_run.index(free_run[4])
    assert stopped == free_run[:first + 1]
    assert eng.generate([prompt], SamplingParams(max_tokens=12, ignore_eos=True))[0] == free_run
    # abort mid-run gives every page back (reference tests/test_engine_greedy.py:174-184)
    eng.add_request("x", prompt, SamplingParams(max_tokens=50, ignore_eos=True))
    eng.add_request("y", random_ids(20, 256, 72), SamplingParams(max_tokens=50, ignore_eos=True))
    for _ in range(3):
        eng.step()
    out = eng.abort_request("x")
    assert out.finished and out.finish_reason == "abort"
    eng.abort_request("y")
    assert not eng.has_unfinished() and eng.cache.num_free_pages == eng.cache.num_pages
    assert eng.abort_request("nobody") is None
    for bad in ([], list(range(40))):
        with pytest.raises(RequestRejected):
            eng.add_request("bad", bad, SamplingParams())
    with pytest.raises(RequestRejected):
        eng.add_request("vocab", [0, 256], SamplingParams())
    eng.add_request("dup", prompt, SamplingParams(max_tokens=1))
    with pytest.raises(RequestRejected):
        eng.add_request("dup", prompt, SamplingParams(max_tokens=1))
    # a prompt that can never fit the pool is finished with an error, not left waiting
    tiny_pool = make_engine(model_dirs["A"], "float32", kv_cache_mb=None, num_blocks=2, max_model_len=200)
    tiny_pool.add_request("big", random_ids(60, 256, 73), SamplingParams(max_tokens=4))
    outs = tiny_pool.step()
    assert outs[0].finished and outs[0].error == "prompt does not fit in the KV cache"
    # a request that has been here longer than request_timeout ends with "timeout", live or queued, and gives
    # its pages back; a younger one goes on (reference src/infer/engine/engine.py:213-216)
    import time
    timed = make_engine(model_dirs["A"], "float32", request_timeout=1000.0, max_num_seqs=1)
    old = timed.add_request("old", prompt, SamplingParams(max_tokens=50, ignore_eos=True))
    queued = timed.add_request("old-queued", prompt, SamplingParams(max_tokens=50, ignore_eos=True),
                               arrival_time=time.monotonic() - 2000.0)
    young = timed.add_request("young", prompt, SamplingParams(max_tokens=3, ignore_eos=True))
    outs = timed.step()
    assert [(o.request_id, o.finish_reason) for o in outs if o.finished] == [("old-queued", "timeout")]
    assert queued.why_done == "timeout" and not queued.generated
    old.t_arrived -= 2000.0
    outs = timed.step()
    assert ("old", "timeout") in [(o.request_id, o.finish_reason) for o in outs]
    assert 1 <= len(old.generated) < 50
    while timed.has_unfinished():
        timed.step()
    assert young.why_done == "length" and len(young.generated) == 3
    assert timed.cache.num_free_pages == timed.cache.num_pages
    # generate() runs a batch that arrives at once to its end: however long the batch takes, none of it times out
    hurried = make_engine(model_dirs["A"], "float32", request_timeout=1e-9)
    assert [len(o) for o in hurried.generate([prompt, prompt[:3]], SamplingParams(max_tokens=4, ignore_eos=True))] == [4, 4]
    assert hurried.cfg.request_timeout == 1e-9
    # ... while a request that came through add_request keeps its timeout during that loop
    own = hurried.add_request("own", prompt, SamplingParams(max_tokens=4, ignore_eos=True))
    assert [len(o) for o in hurried.generate([prompt], SamplingParams(max_tokens=4, ignore_eos=True))] == [4]
    assert own.why_done == "timeout" and not hurried.has_unfinished()
    # one prompt of a batch refused: nothing of the batch stays queued
    with pytest.raises(RequestRejected):
        hurried.generate([prompt, prompt[:4], []], SamplingParams(max_tokens=4))
    assert not hurried.has_unfinished() and not hurried.requests


def test_a_step_that_fails_ends_its_requests_and_gives_their_pages_back(model_dirs, monkeypatch):
    """A step that raises (here: forced from the host) leaves no request live with pages that nobody will ever
    free: the step's requests end with reason "error", the queue is untouched and served afterwards."""
    from tokenmill_amd import SamplingParams
    from tokenmill_amd.engine.runner import StepError
    eng = make_engine(model_dirs["A"], "float32", max_num_seqs=2)
    sp = SamplingParams(max_tokens=6, ignore_eos=True)
    prompts = [random_ids(n, 256, 60 + n) for n in (9, 20, 5)]
    want = make_engine(model_dirs["A"], "float32").generate([prompts[2]], sp)[0]
    reqs = [eng.add_request(f"r{i}", p, sp) for i, p in enumerate(prompts)]
    eng.step()
    eng.step()
    assert eng.num_running == 2 and eng.num_waiting == 1
    real_step = eng.runner.step

    def failing(entries):
        raise StepError("forced from the test")

    monkeypatch.setattr(eng.runner, "step", failing)
    with pytest.raises(StepError):
        eng.step()
    monkeypatch.setattr(eng.runner, "step", real_step)
    assert [r.why_done for r in reqs] == ["error", "error", None] and "forced from the test" in reqs[0].error
    assert eng.num_running == 0 and eng.num_waiting == 1 and eng.cache.num_free_pages == eng.cache.num_pages
    eng.cache.check_invariants()
    while eng.has_unfinished():
        eng.step()
    assert reqs[2].generated == want and eng.cache.num_free_pages == eng.cache.num_pages


def test_the_pool_is_sized_three_ways(model_dirs):
    """Pages as given; from a byte budget; or from what the card has left after the weights and the largest
    step, never more than `max_num_seqs` requests of `max_model_len` tokens can use (reference
    src/infer/engine/engine.py:44-84). Fewer than two pages is an error."""
    from tokenmill_amd import SamplingParams
    from tokenmill_amd.cache.pool import CachePools
    given = make_engine(model_dirs["A"], "float32", kv_cache_mb=None, num_blocks=11)
    assert given.cache.num_pages == 11
    per_page = CachePools.bytes_per_token(given.model, torch.float32) * 16
    assert per_page == 2 * 2 * 2 * 16 * 4 * 16               # K and V, 2 layers, 2 kv heads of 16, float32, 16 tokens
    budget = make_engine(model_dirs["A"], "float32", kv_cache_mb=1.0)
    assert budget.cache.num_pages == 2**20 // per_page
    auto = make_engine(model_dirs["A"], "bfloat16", kv_cache_mb=None, max_num_seqs=3, max_model_len=100,
                       max_num_batched_tokens=64, hip_graphs=True)
    assert auto.cache.num_pages == 3 * 7                      # the card has room for far more than the requests can use
    out = auto.generate([random_ids(9, 256, 90)], SamplingParams(max_tokens=5, ignore_eos=True))
    assert len(out[0]) == 5 and auto.cache.num_free_pages == auto.cache.num_pages
    with pytest.raises(RuntimeError, match="fewer than two pages"):
        make_engine(model_dirs["A"], "float32", kv_cache_mb=None, num_blocks=1)
    with pytest.raises(RuntimeError, match="fewer than two pages"):
        make_engine(model_dirs["A"], "float32", kv_cache_mb=per_page * 1.5 / 2**20)


def test_long_decoding_and_the_first_tokens_of_a_sequence(model_dirs, plains):
    """A 2-token prompt decoded for 230 tokens across many pages; and 1-token prompts."""
    from tokenmill_amd import SamplingParams
    for dtype_name in ("float32", "bfloat16"):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=8)
        prompts = [random_ids(2, 384, 80), [5], [0]]
        outs = eng.generate(prompts, [SamplingParams(max_tokens=230, ignore_eos=True),
                                      SamplingParams(max_tokens=3, ignore_eos=True),
                                      SamplingParams(max_tokens=3, ignore_eos=True)])
        assert len(outs[0]) == 230
        for p, o in zip(prompts, outs):
            verify(plains["B"], p, o, DTYPES[dtype_name])


def test_command_line(model_dirs, plains):
    r = subprocess.run([sys.executable, "-m", "tokenmill_amd.generate", "--model", str(model_dirs["A"]), "--dtype",
                        "float32", "--prompt-ids", "1,2,3;4,5", "--max-tokens", "6", "--ignore-eos",
                        "--kv-cache-mb", "4", "--max-model-len", "64", "--block-size", "8"],
                       capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert [ln["prompt_tokens"] for ln in lines] == [3, 2]
    verify(plains["A"], [1, 2, 3], lines[0]["output_ids"], torch.float32)
    verify(plains["A"], [4, 5], lines[1]["output_ids"], torch.float32)


def test_command_line_random_weights(model_dirs):
    """--random CONFIG: weights drawn on the device from --weights-seed; the same seed gives the same tokens,
    another seed another model. A shipped shape's name stands for its config.json."""
    def run(seed, source=None, more=()):
        r = subprocess.run([sys.executable, "-m", "tokenmill_amd.generate", "--random", source or str(model_dirs["B"]),
                            "--weights-seed", str(seed), "--prompt-lens", "9,4", "--max-tokens", "8", "--ignore-eos",
                            "--num-blocks", "16", "--max-model-len", "64", "--block-size", "8", *more],
                           capture_output=True, text=True, cwd=ROOT, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        return [json.loads(ln)["output_ids"] for ln in r.stdout.splitlines() if ln.startswith("{")]
    first, again, other = run(3), run(3), run(4)
    assert [len(o) for o in first] == [8, 8]
    assert first == again
    assert first != other
    assert run(3, more=("--hip-graphs", "--pipeline-decode")) == first     # replayed, each step queued ahead of the last one's tokens
    named = run(3, "tiny-a")
    by_path = run(3, str(ROOT / "tokenmill_amd" / "config" / "shapes" / "tiny-a.json"))
    assert [len(o) for o in named] == [8, 8] and named == by_path and named != first


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_hip_graphs(model_dirs, plains, dtype_name):
    """Graph replays between eager prefill steps, batch sizes that change as requests come and go:
    every replay gives what the eager engine gives."""
    from tokenmill_amd import SamplingParams
    lengths = [3, 30, 17, 9, 1, 40, 22]
    prompts = [random_ids(n, 384, 90 + i) for i, n in enumerate(lengths)]
    params = [SamplingParams(max_tokens=6 + 5 * i, ignore_eos=True) for i in range(len(lengths))]
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=16, hip_graphs=graphs, max_num_seqs=6,
                          max_num_batched_tokens=48)
        seqs = [eng.add_request(f"r{i}", p, sp) for i, (p, sp) in enumerate(zip(prompts[:4], params[:4]))]
        for _ in range(4):
            eng.step()
        seqs += [eng.add_request(f"r{i + 4}", p, sp) for i, (p, sp) in enumerate(zip(prompts[4:], params[4:]))]
        while eng.has_unfinished():
            eng.step()
        outs[graphs] = [s.generated for s in seqs]
        if graphs:
            assert eng.runner.graphs.replays > 20 and len(eng.runner.graphs.buckets) >= 3
        assert eng.cache.num_free_pages == eng.cache.num_pages
    for p, o in zip(prompts, outs[True]):
        verify(plains["B"], p, o, DTYPES[dtype_name])
    assert outs[True] == outs[False]


@pytest.mark.parametrize("portion", [16, 48])
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_prompt_portions_replayed_from_hip_graphs(model_dirs, plains, dtype_name, portion):
    """Long prompts cut into portions of 16 tokens (run as 32 rows, half of them padding: this library's
    own products) or 48 (run as 64 rows: the library products, which then are nodes of the graph), one
    request at a time: the second portion of a size captures a graph, the later ones (of this prompt and
    of the next prompts, at other positions and on other pages; the last, shorter portions too, which
    run with the same number of rows) replay it, with eager steps and synchronisations in between.
    Every replay must give what the eager engine gives, and what the plain implementation gives."""
    from tokenmill_amd import SamplingParams
    lengths = [100, 77, 33, 120] if portion == 16 else [200, 150, 97, 240]
    prompts = [random_ids(n, 384, 190 + i) for i, n in enumerate(lengths)]
    sp = SamplingParams(max_tokens=5, ignore_eos=True)
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=16, hip_graphs=graphs, max_num_seqs=2,
                          max_num_batched_tokens=portion, enable_chunked_prefill=True, max_model_len=256)
        outs[graphs] = [eng.generate([p], sp)[0] for p in prompts]
        if graphs:
            sg = eng.runner.step_graphs
            assert sg.replays >= (15 if portion == 16 else 8) and (sg.padded_rows(portion), 1, 0, 0) in sg.captured
        assert eng.cache.num_free_pages == eng.cache.num_pages
    for p, o in zip(prompts, outs[True]):
        verify(plains["B"], p, o, DTYPES[dtype_name])
    assert outs[True] == outs[False]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_prompts_of_similar_lengths_replay_one_graph(model_dirs, plains, dtype_name):
    """Whole prompts of many different lengths, one request at a time: a step runs with its rows padded to
    a few sizes, so lengths 17..32 share one graph and 33..64 another (padding rows carry token 0 without
    a cache slot, and repeated attention tiles fill the tile table). Tokens as from the eager engine and
    the plain implementation; a prompt of one token (a decode step) and the cache pages are untouched by
    the padding."""
    from tokenmill_amd import SamplingParams
    lengths = [19, 31, 17, 32, 40, 33, 64, 61, 1, 2, 47, 90, 5, 96, 70]
    prompts = [random_ids(n, 384, 500 + i) for i, n in enumerate(lengths)]
    sp = SamplingParams(max_tokens=4, ignore_eos=True)
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=8, hip_graphs=graphs, max_num_seqs=2,
                          max_num_batched_tokens=128, max_model_len=128)
        outs[graphs] = [eng.generate([p], sp)[0] for p in prompts]
        if graphs:
            sg = eng.runner.step_graphs
            assert set(sg.captured) == {(32, 1, 0, 1), (64, 1, 0, 1), (96, 1, 0, 1)} and sg.replays >= 9
        assert eng.cache.num_free_pages == eng.cache.num_pages
    for p, o in zip(prompts, outs[True]):
        verify(plains["B"], p, o, DTYPES[dtype_name])
    assert outs[True] == outs[False]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_mixed_steps_replayed_from_hip_graphs(model_dirs, plains, dtype_name):
    """Many requests at once with a small token budget: most steps hold portions of several prompts beside
    the decoded tokens of the running requests, in numbers that change from step to step. Such steps are
    laid out in a padded shape (rows, portions, single tokens and logit rows rounded up) and replayed from
    a few graphs; requests come and go, pages are handed out again. Tokens as from the eager engine and as
    the plain implementation gives them."""
    from tokenmill_amd import SamplingParams
    lengths = [1 + (11 * i) % 37 for i in range(40)]
    prompts = [random_ids(n, 384, 700 + i) for i, n in enumerate(lengths)]
    params = [SamplingParams(max_tokens=3 + i % 9, ignore_eos=True) for i in range(len(prompts))]
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=8, num_blocks=40, hip_graphs=graphs, max_num_seqs=6,
                          max_num_batched_tokens=24, enable_chunked_prefill=True, max_model_len=96)
        outs[graphs] = eng.generate(prompts, params)
        if graphs:
            sg = eng.runner.step_graphs
            assert sg.replays >= 20 and any(k[2] > 0 for k in sg.captured) and any(k[1] > 1 for k in sg.captured)
        assert eng.cache.num_free_pages == eng.cache.num_pages
    for p, o in zip(prompts, outs[True]):
        verify(plains["B"], p, o, DTYPES[dtype_name])
    assert outs[True] == outs[False]


def test_steps_run_kernel_by_kernel_when_a_capture_fails(model_dirs, plains, monkeypatch):
    """A capture that fails (out of memory for a graph's activations, in the field; forced from the host here)
    leaves its steps to the eager path: same tokens, the shape is not tried again, other shapes still replay."""
    from tokenmill_amd import SamplingParams
    from tokenmill_amd.engine import graphs as G
    prompts = [random_ids(n, 384, 800 + i) for i, n in enumerate([20, 19, 35, 18, 5, 40, 22])]
    sp = SamplingParams(max_tokens=6, ignore_eos=True)
    want = [make_engine(model_dirs["B"], "float32", block_size=8, max_num_seqs=2, max_model_len=96).generate([p], sp)[0]
            for p in prompts]
    decode_capture, step_capture = G.DecodeGraphs._capture, G.StepGraphs._capture

    def failing_decode(self, bk):
        if bk.B == 1:
            raise RuntimeError("out of memory (forced)")
        return decode_capture(self, bk)

    def failing_step(self, entries, key):
        if key[0] == 32:
            raise RuntimeError("out of memory (forced)")
        return step_capture(self, entries, key)

    monkeypatch.setattr(G.DecodeGraphs, "_capture", failing_decode)
    monkeypatch.setattr(G.StepGraphs, "_capture", failing_step)
    eng = make_engine(model_dirs["B"], "float32", block_size=8, hip_graphs=True, max_num_seqs=2, max_model_len=96)
    got = [eng.generate([p], sp)[0] for p in prompts]
    assert got == want
    assert eng.runner.graphs.failed == {1} and eng.runner.graphs.replays == 0
    assert eng.runner.step_graphs.failed == {(32, 1, 0, 1)} and (64, 1, 0, 1) in eng.runner.step_graphs.captured
    assert eng.cache.num_free_pages == eng.cache.num_pages


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_graphs_with_portions_and_a_starved_pool(model_dirs, plains, dtype_name):
    """Graph replays, prompt portions and evictions together: so few pages that requests lose theirs and are
    recomputed while decode steps and mixed steps replay from graphs. A decode graph keeps, per row of its
    batch, whose block table the row holds (only new pages are written); a request that comes back after an
    eviction has another table on other pages and must not find its old one there."""
    from tokenmill_amd import SamplingParams
    lengths = [9, 30, 17, 4, 26, 12, 21, 7, 33, 15, 2, 28]
    prompts = [random_ids(n, 384, 900 + i) for i, n in enumerate(lengths)]
    params = [SamplingParams(max_tokens=14 + 3 * (i % 5), ignore_eos=True) for i in range(len(prompts))]
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], dtype_name, block_size=4, kv_cache_mb=None, num_blocks=36,
                          hip_graphs=graphs, max_num_seqs=5, max_num_batched_tokens=16,
                          enable_chunked_prefill=True, max_model_len=96)
        outs[graphs] = eng.generate(prompts, params)
        assert eng.scheduler.evictions > 0, "the pool must be small enough to evict"
        eng.cache.check_invariants()
        assert eng.cache.num_free_pages == eng.cache.num_pages and not eng.scheduler.live
        if graphs:
            assert eng.runner.graphs.replays > 20 and eng.runner.step_graphs.replays > 0
    for p, o, sp in zip(prompts, outs[True], params):
        assert len(o) == sp.max_tokens
        verify(plains["B"], p, o, DTYPES[dtype_name])
    assert outs[True] == outs[False]


def test_decode_graphs_over_contexts_that_need_the_split_attention(model_dirs, plains):
    """max_model_len 1,024 makes the decode graphs launch the split attention (chunks of 256 keys merged
    afterwards), as every real run does; the contexts grow across 256 and 512 keys while they replay."""
    from tokenmill_amd import SamplingParams
    lengths = [250, 505, 30, 761]
    prompts = [random_ids(n, 384, 950 + i) for i, n in enumerate(lengths)]
    sp = SamplingParams(max_tokens=14, ignore_eos=True)
    outs = {}
    for graphs in (False, True):
        eng = make_engine(model_dirs["B"], "bfloat16", block_size=16, kv_cache_mb=16, hip_graphs=graphs,
                          max_num_seqs=4, max_num_batched_tokens=1024, max_model_len=1024)
        outs[graphs] = eng.generate(prompts, sp)
        if graphs:
            assert eng.runner.graphs.replays >= 12
        eng.cache.check_invariants()
        assert eng.cache.num_free_pages == eng.cache.num_pages
    for p, o in zip(prompts, outs[True]):
        verify(plains["B"], p, o, torch.bfloat16)
    assert outs[True] == outs[False]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_generation_with_peaked_attention_at_a_published_head_size(model_dirs, plains, dtype_name):
    """Configuration D (head size 64, seven query heads on one kv head, weights wide enough that a single
    key can carry a query): whole prompts and portions mixed with decodes, the pool so small that pages are
    handed out again."""
    from tokenmill_amd import SamplingParams
    prompts = [random_ids(n, 500, 970 + i) for i, n in enumerate([3, 70, 33, 18, 120, 47, 9, 64])]
    sp = SamplingParams(max_tokens=12, ignore_eos=True)
    dt = DTYPES[dtype_name]
    whole = make_engine(model_dirs["D"], dtype_name, max_num_seqs=8, kv_cache_mb=None, num_blocks=40)
    cut = make_engine(model_dirs["D"], dtype_name, max_num_seqs=4, kv_cache_mb=None, num_blocks=24,
                      enable_chunked_prefill=True, max_num_batched_tokens=20)
    flips = 0
    for eng in (whole, cut):
        for p, o in zip(prompts, eng.generate(prompts, sp)):
            flips += verify(plains["D"], p, o, dt)
        assert eng.cache.num_free_pages == eng.cache.num_pages
    assert flips == 0 or dtype_name == "bfloat16"       # (bfloat16: never more than the near-ties, checked by verify)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 8), ("D", 16)])
def test_operations_run_one_by_one_give_the_bits_of_one_run(model_dirs, name, page, dtype_name):
    """The step program runs consecutive operations of the library's in one call; a model with a part of
    another kind runs them in several calls with that part's own code in between. What crosses between two
    calls (the residual stream and the result still to be added to it) is all the state there is: the same
    steps run with one call per operation, and with every block's operations called through the parts' own
    `forward` (each part's one-operation program), give equal logits, bit for bit, over whole prompts,
    portions, single tokens and mixed steps with reused pages."""
    from tokenmill_amd.hip.program import _Foreign, _Native
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import make_requests, mixed, portions, prefill_then_decode, run_trace
    reqs = make_requests(name, [37, 64, 21, 90, 48, 33, 75, 18], 14)
    traces = prefill_then_decode(reqs) + portions(reqs) + mixed(reqs, seed=15)
    whole = ReplaySession(model_dirs[name], dtype_name, 4 * 128, page_size=page)
    single = ReplaySession(model_dirs[name], dtype_name, 4 * 128, page_size=page)
    blocks = ReplaySession(model_dirs[name], dtype_name, 4 * 128, page_size=page)
    program = single.runner.program
    assert [type(s) for s in program.steps] == [_Native] and program.steps[0].count == 2 + 2 * len(single.model.run)
    program.steps = [_Native(i, 1) for i in range(program.steps[0].count)]
    # the third: embedding and head stay operations, every block in between runs through Block.forward
    model, prog3 = blocks.model, blocks.runner.program
    n_ops = prog3.steps[0].count
    steps3 = [_Native(0, 1)]
    for j, call in enumerate(model.run):
        def run_block(flow, step, block=model.layers[call.layer], cache=blocks.pools.views[j]):
            flow.delta = block.forward(flow.resid, flow.delta, step, cache, model.dtype)
        steps3.append(_Foreign(model.layers[call.layer], run_block))
    steps3.append(_Native(n_ops - 1, 1))
    prog3.steps = steps3
    for rec in traces:
        a, b, c = whole.run_step(rec), single.run_step(rec), blocks.run_step(rec)
        assert (a is None) == (b is None) == (c is None)
        if a is not None:
            assert (a == b).all(), f"step {rec['step']} of {len(traces)}, one call per operation"
            assert (a == c).all(), f"step {rec['step']} of {len(traces)}, blocks through their own forward"
    assert whole.runner.program.runs == len(traces)


def test_engines_with_different_options_in_one_process(model_dirs, plains):
    """Four engines (float32 eager; bfloat16 with graphs and chunking; bfloat16 with graphs and no packed
    matrices; bfloat16 with graphs and the library's algorithms chosen by timing) stepped in turn give the
    tokens each gives alone: no option travels through state that the engines share (the kernel library, its
    plan cache and workspace, the graphs' pools). In particular an engine without timing keeps its bits beside
    one that times the same shapes of the same model (configuration D twice: the timed plans are kept apart)."""
    from tokenmill_amd import SamplingParams
    setups = [("A", "float32", dict(hip_graphs=False)),
              ("B", "bfloat16", dict(hip_graphs=True, enable_chunked_prefill=True, max_num_batched_tokens=64)),
              ("D", "bfloat16", dict(hip_graphs=True, pack_weights=False)),
              ("D", "bfloat16", dict(hip_graphs=True, pack_weights=False, tune_gemm=True))]
    prompts = {n: [random_ids(k, TINY[n][0]["vocab_size"], 50 + i) for i, k in enumerate((5, 33, 70, 17, 2, 48))] for n in "ABD"}
    sp = SamplingParams(max_tokens=20, ignore_eos=True)
    alone = [make_engine(model_dirs[n], dtype, max_num_seqs=8, **kw).generate(prompts[n], sp) for n, dtype, kw in setups[:3]]
    engines = [(n, make_engine(model_dirs[n], dtype, max_num_seqs=8, **kw)) for n, dtype, kw in setups]
    reqs = [[eng.add_request(f"{n}{i}", p, sp) for i, p in enumerate(prompts[n])] for n, eng in engines]
    while any(eng.has_unfinished() for _, eng in engines):
        for _, eng in engines:
            if eng.has_unfinished():
                eng.step()
    for k, (n, eng) in enumerate(engines):
        if k < 3:
            assert [r.generated for r in reqs[k]] == alone[k], n
        assert eng.cache.num_free_pages == eng.cache.num_pages
    assert engines[3][1].runner.program.tune and not engines[2][1].runner.program.tune
    for p, r in zip(prompts["D"], reqs[3]):                     # the timed engine's tokens are right by themselves
        verify(plains["D"], p, r.generated, torch.bfloat16)


def test_the_step_program_refuses_what_its_kernels_do_not_run(model_dirs):
    """The library's step program checks a step by itself (it is reached without the checks of the Python
    wrappers): a context beyond the rotary table, a block table narrower than the context, a layer group the
    step does not bring and a workspace that is too small are refused before the kernel that would read
    beyond them is launched."""
    import ctypes
    from tokenmill_amd.hip import abi
    from tokenmill_amd.engine.runner import StepEntry
    from tokenmill_amd.hip import ops
    from tokenmill_amd.replay import ReplaySession
    session = ReplaySession(model_dirs["A"], "bfloat16", 64)
    runner, program = session.runner, session.runner.program
    cache = session.manager.allocate("r", 20)
    step, _ = runner.prepare([StepEntry(cache, 0, random_ids(20, 256, 7), [19])])
    want = program.run(step).clone()
    assert torch.equal(program.run(step), want)                            # the step itself is fine, twice
    for field, value in (("max_context_len", 65), ("num_decode", 2)):
        saved = getattr(step, field)
        setattr(step, field, value)
        try:
            with pytest.raises((ops.KernelArgumentError, RuntimeError)):
                program.run(step)
        finally:
            setattr(step, field, saved)
    narrow = step.groups[0].block_tables
    step.groups[0].block_tables = narrow[:, :1]                            # one page of 16 for 20 positions
    with pytest.raises((ops.KernelArgumentError, RuntimeError)):
        program.run(step)
    step.groups[0].block_tables = narrow
    groups, step.groups = step.groups, []
    with pytest.raises((ops.KernelArgumentError, RuntimeError)):
        program.run(step)
    step.groups = groups
    # too small a workspace, straight at the entry point
    lib = program._lib
    s = abi.TmStep()
    s.T = s.max_context_len = 20
    s.S = s.R = 1
    s.num_groups = 1
    io = abi.TmStream()
    small = torch.empty(256, dtype=torch.uint8, device="cuda:0")
    resid = torch.empty((20, 64), device="cuda:0")
    io.resid, io.accumulate = resid.data_ptr(), 1
    rc = lib.tm_program_run(program._handle, 0, len(program.parts), ctypes.byref(s), ctypes.byref(io), small.data_ptr(), 256,
                            None, 0, None, 0, None)
    assert rc == 1
    for first, count in ((-1, 1), (0, 0), (1, len(program.parts))):      # operations the program does not have
        assert lib.tm_program_run(program._handle, first, count, ctypes.byref(s), ctypes.byref(io), small.data_ptr(), 256,
                                  None, 0, None, 0, None) == 1
    assert torch.equal(program.run(step), want)                            # and nothing of this broke the program
    session.manager.free(cache)



# ------------------------------------------------------------------------------------------------
# decode steps queued ahead of their tokens
# ------------------------------------------------------------------------------------------------

def _both(model_dir, dtype_name, run, **kw):
    """``run(engine)`` on an engine that reads every step's tokens before it plans the next, and on one that queues
    decode steps ahead; both results."""
    results = []
    for ahead in (False, True):
        eng = make_engine(model_dir, dtype_name, hip_graphs=True, pipeline_decode=ahead, **kw)
        results.append((run(eng), eng))
    return results


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_decode_steps_queued_ahead_give_the_same_tokens(model_dirs, plains, dtype_name):
    """With ``pipeline_decode`` the next decode step is queued behind the running one, its ids fed on the device:
    requests that end by length at different steps, pages crossed every 16 tokens, and requests that end at an
    end-of-sequence token after the step ahead of them was queued (their extra token is dropped): the same tokens
    as the engine that waits for every step, and they are the plain implementation's."""
    from tokenmill_amd import SamplingParams
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    prompts = [random_ids(n, 256, 300 + i) for i, n in enumerate((5, 17, 33, 30, 12))]
    limits = [3, 40, 64, 17, 50]

    def by_length(eng):
        return eng.generate(prompts, [SamplingParams(max_tokens=m, ignore_eos=True) for m in limits])

    (plain_out, waiting), (ahead_out, ahead) = _both(model_dirs["A"], dtype_name, by_length)
    assert ahead_out == plain_out and [len(o) for o in ahead_out] == limits
    assert ahead.stats["steps_ahead"] > 30 and waiting.stats["steps_ahead"] == 0
    for p, o in zip(prompts, ahead_out):
        verify(plains["A"], p, o, dt)
    # now one of those tokens ends requests: one that no request meets before its 7th token (by then the request with
    # three tokens is gone and steps are queued ahead) and some request meets well before its limit
    def first_met(tok):
        return min((o.index(tok) for o in ahead_out if tok in o), default=10 ** 6)
    stops = {next(o[j] for o, m in zip(ahead_out, limits) for j in range(6, m - 4) if first_met(o[j]) == j)}

    def by_stop_token(eng):
        eng.eos_ids = set(stops)
        return eng.generate(prompts, [SamplingParams(max_tokens=m) for m in limits])

    (plain_out, waiting), (ahead_out, ahead) = _both(model_dirs["A"], dtype_name, by_stop_token)
    assert ahead_out == plain_out
    assert any(o[-1] in stops and len(o) < m for o, m in zip(ahead_out, limits))
    assert ahead.stats["tokens_dropped"] > 0 and waiting.stats["tokens_dropped"] == 0, (ahead.stats, [len(o) for o in ahead_out])
    for eng in (waiting, ahead):
        eng.cache.check_invariants()
        assert eng.cache.num_free_pages == eng.cache.num_pages


def test_decode_steps_queued_ahead_with_sampling_arrivals_aborts_and_few_pages(model_dirs, plains):
    """The same with sampled tokens (the random number of a token is a function of the request's seed and the token's
    index, which the step ahead knows), with requests that arrive and are aborted while a step is in flight, with
    prompts cut into portions, and on a pool so small that requests are evicted: nothing is queued ahead where the
    next step is not simply the same requests one position on, and every request's tokens are as without it."""
    from tokenmill_amd import SamplingParams
    prompts = [random_ids(n, 256, 400 + i) for i, n in enumerate((9, 21, 40, 33, 14, 27))]
    sampled = [SamplingParams(max_tokens=24, temperature=0.8, top_k=40, top_p=0.9, seed=50 + i, ignore_eos=True)
               for i in range(len(prompts))]
    (a, _), (b, ahead) = _both(model_dirs["A"], "float32", lambda eng: eng.generate(prompts, sampled))
    assert a == b and ahead.stats["steps_ahead"] > 10
    for p, o, sp in zip(prompts, b, sampled):
        verify(plains["A"], p, o, torch.float32, sp, sp.seed)

    def arrivals_and_an_abort(eng):
        got: dict[str, list[int]] = {}
        sp = SamplingParams(max_tokens=30, ignore_eos=True)
        for i in range(3):
            eng.add_request(f"r{i}", prompts[i], sp)
        calls = 0
        while eng.has_unfinished():
            for o in eng.step():
                got.setdefault(o.request_id, []).extend(o.new_token_ids)
            calls += 1
            if calls == 6:
                eng.add_request("late", prompts[3], sp)
            if calls == 11:
                eng.abort_request("r1")
        got.pop("r1")                                  # ended at a call, not at a token: how far it got differs
        return got

    (a, _), (b, ahead) = _both(model_dirs["A"], "float32", arrivals_and_an_abort, enable_chunked_prefill=True,
                               max_num_batched_tokens=16)
    assert a == b and set(b) == {"r0", "r2", "late"} and all(len(t) == 30 for t in b.values())
    assert ahead.stats["steps_ahead"] > 10
    ahead.cache.check_invariants()
    assert ahead.cache.num_free_pages == ahead.cache.num_pages

    # more requests than slots: steps are queued ahead while the rest wait for a slot
    several = [SamplingParams(max_tokens=m, ignore_eos=True) for m in (20, 9, 31, 14, 25, 18)]
    for more in ({}, dict(enable_chunked_prefill=True, max_num_batched_tokens=24)):
        (a, _), (b, ahead) = _both(model_dirs["A"], "float32", lambda eng: eng.generate(prompts, several),
                                   max_num_seqs=3, **more)
        assert a == b and ahead.stats["steps_ahead"] > 20 and ahead.stats["peak_live"] == 3

    greedy = SamplingParams(max_tokens=40, ignore_eos=True)
    (a, waiting), (b, ahead) = _both(model_dirs["A"], "float32", lambda eng: eng.generate(prompts, greedy),
                                     kv_cache_mb=None, num_blocks=14)
    assert a == b and waiting.scheduler.evictions > 0 and ahead.scheduler.evictions > 0
    ahead.cache.check_invariants()
    assert ahead.cache.num_free_pages == ahead.cache.num_pages


def test_no_graph_is_destroyed_while_another_is_recorded(model_dirs):
    """An engine that was dropped frees nothing at once (it holds reference cycles); if Python's collector found it
    while a later engine records a graph, its graphs would be destroyed inside the recording, which HIP refuses from a
    destructor: the process would end. A recording therefore collects what is garbage before it starts and lets the
    collector rest until it ends."""
    import contextlib
    import gc
    import weakref
    from tokenmill_amd import SamplingParams
    from tokenmill_amd.engine import graphs as G
    sp = SamplingParams(max_tokens=6, ignore_eos=True)
    prompts = [random_ids(n, 256, 700 + i) for i, n in enumerate((5, 9))]
    gc.collect()
    gc.disable()
    try:
        first = make_engine(model_dirs["A"], "float32", hip_graphs=True)
        want = first.generate(prompts, sp)
        dropped = weakref.ref(next(iter(first.runner.graphs.buckets.values())).graph)
        del first                                   # no collection runs: what the engine holds in cycles stays
        gc.enable()
        second = make_engine(model_dirs["A"], "float32", hip_graphs=True)
        seen = []
        recording = G._recording

        @contextlib.contextmanager
        def watched(graph):
            with recording(graph):
                seen.append((dropped() is not None, gc.isenabled()))
                yield

        G._recording = watched
        try:
            assert second.generate(prompts, sp) == want
        finally:
            G._recording = recording
        assert seen and all(s == (False, False) for s in seen)    # the dropped graph is gone, the collector rests
        assert gc.isenabled()
    finally:
        gc.enable()

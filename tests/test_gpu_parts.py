"""Each part of a layer alone against the plain implementation, and the generality of their
assembly: architectures defined HERE, in the test, are registered, built, loaded and stepped
through the engine without a change to the framework's files:

  * a mixer with state of its own per request (a decayed running sum), beside attention layers;
  * layers that keep a window of keys beside layers that keep all, a layer that runs twice, and a
    layer that reads another layer's cache.

None of these is a model of anyone's; they exist to show what the parts' interfaces carry."""
from __future__ import annotations

import json
from dataclasses import dataclass

import pytest
import torch

from conftest import random_ids
from plain import qwen2_plain as P
from tolerances import assert_logits_close, assert_part_close, measured_noise

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=1e-5, atol=1e-5) if dt == torch.float32 else dict(rtol=1.6e-2, atol=1.2e-2)


def q(x, dt):
    return x.to(dt).float()


# ----------------------------------------------------------------------------------------------- helpers

class OneLayer:
    """The least a cache pool needs to know of a model: its cache specs and run list."""

    def __init__(self, mixer):
        from tokenmill_amd.models.decoder import LayerCall
        self._spec = mixer.cache_spec()
        self.run = [LayerCall(0)]

    def cache_specs(self):
        return [self._spec]


def step_for(mixer, dt, requests, page=16, pages=64):
    """Cache pools, manager and a step context for ``requests`` = [(start, n_tokens)], built with the
    engine's own runner (whose model is only asked for its device and vocabulary here)."""
    from tokenmill_amd.cache import CacheManager
    from tokenmill_amd.cache.pool import CachePools
    from tokenmill_amd.engine.runner import ModelRunner, StepEntry

    holder = OneLayer(mixer)
    pools = CachePools(holder, pages, page, 8, dt, DEV)
    manager = CacheManager(pools.windows, pages, page, 8)

    class Shell:
        device = torch.device(DEV)

        class head:
            vocab = 1 << 20

    runner = ModelRunner(Shell, pools, max_positions=4096)
    entries = []
    for i, (start, n) in enumerate(requests):
        rc = manager.allocate(f"r{i}", start + n)
        entries.append(StepEntry(rc, start, [0] * n, []))
    ctx, _ = runner.prepare(entries)
    return pools, ctx, entries


@pytest.mark.parametrize("dt", DTS)
def test_linear_part(dt):
    from tokenmill_amd.parts import Linear
    torch.manual_seed(0)
    lin = Linear(120, [48, 24, 24], ["a", "b", "c"], bias=True)
    specs = lin.tensor_specs("x.")
    assert specs["x.a.weight"].shape == (48, 120) and specs["x.c.bias"].shape == (24,)
    t = {n: q(torch.randn(s.shape) * 0.1, dt) for n, s in specs.items()}
    lin.load({n: v.to(dt).to(DEV) for n, v in t.items()}, "x.")
    for M in (3, 70):                                                   # few rows and many: different kernels
        x = q(torch.randn(M, 120), dt)
        got = lin.forward(x.to(dt).to(DEV)).float().cpu()
        want = torch.cat([P.linear(x, t[f"x.{n}.weight"], t[f"x.{n}.bias"], dt) for n in "abc"], dim=-1)
        torch.testing.assert_close(got, want, **tol(dt))
        resid = torch.randn(M, 96)                                      # the result added into a 32-bit residual
        acc = resid.to(DEV)
        if lin.forward(x.to(dt).to(DEV), accumulate_into=acc) is None:
            torch.testing.assert_close(acc.cpu(), resid + want, **tol(dt))


@pytest.mark.parametrize("dt", DTS)
def test_norm_part_and_lazy_input(dt):
    from tokenmill_amd.parts import NormedInput, RMSNorm, as_tensor
    torch.manual_seed(1)
    norm = RMSNorm(200, 3e-6)
    w = q(torch.rand(200) + 0.5, dt)
    norm.load({"n.weight": w.to(dt).to(DEV)}, "n.")
    resid, delta = torch.randn(5, 200) * 2, q(torch.randn(5, 200), dt)
    r = resid.to(DEV)
    x = NormedInput(norm, r, delta.to(dt).to(DEV), dt)
    assert x.fusable_rms() is None                                      # something is still to be added
    got = as_tensor(x)
    torch.testing.assert_close(got.float().cpu(), P.rms_norm(resid + delta, w, 3e-6, dt), **tol(dt))
    torch.testing.assert_close(r.cpu(), resid + delta, rtol=0, atol=0)  # the residual took the delta
    assert as_tensor(x) is got                                          # computed once
    y = NormedInput(norm, r, None, dt)
    assert y.fusable_rms() is not None and y.fusable_rms()[1] == 3e-6


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("rotary_dim", [32, 16])
def test_rotary_part(dt, rotary_dim):
    from tokenmill_amd.parts import GQAttention, RotaryEmbedding
    torch.manual_seed(2)
    H, KVH, D = 3, 1, 32
    rope = RotaryEmbedding(D, 5e4, 600, rotary_dim=rotary_dim)
    rope.build_tables(DEV)
    attn = GQAttention(64, H, KVH, D, D ** -0.5, rope)
    pools, ctx, _ = step_for(attn, dt, [(0, 7), (293, 2), (599, 1)])
    T = ctx.num_tokens
    qkv = q(torch.randn(T, (H + 2 * KVH) * D), dt)
    dev = qkv.to(dt).to(DEV)
    rope.encode_and_store(dev, H, KVH, D, ctx, pools.views[0])
    pos = ctx.positions.cpu().long()
    cos, sin = P.rope_tables(600, rotary_dim, 5e4)
    got = dev.float().cpu()
    for lo, n in ((0, H), (H * D, KVH)):
        x = qkv[:, lo:lo + n * D].view(T, n, D)
        want = x.clone()
        want[..., :rotary_dim] = P.apply_rope(x[..., :rotary_dim], cos, sin, pos, dt)      # the rest passes through
        torch.testing.assert_close(got[:, lo:lo + n * D].view(T, n, D), want, **tol(dt))
    slots = ctx.groups[0].slot_mapping.cpu().long()
    kflat = pools.views[0].k.float().cpu().view(-1, KVH, D)
    vflat = pools.views[0].v.float().cpu().permute(0, 3, 1, 2).reshape(-1, KVH, D)
    assert torch.equal(kflat[slots], got[:, H * D:(H + KVH) * D].view(T, KVH, D))
    assert torch.equal(vflat[slots], qkv[:, (H + KVH) * D:].view(T, KVH, D))
    with pytest.raises(ValueError, match="beyond the rotary table"):
        _, far, _ = step_for(attn, dt, [(600, 1)])
        rope.encode_and_store(dev[:1], H, KVH, D, far, pools.views[0])


def attention_tensors(hidden, H, KVH, D, dt, std=0.15):
    t = {"a.q_proj.weight": torch.randn(H * D, hidden) * std, "a.q_proj.bias": torch.randn(H * D) * 0.3,
         "a.k_proj.weight": torch.randn(KVH * D, hidden) * std, "a.k_proj.bias": torch.randn(KVH * D) * 0.3,
         "a.v_proj.weight": torch.randn(KVH * D, hidden) * std, "a.v_proj.bias": torch.randn(KVH * D) * 0.3,
         "a.o_proj.weight": torch.randn(hidden, H * D) * std}
    return {k: q(v, dt) for k, v in t.items()}


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,KVH,D,window", [(4, 2, 16, None), (6, 1, 32, None), (6, 3, 64, 9), (5, 5, 48, None)])
def test_attention_part_whole_then_portions_then_tokens(dt, H, KVH, D, window):
    """The mixer alone: a whole prompt in one call equals the plain attention block; the same
    prompt in portions and single tokens through the cache equals it too."""
    from tokenmill_amd.cache import CacheManager
    from tokenmill_amd.cache.pool import CachePools
    from tokenmill_amd.engine.runner import ModelRunner, StepEntry
    from tokenmill_amd.parts import GQAttention, RotaryEmbedding
    torch.manual_seed(3)
    hidden, L, theta = 96, 45, 1e4
    rope = RotaryEmbedding(D, theta, 128)
    attn = GQAttention(hidden, H, KVH, D, D ** -0.5, rope, window=window, names=("q_proj", "k_proj", "v_proj", "o_proj"))
    t = attention_tensors(hidden, H, KVH, D, dt)
    attn.load({k: v.to(dt).to(DEV) for k, v in t.items()}, "a.")
    attn.prepare(pack_weights=True)
    x = q(torch.randn(L, hidden), dt)
    cfg = {"heads": H, "kv_heads": KVH, "head_dim": D}
    cos, sin = P.rope_tables(L, D, theta)
    w = {k.replace("a.", "p."): v for k, v in t.items()}
    want = P.attention_block(x, w, "p.", cfg, torch.arange(L), cos, sin, dt, window)

    holder = OneLayer(attn)
    pools = CachePools(holder, 8, 16, 4, dt, DEV)
    manager = CacheManager(pools.windows, 8, 16, 4)

    class Shell:
        device = torch.device(DEV)

        class head:
            vocab = 10

    runner = ModelRunner(Shell, pools, max_positions=128)
    for cuts in ([L], [20, 2, 7, 1, 1, 1, 13]):
        rc = manager.allocate("r", 1)
        outs, start = [], 0
        for n in cuts:
            manager.append(rc, start + n)
            ctx, _ = runner.prepare([StepEntry(rc, start, [0] * n, [])])
            outs.append(attn.forward(x[start:start + n].to(dt).to(DEV), ctx, pools.views[0]).float().cpu())
            start += n
        manager.free(rc)
        assert_part_close(torch.cat(outs), want, dt, f"attention part, cuts {cuts}")


@pytest.mark.parametrize("dt", DTS)
def test_feed_forward_part(dt):
    from tokenmill_amd.parts import SwiGLU
    torch.manual_seed(4)
    hidden, inter = 120, 200
    ffn = SwiGLU(hidden, inter)
    t = {"m.gate_proj.weight": q(torch.randn(inter, hidden) * 0.2, dt),
         "m.up_proj.weight": q(torch.randn(inter, hidden) * 0.2, dt),
         "m.down_proj.weight": q(torch.randn(hidden, inter) * 0.2, dt)}
    assert set(ffn.tensor_specs("m.")) == set(t)
    ffn.load({k: v.to(dt).to(DEV) for k, v in t.items()}, "m.")
    ffn.prepare(pack_weights=True)
    for M in (4, 90):
        x = q(torch.randn(M, hidden), dt)
        got = ffn.forward(x.to(dt).to(DEV)).float().cpu()
        assert_part_close(got, P.mlp_block(x, t, "m.", dt), dt, f"feed-forward part, {M} rows")


@pytest.mark.parametrize("dt", DTS)
def test_embedding_and_tied_head_parts(dt):
    from tokenmill_amd.parts import OutputHead, TokenEmbedding
    torch.manual_seed(5)
    emb = TokenEmbedding(307, 120)
    table = q(torch.randn(307, 120), dt)
    emb.load({"e.weight": table.to(dt).to(DEV)}, "e.")
    head = OutputHead(120, 307, tied_to=emb)
    assert head.tensor_specs("") == {}
    head.load({}, "")
    assert head.proj.weight.data_ptr() == emb.weight.data_ptr()         # no second copy (reference tests/test_layers.py:90-93)
    ids = torch.tensor([5, 306, 0, 5], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(ids).cpu(), table[ids.cpu().long()])
    h = q(torch.randn(4, 120), dt)
    logits = head.forward(h.to(dt).to(DEV))
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), h @ table.t(), rtol=1e-4, atol=1e-3)
    untied = OutputHead(120, 307, tied_to=None)
    assert list(untied.tensor_specs("")) == ["lm_head.weight"]


# ----------------------------------------------------------------------------------------------- a mixer with state

@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    decay: float
    window: int
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw, generation=None):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["num_hidden_layers"], raw.get("decay", 0.9),
                   raw.get("window", 0))


def build_toy_state_model(cfg: ToyConfig, max_positions=None):
    """Layers alternate between a mixer with per-request state and grouped-query attention."""
    from tokenmill_amd.hip import ops
    from tokenmill_amd.models.decoder import DecoderModel
    from tokenmill_amd.parts import (GQAttention, Linear, Mixer, OutputHead, PreNormBlock, RMSNorm, RotaryEmbedding,
                                     StateSpec, SwiGLU, TokenEmbedding, as_tensor)

    class DecayedSumMixer(Mixer):
        """state_t = decay * state_{t-1} + x_t (32-bit, per request); out_t = proj(state_t). The state
        is advanced in token order inside a portion and carried from one step to the next."""

        def __init__(self, hidden, decay):
            self.hidden, self.decay = hidden, decay
            self.proj = Linear(hidden, hidden, "proj")

        def tensor_specs(self, prefix):
            return self.proj.tensor_specs(prefix)

        def load(self, tensors, prefix):
            self.proj.load(tensors, prefix)

        def cache_spec(self):
            return StateSpec((self.hidden,), torch.float32)

        def forward(self, x, step, cache, residual=None):
            x = as_tensor(x)
            if step.max_q_len == 1:
                # single tokens: index operations on the device alone, which a HIP graph can record (the
                # padding rows of a replayed step carry a slot that belongs to no request)
                slots = step.state_slots.long()
                state = cache.state.index_select(0, slots) * self.decay + x.float()
                cache.state.index_copy_(0, slots, state)
                return self.proj.forward(state.to(x.dtype))
            out = torch.empty_like(x)
            cu = step.cu_q_lens.tolist()
            slots = step.state_slots.tolist()
            for s in range(step.num_seqs):
                state = cache.state[slots[s]]
                for t in range(cu[s], cu[s + 1]):
                    state.mul_(self.decay).add_(x[t].float())
                    out[t] = state.to(x.dtype)
            return self.proj.forward(out)

    hidden = cfg.hidden_size
    n_pos = max_positions or 4096
    rope = RotaryEmbedding(16, 1e4, n_pos)
    emb = TokenEmbedding(cfg.vocab_size, hidden)
    layers = []
    for i in range(cfg.num_hidden_layers):
        mixer = DecayedSumMixer(hidden, cfg.decay) if i % 2 == 0 else \
            GQAttention(hidden, hidden // 16, 1, 16, 0.25, rope, qkv_bias=False)
        layers.append(PreNormBlock(RMSNorm(hidden, 1e-6), mixer, RMSNorm(hidden, 1e-6), SwiGLU(hidden, 2 * hidden)))
    return DecoderModel(cfg, emb, layers, RMSNorm(hidden, 1e-6), OutputHead(hidden, cfg.vocab_size, tied_to=emb))


def plain_toy_state_logits(w, cfg, ids, dt):
    """The same model with plain functions, whole sequence."""
    T, hidden = len(ids), cfg["hidden_size"]
    pos = torch.arange(T)
    cos, sin = P.rope_tables(T, 16, 1e4)
    x = P.rnd(w["model.embed_tokens.weight"], dt)[torch.tensor(ids)]
    acfg = {"heads": hidden // 16, "kv_heads": 1, "head_dim": 16}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6, dt)
        if i % 2 == 0:
            state = torch.zeros(hidden)
            mixed = torch.empty(T, hidden)
            for t in range(T):
                state = cfg["decay"] * state + h[t]
                mixed[t] = P.rnd(state, dt)
            x = x + P.linear(mixed, w[p + "self_attn.proj.weight"], None, dt)
        else:
            zero = {p + f"self_attn.{n}_proj.bias": torch.zeros(w[p + f"self_attn.{n}_proj.weight"].shape[0]) for n in "qkv"}
            x = x + P.attention_block(h, {**w, **zero}, p + "self_attn.", acfg, pos, cos, sin, dt)
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6, dt)
        x = x + P.mlp_block(h, w, p + "mlp.", dt)
    h = P.rms_norm(x, w["model.norm.weight"], 1e-6, dt)
    return P.linear(h, w["model.embed_tokens.weight"], None, dt, out_dt=torch.float32)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, dtype_name):
    from tokenmill_amd.config import register_architecture
    from tokenmill_amd.replay import ReplaySession
    from tokenmill_amd.weights import write_random_model
    from test_gpu_replay import mixed, portions, run_trace, whole

    register_architecture("ToyStateLM", ToyConfig.from_dict, build_toy_state_model, replace=True)
    cfg = {"architectures": ["ToyStateLM"], "vocab_size": 200, "hidden_size": 64, "num_hidden_layers": 4, "decay": 0.8}
    d = write_random_model(cfg, tmp_path / "toy", seed=3, std=0.06, norm_std=0.1)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    w = P.read_weights(d)
    session = ReplaySession(d, dtype_name, 4 * 128)
    assert len(session.pools.states) == 2 and len(session.pools.groups) == 1     # 2 state layers, 1 group of kv layers
    reqs = {f"r{i}": random_ids(n, 200, 300 + i) for i, n in enumerate([19, 40, 7, 33, 26, 50])}
    noise = measured_noise(lambda ids: plain_toy_state_logits(w, cfg, ids, torch.bfloat16), list(reqs.values())[:3])
    for name, steps in (("whole", whole(reqs)), ("portions", portions(reqs)), ("mixed", mixed(reqs, seed=8))):
        got = run_trace(session, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        for (rid, p), row in got.items():
            want = plain_toy_state_logits(w, cfg, reqs[rid], dt)[p]
            assert_logits_close(row, want, dt, f"toy state model, {name}, {rid} position {p}", noise)
        session.manager.check_invariants()
        assert not session.manager.live
    # through the engine: the decode steps of a model with per-request state replay from graphs like any
    # other's (this mixer's single-token path is capturable), with requests coming and going in the batch;
    # a mixer that does not say so turns the graphs off for its model, loudly, and the tokens are the same
    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams
    prompts = [random_ids(n, 200, 350 + i) for i, n in enumerate([12, 3, 30, 7, 21, 16, 9, 25, 5, 18])]
    params = [SamplingParams(max_tokens=6 + 3 * (i % 4), ignore_eos=True) for i in range(len(prompts))]
    outs = {}
    for mode in ("eager", "graphs", "ahead", "refused"):
        eng = LLMEngine(EngineConfig(model=str(d), dtype=dtype_name, block_size=8, num_blocks=64, max_model_len=64,
                                     max_num_seqs=4, max_num_batched_tokens=64, watermark=0.0, hip_graphs=mode != "eager",
                                     pipeline_decode=mode == "ahead"))
        # the mixer with state runs through its own code, between the library's operations: two hops a step, not the model
        assert [type(p).__name__ for p in eng.runner.program.foreign_parts] == ["DecayedSumMixer"] * 2
        assert len(eng.runner.program.parts) == 2 + 2 + 4      # embedding, head, two attentions, four feed-forwards
        if mode == "refused":
            for layer in eng.model.layers[::2]:
                layer.mixer.capturable = False
            from tokenmill_amd.engine.graphs import DecodeGraphs
            eng.runner.graphs = DecodeGraphs(eng.runner, eng.cfg)
            assert not eng.runner.graphs.stateful_ok
        outs[mode] = eng.generate(prompts, params)
        if mode in ("graphs", "ahead"):
            assert eng.runner.graphs.replays > 10
        # decode steps queued ahead of the running step's tokens advance every live request's state once a step too
        assert (eng.stats["steps_ahead"] > 5) == (mode == "ahead")
        if mode == "refused":
            assert eng.runner.graphs.replays == 0
        assert eng.cache.num_free_pages == eng.cache.num_pages
    assert outs["graphs"] == outs["eager"] == outs["refused"] == outs["ahead"]


# ----------------------------------------------------------------------------------------------- windows, a layer twice, a shared cache

def build_toy_window_model(cfg: ToyConfig, max_positions=None):
    """Four run calls over three layers: layer 0 keeps every key; layer 1 keeps a window; layer 0 runs
    again with a cache of its own; layer 2 has no k/v use of its own weights' cache: it reads the
    cache the first call wrote."""
    from tokenmill_amd.models.decoder import DecoderModel, LayerCall
    from tokenmill_amd.parts import (GQAttention, OutputHead, PreNormBlock, RMSNorm, RotaryEmbedding, SwiGLU,
                                     TokenEmbedding)
    hidden = cfg.hidden_size
    rope = RotaryEmbedding(32, 1e5, max_positions or 4096)
    emb = TokenEmbedding(cfg.vocab_size, hidden)

    def block(window):
        return PreNormBlock(RMSNorm(hidden, 1e-5), GQAttention(hidden, 4, 2, 32, 32 ** -0.5, rope, window=window),
                            RMSNorm(hidden, 1e-5), SwiGLU(hidden, 160))

    layers = [block(None), block(cfg.window), block(None)]
    run = [LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(2, cache_of=0)]
    return DecoderModel(cfg, emb, layers, RMSNorm(hidden, 1e-5), OutputHead(hidden, cfg.vocab_size, tied_to=None), run=run)


def plain_toy_window_logits(w, cfg, ids, dt):
    T = len(ids)
    pos = torch.arange(T)
    cos, sin = P.rope_tables(T, 32, 1e5)
    acfg = {"heads": 4, "kv_heads": 2, "head_dim": 32, "eps": 1e-5}
    x = P.rnd(w["model.embed_tokens.weight"], dt)[torch.tensor(ids)]
    kv_of_first = None
    for call, (layer, window, shared) in enumerate([(0, None, False), (1, cfg["window"], False), (0, None, False),
                                                    (2, None, True)]):
        p = f"model.layers.{layer}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-5, dt)
        a = p + "self_attn."
        qq = P.apply_rope(P.linear(h, w[a + "q_proj.weight"], w[a + "q_proj.bias"], dt).view(T, 4, 32), cos, sin, pos, dt)
        if shared:                                   # reads the keys and values the first call cached
            kk, vv = kv_of_first
        else:
            kk = P.apply_rope(P.linear(h, w[a + "k_proj.weight"], w[a + "k_proj.bias"], dt).view(T, 2, 32), cos, sin, pos, dt)
            vv = P.linear(h, w[a + "v_proj.weight"], w[a + "v_proj.bias"], dt).view(T, 2, 32)
            if call == 0:
                kv_of_first = (kk, vv)
        att = P.causal_attention(qq, kk, vv, 32 ** -0.5, dt, window)
        x = x + P.linear(att.reshape(T, 128), w[a + "o_proj.weight"], None, dt)
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5, dt)
        x = x + P.mlp_block(h, w, p + "mlp.", dt)
    h = P.rms_norm(x, w["model.norm.weight"], 1e-5, dt)
    return P.linear(h, w["lm_head.weight"], None, dt, out_dt=torch.float32)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_window_groups_a_layer_twice_and_a_shared_cache(tmp_path, dtype_name):
    from tokenmill_amd.config import register_architecture
    from tokenmill_amd.replay import ReplaySession
    from tokenmill_amd.weights import write_random_model
    from test_gpu_replay import mixed, portions, prefill_then_decode, run_trace

    register_architecture("ToyWindowLM", ToyConfig.from_dict, build_toy_window_model, replace=True)
    cfg = {"architectures": ["ToyWindowLM"], "vocab_size": 150, "hidden_size": 96, "num_hidden_layers": 3, "window": 21}
    # spread 0.04: the plain implementation's own bfloat16-vs-float32 difference is then 0.8 % of the logits' scale
    # (1.9 % at 0.08, 4.3 % at 0.12: four calls through peaked attention amplify every rounding)
    d = write_random_model(cfg, tmp_path / "toyw", seed=4, std=0.04, norm_std=0.1)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    w = P.read_weights(d)
    session = ReplaySession(d, dtype_name, 4 * 128)
    assert [g.window for g in session.pools.groups] == [None, 21]       # two groups, pages of their own
    assert session.pools.k[0].shape[0] == 2 and session.pools.k[1].shape[0] == 1    # 2 + 1 cache layers for 4 calls
    reqs = {f"r{i}": random_ids(n, 150, 400 + i) for i, n in enumerate([90, 35, 64, 50, 77])}
    noise = measured_noise(lambda ids: plain_toy_window_logits(w, cfg, ids, torch.bfloat16), list(reqs.values())[:3])
    for name, steps in (("prefill+decode", prefill_then_decode(reqs)), ("portions", portions(reqs)),
                        ("mixed", mixed(reqs, seed=9))):
        freed_early = 0
        got = {}
        for rec in steps:
            before = session.manager.allocators[1].num_free
            got.update(run_trace(session, [rec]))
            live_pages = sum(sum(p >= 0 for p in rc.tables[1]) for rc in session.manager.live.values())
            assert session.manager.allocators[1].num_free + live_pages == session.num_pages
            freed_early += any(-1 in rc.tables[1] for rc in session.manager.live.values())
        assert freed_early > 0, "the windowed group must give pages back while requests still run"
        for (rid, p), row in got.items():
            want = plain_toy_window_logits(w, cfg, reqs[rid], dt)[p]
            assert_logits_close(row, want, dt, f"toy window model, {name}, {rid} position {p}", noise)
        session.manager.check_invariants()
        assert not session.manager.live and all(a.num_free == session.num_pages for a in session.manager.allocators)
    # through the engine: decode steps and mixed steps replayed from graphs give the eager engine's tokens,
    # with pages of the windowed group handed back under way
    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams
    prompts = [random_ids(n, 150, 450 + i) for i, n in enumerate([40, 3, 27, 55, 18, 33] * 4)]
    outs = {}
    for graphs in (False, True):
        eng = LLMEngine(EngineConfig(model=str(d), dtype=dtype_name, block_size=8, num_blocks=64, max_model_len=128,
                                     max_num_seqs=4, max_num_batched_tokens=24, enable_chunked_prefill=True,
                                     watermark=0.0, hip_graphs=graphs))
        outs[graphs] = eng.generate(prompts, SamplingParams(max_tokens=24, ignore_eos=True))
        if graphs:
            assert eng.runner.graphs.replays > 0 and eng.runner.step_graphs.replays > 0
        assert eng.cache.num_free_pages == eng.cache.num_pages
    assert outs[True] == outs[False]


# ----------------------------------------------------------------------------------------------- routed experts, another position encoding

@dataclass(frozen=True)
class ToyRoutedConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_experts: int
    max_positions: int
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw, generation=None):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["num_hidden_layers"], raw["num_experts"],
                   raw["max_positions"])


ROUTED_HEADS, ROUTED_KV_HEADS, ROUTED_D, ROUTED_I = 3, 1, 32, 96


def plant_routing_signal(model_dir, num_experts, amplitude=1.5, gain=2.0):
    """Random router weights decide hundreds of tokens by margins that a rounding difference can flip,
    and a flipped token gets another expert's output: no tolerance would be the right one. So the
    decision is planted: channels 0 and 1 of every token's embedding hold one of `num_experts`
    directions (by token id), and the routers read those two channels. The attention in between
    moves them by far less than the angle between two directions, so engine and plain implementation
    route alike, while every expert is used and the other 78 channels carry the random signal."""
    import math

    from safetensors.torch import load_file, save_file
    path = str(model_dir / "model.safetensors")
    tensors = load_file(path)
    angle = [2 * math.pi * e / num_experts for e in range(num_experts)]
    emb = tensors["model.embed_tokens.weight"]
    ids = torch.arange(emb.shape[0])
    emb[:, 0] = (amplitude * torch.tensor([math.cos(a) for a in angle]))[ids % num_experts].to(emb.dtype)
    emb[:, 1] = (amplitude * torch.tensor([math.sin(a) for a in angle]))[ids % num_experts].to(emb.dtype)
    for name, t in tensors.items():
        if name.endswith("mlp.router.weight"):
            t.zero_()
            t[:, 0] = gain * torch.tensor([math.cos(a) for a in angle]).to(t.dtype)
            t[:, 1] = gain * torch.tensor([math.sin(a) for a in angle]).to(t.dtype)
    save_file(tensors, path)


def build_toy_routed_model(cfg: ToyRoutedConfig, max_positions=None):
    """Attention whose position encoding is a learned table added to q and k, and a feed-forward that
    sends every token to one of several experts: both defined here, outside the framework."""
    from tokenmill_amd.hip import ops
    from tokenmill_amd.models.decoder import DecoderModel
    from tokenmill_amd.parts import (FeedForward, GQAttention, Linear, OutputHead, PositionEncoding, PreNormBlock,
                                     RMSNorm, SwiGLU, TokenEmbedding, as_tensor)
    from tokenmill_amd.weights.loader import TensorSpec

    class AddedPositions(PositionEncoding):
        """q and k of every head get the row of their position from a learned [positions, D] table."""

        def __init__(self, head_dim, positions):
            self.head_dim, self.positions = head_dim, positions
            self.table = None

        def tensor_specs(self, prefix):
            return {prefix + "pos_table.weight": TensorSpec((self.positions, self.head_dim))}

        def load(self, tensors, prefix):
            self.table = tensors[prefix + "pos_table.weight"]

        def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, step, cache):
            rows = self.table[step.positions.long()].float()                       # [T, D]
            n = (num_heads + num_kv_heads) * head_dim
            qk = qkv[:, :n].view(-1, num_heads + num_kv_heads, head_dim)
            qk.copy_((qk.float() + rows[:, None, :]).to(qkv.dtype))
            if cache is not None and cache.write:                                  # store k and v as they now are
                ops.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, None, None, None,
                                  step.groups[cache.group].slot_mapping, cache.k, cache.v)

    class TopOneExperts(FeedForward):
        """Router logits in 32-bit; a token goes to the expert with the largest logit and its output is
        weighted by that expert's softmax probability."""

        def __init__(self, hidden, intermediate, num_experts):
            self.router = Linear(hidden, num_experts, "router")
            self.experts = [SwiGLU(hidden, intermediate) for _ in range(num_experts)]

        def _parts(self, prefix):
            return [(self.router, prefix)] + [(e, prefix + f"experts.{i}.") for i, e in enumerate(self.experts)]

        def tensor_specs(self, prefix):
            specs = {}
            for part, p in self._parts(prefix):
                specs.update(part.tensor_specs(p))
            return specs

        def load(self, tensors, prefix):
            for part, p in self._parts(prefix):
                part.load(tensors, p)

        def prepare(self, pack_weights):
            for expert in self.experts:
                expert.prepare(pack_weights)

        def forward(self, x, step, residual=None):
            x = as_tensor(x)
            probs = torch.softmax(self.router.forward(x, out_dtype=torch.float32), dim=-1)
            weight, choice = probs.max(dim=-1)
            out = torch.zeros_like(x)
            for e, expert in enumerate(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    y = expert.forward(x[rows].contiguous(), step)
                    out[rows] = (weight[rows, None] * y.float()).to(x.dtype)
            return out

    hidden = cfg.hidden_size
    emb = TokenEmbedding(cfg.vocab_size, hidden)
    layers = []
    for i in range(cfg.num_hidden_layers):
        attention = GQAttention(hidden, ROUTED_HEADS, ROUTED_KV_HEADS, ROUTED_D, ROUTED_D ** -0.5,
                                AddedPositions(ROUTED_D, cfg.max_positions), qkv_bias=False)
        ffn = TopOneExperts(hidden, ROUTED_I, cfg.num_experts) if i % 2 == 0 else SwiGLU(hidden, ROUTED_I)
        layers.append(PreNormBlock(RMSNorm(hidden, 1e-6), attention, RMSNorm(hidden, 1e-6), ffn))
    return DecoderModel(cfg, emb, layers, RMSNorm(hidden, 1e-6), OutputHead(hidden, cfg.vocab_size, tied_to=None))


def plain_toy_routed_logits(w, cfg, ids, dt):
    """The same model with plain functions, whole sequence. Also returns the smallest gap between the
    two largest router probabilities of any token (the test wants it wide: see plant_routing_signal)
    and which experts were used."""
    T, hidden = len(ids), cfg["hidden_size"]
    H, KVH, D = ROUTED_HEADS, ROUTED_KV_HEADS, ROUTED_D
    x = P.rnd(w["model.embed_tokens.weight"], dt)[torch.tensor(ids)]
    margin = 1.0
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = p + "self_attn."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6, dt)
        rows = P.rnd(w[a + "pos_table.weight"], dt)[:T]
        qq = P.rnd(P.linear(h, w[a + "q_proj.weight"], None, dt).view(T, H, D) + rows[:, None, :], dt)
        kk = P.rnd(P.linear(h, w[a + "k_proj.weight"], None, dt).view(T, KVH, D) + rows[:, None, :], dt)
        vv = P.linear(h, w[a + "v_proj.weight"], None, dt).view(T, KVH, D)
        att = P.causal_attention(qq, kk, vv, D ** -0.5, dt)
        x = x + P.linear(att.reshape(T, H * D), w[a + "o_proj.weight"], None, dt)
        h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6, dt)
        m = p + "mlp."
        if i % 2 == 0:
            probs = torch.softmax(P.linear(h, w[m + "router.weight"], None, dt, out_dt=torch.float32), dim=-1)
            top2 = probs.topk(2, dim=-1).values
            margin = min(margin, float((top2[:, 0] - top2[:, 1]).min()))
            weight, choice = probs.max(dim=-1)
            delta = torch.zeros(T, hidden)
            for t in range(T):
                y = P.mlp_block(h[t:t + 1], w, m + f"experts.{int(choice[t])}.", dt)
                delta[t] = P.rnd(weight[t] * y[0], dt)
            x = x + delta
        else:
            x = x + P.mlp_block(h, w, m, dt)
    h = P.rms_norm(x, w["model.norm.weight"], 1e-6, dt)
    return P.linear(h, w["lm_head.weight"], None, dt, out_dt=torch.float32), margin


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_routed_experts_and_added_positions_are_registered_built_and_stepped(tmp_path, dtype_name):
    """A feed-forward with routing and another position encoding, both defined in this file, go through
    registry, random weights, loader, cache manager, step function and replay unchanged; the positions
    enter only through the table, so cutting a request anywhere must give the same logits."""
    from tokenmill_amd.config import register_architecture
    from tokenmill_amd.replay import ReplaySession
    from tokenmill_amd.weights import write_random_model
    from test_gpu_replay import mixed, portions, prefill_then_decode, run_trace

    register_architecture("ToyRoutedLM", ToyRoutedConfig.from_dict, build_toy_routed_model, replace=True)
    cfg = {"architectures": ["ToyRoutedLM"], "vocab_size": 180, "hidden_size": 80, "num_hidden_layers": 3,
           "num_experts": 3, "max_positions": 128}
    d = write_random_model(cfg, tmp_path / "toyr", seed=5, std=0.05, norm_std=0.1)
    plant_routing_signal(d, 3)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    w = P.read_weights(d)
    assert sum("experts." in k for k in w) == 2 * 3 * 3 and "model.layers.0.self_attn.pos_table.weight" in w
    session = ReplaySession(d, dtype_name, 4 * 128)
    reqs = {f"r{i}": random_ids(n, 180, 500 + i) for i, n in enumerate([60, 35, 47, 90, 21])}
    noise = measured_noise(lambda ids: plain_toy_routed_logits(w, cfg, ids, torch.bfloat16)[0], list(reqs.values())[:3])
    want = {}
    for rid, ids in reqs.items():
        want[rid], margin = plain_toy_routed_logits(w, cfg, ids, dt)
        assert margin > 0.5, f"{rid}: a router decision is too close to call ({margin})"
    for name, steps in (("prefill+decode", prefill_then_decode(reqs)), ("portions", portions(reqs)),
                        ("mixed", mixed(reqs, seed=10))):
        got = run_trace(session, steps)
        assert len(got) == sum(len(v) for v in reqs.values()) or name == "prefill+decode"
        for (rid, p), row in got.items():
            assert_logits_close(row, want[rid][p], dt, f"toy routed model, {name}, {rid} position {p}", noise)
        session.manager.check_invariants()
        assert not session.manager.live

"""HIP graphs for decode steps, and for prompt portions of a repeated length.

A step in which every request decodes one token launches the same kernels with the same grids
whatever the requests are, once the batch is padded to a bucket size and the block tables to the
width of the longest request the engine allows. Such a step is captured once per bucket and then
replayed: one graph launch instead of a few hundred kernel launches from the host. (The reference
has the same device for the same reason: reference src/infer/engine/cuda_graphs.py:88-115, and its
profile of where an eager decode step's time goes, bench/results/profile/decode_breakdown_b32.json.)

Padding rows carry token 0 at position 0, a context of one key, and cache slot -1, which the cache
write skips; their logits are never looked at. The graphs hold no memset node.

A step that holds prompt portions, alone or beside single tokens, launches the same kernels with the
same grids as any other step of its padded shape (positions, pages and tiles are data), so the equal
portions of a long prompt, prompts of similar lengths arriving one after the other, and the mixed
steps of a serving run replay a handful of graphs: ``StepGraphs``.
"""
from __future__ import annotations

import contextlib
import gc
import logging

import numpy as np
import torch

from tokenmill_amd.cache.manager import RELEASED
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import GroupStep, StepContext

log = logging.getLogger(__name__)


@contextlib.contextmanager
def _recording(graph: torch.cuda.CUDAGraph):
    """``torch.cuda.graph(graph)`` during which nothing is destroyed. While a stream records, HIP refuses to
    destroy a graph; Python's collector runs whenever enough objects have been made, and if it then finds an engine
    that was dropped earlier (engines hold reference cycles, so dropping one frees nothing at once), that engine's
    graphs are destroyed in the middle of the recording: an error inside a destructor, which ends the process.
    So what is garbage is collected before the recording starts, and the collector rests until it ends."""
    gc.collect()
    resting = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if resting:
            gc.enable()


class _Bucket:
    def __init__(self, runner, B: int, W: int):
        self.B, self.W = B, W
        n_groups = len(runner.pools.groups)
        self.n_ints = 3 * B + (B + 1) + 3 * B + n_groups * (B + B * W)
        self.pinned = torch.zeros(self.n_ints, dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(self.n_ints, dtype=torch.int32, device=runner.device)
        off = 0

        def take(n):
            nonlocal off
            span = (off, off + n)
            off += n
            return span

        self.ids, self.pos, self.seq_of = take(B), take(B), take(B)
        self.cu, self.ctx, self.state, self.rows = take(B + 1), take(B), take(B), take(B)
        self.g_slot = [take(B) for _ in range(n_groups)]
        self.g_tab = [take(B * W) for _ in range(n_groups)]
        host = self.pinned.numpy()
        host[self.seq_of[0]:self.seq_of[1]] = np.arange(B)
        host[self.cu[0]:self.cu[1]] = np.arange(B + 1)
        host[self.rows[0]:self.rows[1]] = np.arange(B)
        self.rows_held: list[list] = [[None] * B for _ in range(n_groups)]   # whose table each row holds
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits: torch.Tensor | None = None

    def view(self, span):
        return self.dev[span[0]:span[1]]

    def context(self, max_positions: int) -> StepContext:
        B, W = self.B, self.W
        groups = [GroupStep(block_tables=self.view(t).view(B, W), slot_mapping=self.view(s))
                  for s, t in zip(self.g_slot, self.g_tab)]
        return StepContext(num_tokens=B, num_seqs=B, token_ids=self.view(self.ids), positions=self.view(self.pos),
                           seq_of_token=self.view(self.seq_of), cu_q_lens=self.view(self.cu),
                           context_lens=self.view(self.ctx), state_slots=self.view(self.state),
                           logit_rows=self.view(self.rows), groups=groups, q_lens=[1] * B, start_positions=[0] * B,
                           max_q_len=1, max_context_len=max_positions, num_logit_rows=B, num_decode=B,
                           max_decode_context=max_positions)


class DecodeGraphs:
    def __init__(self, runner, cfg, max_batch: int = 256):
        self.runner = runner
        ops.library_workspace(runner.device)      # made now: a capture must not allocate it
        self.page = runner.page_size
        self.max_positions = runner.max_positions
        self.W = -(-runner.max_positions // self.page)
        top = min(cfg.max_num_seqs, max_batch)
        # batch sizes a step is padded to: powers of two and the sizes in between from 16 on (48 keeps 33 to 48
        # requests on the products that hold the input in LDS, which 64 rows leave)
        self.sizes = [b for b in (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256) if b < top] + [top]
        self.buckets: dict[int, _Bucket] = {}
        self.failed: set[int] = set()                       # bucket sizes whose capture failed: those steps run eagerly
        self.replays = 0
        self._copied = torch.cuda.Event()
        # A model with per-request state replays its decode steps too (the slot of each row is data like its
        # block table; a row of padding updates a slot that belongs to nobody), if its mixers say that they
        # can be recorded. Otherwise every step of it runs kernel by kernel, and that is said once, here.
        model = runner.model
        holders = [model.layers[call.layer].mixer for j, call in enumerate(model.run) if j in runner.pools.states]
        refusing = [type(m).__name__ for m in holders if not getattr(m, "capturable", False)]
        self.stateful_ok = not refusing
        if refusing:
            log.warning("HIP graphs are off for this model: %s keeps per-request state and does not declare itself "
                        "capturable; its steps are launched kernel by kernel", ", ".join(sorted(set(refusing))))

    def can_run(self, entries) -> bool:
        return 0 < len(entries) <= self.sizes[-1] and all(len(e.tokens) == 1 for e in entries) and self.stateful_ok

    def _bucket(self, n: int) -> _Bucket:
        B = next(b for b in self.sizes if b >= n)
        if B not in self.buckets:
            self.buckets[B] = _Bucket(self.runner, B, self.W)
        return self.buckets[B]

    @torch.inference_mode()
    def run(self, entries, ids_from: torch.Tensor | None = None) -> torch.Tensor | None:
        """Float32 logits [wanted, vocab], entries in the given order (each wants place 0 or nothing); None
        if the graph of this batch size could not be captured (the caller then runs the step kernel by
        kernel, as the reference does when it runs out of memory for graphs: reference
        src/infer/engine/cuda_graphs.py:88-110). With ``ids_from`` (int32 on the device, one id per entry) the
        entries' tokens are taken from there, in stream order, instead of from the entries: the step before this
        one may still be running, and what it samples goes into this one without a trip to the host."""
        runner = self.runner
        bk = self._bucket(len(entries))
        B, W, page = bk.B, bk.W, self.page
        self._copied.synchronize()                          # the last replay's copy has left the pinned buffer
        host = bk.pinned.numpy()
        n = len(entries)
        ids = np.zeros(B, dtype=np.int64)
        pos = np.zeros(B, dtype=np.int64)
        ids[:n] = [e.tokens[0] for e in entries]
        pos[:n] = [e.start for e in entries]
        if ids.min() < 0 or ids.max() >= runner.vocab:
            raise ValueError("a token id is outside the vocabulary")
        if pos.max() >= self.max_positions:
            raise ValueError(f"a position exceeds the model's {self.max_positions}")
        host[bk.ids[0]:bk.ids[1]] = ids
        host[bk.pos[0]:bk.pos[1]] = pos
        ctx = pos + 1
        ctx[n:] = 1
        host[bk.ctx[0]:bk.ctx[1]] = ctx
        state = host[bk.state[0]:bk.state[1]]
        state[:] = runner.pools.padding_state_slot
        state[:n] = [e.cache.state_slot for e in entries]
        for g in range(len(runner.pools.groups)):
            slots = host[bk.g_slot[g][0]:bk.g_slot[g][1]]
            tabs = host[bk.g_tab[g][0]:bk.g_tab[g][1]].reshape(B, W)
            slots[:] = -1
            windowed = runner.pools.groups[g].window is not None
            rows = bk.rows_held[g]
            new_slots = []
            for i, e in enumerate(entries):
                table = e.cache.tables[g]
                need = e.start // page + 1
                if len(table) < need or table[need - 1] == RELEASED:
                    raise ValueError(f"{e.cache.request_id}: no page for position {e.start}")
                # a row that held this request's table last time only needs its new pages
                held = rows[i]
                have = held[1] if (held is not None and held[0] is e.cache and not windowed and held[1] <= need) else 0
                if have < need:
                    row = np.asarray(table[have:need], dtype=np.int64)
                    tabs[i, have:need] = np.where(row == RELEASED, 0, row)
                rows[i] = (e.cache, need)
                new_slots.append(table[need - 1] * page + e.start % page)
            slots[:n] = new_slots
            for i in range(n, B):
                rows[i] = None
        bk.dev.copy_(bk.pinned, non_blocking=True)
        self._copied.record()
        if ids_from is not None:
            bk.view(bk.ids)[:n].copy_(ids_from[:n])
        if bk.graph is None:
            if bk.B in self.failed:
                return None
            try:
                self._capture(bk)
            except RuntimeError as e:                       # out of memory for the graph's activations, mostly
                self.failed.add(bk.B)
                bk.graph = None
                log.warning("no graph for decode steps of %d requests (%s); they run kernel by kernel", bk.B, e)
                return None
        bk.graph.replay()
        self.replays += 1
        wanted = [i for i, e in enumerate(entries) if e.want]
        if wanted == list(range(n)):
            return bk.logits[:n]
        return bk.logits[torch.tensor(wanted, dtype=torch.long, device=bk.logits.device)]

    def _capture(self, bk: _Bucket) -> None:
        runner = self.runner
        step = bk.context(self.max_positions)
        torch.cuda.synchronize()
        # The run before the capture really executes: keys and values written twice are the same keys and
        # values, but per-request state would be advanced twice. For that run every row's state is the
        # row that belongs to nobody; the requests' own slots come back before the replay.
        slots = bk.view(bk.state)
        real_slots = slots.clone()
        slots.fill_(runner.pools.padding_state_slot)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        # a first run outside the graph: lazy set-up happens here, and the library's products are timed now
        with torch.cuda.stream(side):
            runner.forward(step, about_to_be_captured=True)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with _recording(graph):
            bk.logits = runner.forward(step)
        slots.copy_(real_slots)
        bk.graph = graph


class _Captured:
    def __init__(self):
        self.dev: torch.Tensor | None = None
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits: torch.Tensor | None = None


def _next_power_of_two(n: int) -> int:
    return 1 << (n - 1).bit_length() if n > 0 else 0


class StepGraphs:
    """Graphs for steps that hold prompt portions (whole prompts or parts of them), alone or beside
    single decoded tokens, where every entry wants at most one row of logits. The step is laid out
    in a padded shape (``padded_shape``): the portions' rows up to a few sizes, the numbers of
    portions, single tokens and logit rows up to powers of two, so that steps of similar sizes launch
    the same grids. A shape is captured when it comes the second time (the fourth, for a step of
    several entries); the most recently used
    ``max_graphs`` shapes are kept (each holds the activations of a step of its size)."""

    def __init__(self, runner, max_graphs: int = 16, max_singles: int = 256):
        self.runner = runner
        ops.library_workspace(runner.device)
        self.W = -(-runner.max_positions // runner.page_size)
        self.max_graphs, self.max_singles = max_graphs, max_singles
        self.max_mixed_rows = 1024
        self.seen: dict[tuple, int] = {}
        self.captured: dict[tuple, _Captured] = {}         # insertion order = least recently used first
        self.failed: set[tuple] = set()                     # shapes whose capture failed: those steps run eagerly
        self.replays = 0

    @staticmethod
    def padded_rows(n: int) -> int:
        """Rows that portions of n tokens in all run with: the next multiple of 32 (64 above 512
        tokens, 128 above 1,024, 256 above 2,048); at most an eighth of the rows is padding beyond
        the first steps."""
        step = 32 if n <= 512 else (64 if n <= 1024 else (128 if n <= 2048 else 256))
        return -(-n // step) * step

    @classmethod
    def padded_shape(cls, entries) -> tuple[int, int, int, int]:
        """(rows of the portions, portions, single tokens, logit rows) the step is laid out with."""
        rows = sum(len(e.tokens) for e in entries if len(e.tokens) > 1)
        portions = sum(1 for e in entries if len(e.tokens) > 1)
        wanted = sum(len(e.want) for e in entries)
        return (cls.padded_rows(rows), _next_power_of_two(portions), _next_power_of_two(len(entries) - portions),
                _next_power_of_two(wanted))

    def can_run(self, entries) -> bool:
        if self.runner.pools.states:
            return False        # state is advanced token by token inside a portion, from the host's view of the step
        portions = sum(1 for e in entries if len(e.tokens) > 1)
        if portions == 0 or len(entries) - portions > self.max_singles or any(len(e.want) > 1 for e in entries):
            return False
        if portions == 1 and len(entries) == 1:
            return True                                     # few shapes: every size pays
        # Steps of several entries come in many shapes. A replay saves host time, which only shows while
        # the step's kernels take less time than launching them one by one (about 4 ms): beyond that many
        # rows a capture and the padding cost more than the replays give back.
        rows = sum(len(e.tokens) for e in entries)
        return rows <= self.max_mixed_rows

    @torch.inference_mode()
    def run(self, entries) -> torch.Tensor | None:
        """The step's logits [wanted, vocab] in the entries' order, or None if this shape has no graph
        yet (the caller then runs the step kernel by kernel)."""
        runner = self.runner
        key = self.padded_shape(entries)
        wanted = sum(len(e.want) for e in entries)
        slot = self.captured.pop(key, None)
        if slot is None:
            self.seen[key] = self.seen.get(key, 0) + 1
            # a capture costs about as much as ten replays save: a shape of several entries (there are
            # many of them) has to come back a few times first
            if self.seen[key] < (2 if len(entries) == 1 else 4) or key in self.failed:
                return None
            try:
                slot = self._capture(entries, key)
            except RuntimeError as e:
                self.failed.add(key)
                log.warning("no graph for steps of shape %s (%s); they run kernel by kernel", key, e)
                return None
            while len(self.captured) >= self.max_graphs:   # the least recently used shape gives its memory back
                self.captured.pop(next(iter(self.captured)))
        else:
            runner.prepare(entries, into=slot.dev, table_width=self.W, shape=key)
        self.captured[key] = slot
        slot.graph.replay()
        self.replays += 1
        return slot.logits[:wanted]

    @torch.inference_mode()
    def _capture(self, entries, key) -> _Captured:
        """A first run of the step outside the graph, then the capture; the step's metadata lie in the
        buffer the graph reads."""
        runner = self.runner
        slot = _Captured()
        slot.dev = torch.zeros(runner.metadata_ints(key, self.W), dtype=torch.int32, device=runner.device)
        step, _ = runner.prepare(entries, into=slot.dev, table_width=self.W, shape=key)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        # a first run outside the graph: lazy set-up happens here, and the library's products are timed now
        with torch.cuda.stream(side):
            runner.forward(step, about_to_be_captured=True)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with _recording(graph):
            slot.logits = runner.forward(step)
        slot.graph = graph
        return slot

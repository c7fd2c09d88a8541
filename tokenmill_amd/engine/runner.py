"""The step function: one batch of (request, its next tokens) in, logits at the wanted places out.

It is the reference's ModelRunner.prepare/execute (reference src/infer/engine/model_runner.py:40-97)
with three differences: any row of the step may ask for logits, not only a request's last; the
per-step metadata goes to the device in ONE pinned buffer and one copy instead of one per array;
and attention reads the cache in place, so no per-request segment objects are built.

A step runs only the tokens it is given. Portions of prompts (any length, starting anywhere) and
single decoded tokens sit side by side in one flat batch; every token carries its absolute
position in its own request and the flat cache slot its key and value go to.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from tokenmill_amd.cache.manager import RELEASED, RequestCache
from tokenmill_amd.cache.pool import CachePools
from tokenmill_amd.parts.base import GroupStep, StepContext


@dataclass
class StepEntry:
    """One request's share of a step."""
    cache: RequestCache              # its block tables and state slot
    start: int                       # position of tokens[0] = number of its tokens already cached
    tokens: list[int]
    want: list[int] = field(default_factory=list)    # indices into ``tokens`` whose logits are wanted


class StepError(ValueError):
    """The batch cannot run as given (an id outside the vocabulary, a position without a page, ...)."""


class ModelRunner:
    def __init__(self, model, pools: CachePools, max_positions: int, tune: tuple[int, bool] | None = None):
        self.model = model
        self.pools = pools
        # the model's one forward pass: its parts' operations in run order, described once to the kernel library
        # (``tune``: (candidates, every) if this runner's library products are to be timed)
        self.program = model.program(pools.views, tune) if hasattr(model, "program") else None
        self.page_size = pools.page_size
        self.max_positions = max_positions
        self.device = model.device
        self.vocab = model.head.vocab
        self._pinned = torch.empty(1 << 14, dtype=torch.int32, pin_memory=True)
        self._copied = torch.cuda.Event()
        self._copy_pending = False
        self.graphs = None                        # DecodeGraphs when the engine runs with --hip-graphs
        self.step_graphs = None                # StepGraphs likewise

    # ------------------------------------------------------------------------------------------------

    def _staging(self, n: int) -> np.ndarray:
        if self._copy_pending:
            self._copied.synchronize()            # the last step's copy has left the buffer
            self._copy_pending = False
        if self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 2 * self._pinned.numel()), dtype=torch.int32, pin_memory=True)
        return self._pinned.numpy()

    def prepare(self, entries: list[StepEntry], into: torch.Tensor | None = None,
                table_width: int | None = None, shape: tuple[int, int, int, int] | None = None
                ) -> tuple[StepContext, list[int]]:
        """Flatten the entries into device metadata. Returns the context and, for each wanted logit
        in the caller's order (entries in the given order, ``want`` in its order), its row in the
        step's logits. ``into``: a device int32 buffer to hold the metadata (a captured graph reads
        it at a fixed address; steps of the same shape lay it out the same way); ``table_width``:
        pad the block tables to this width instead of the widest of the step; ``shape`` = (rows of the
        prompt portions, portions, single tokens, logit rows): lay the step out with this many of each,
        so that steps of similar sizes launch the same grids (see ``padded_shape``). What is added:
        rows behind the portions' tokens and single tokens behind the real ones, each token 0 at
        position 0 with no cache slot (its keys are not stored) and, for a single token, a context of
        one key in page 0; portions without tokens; repeats of the first logit row; repeats of a real
        attention tile (which compute the same rows again). Every kernel treats rows apart, so what a
        padding row holds reaches no other row. The contexts the launches are sized for are then the
        longest the model allows."""
        if not entries:
            raise StepError("a step needs at least one entry")
        page = self.page_size
        n_groups = len(self.pools.groups)
        # prompt portions first, single tokens last (the order the attention kernels split on)
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) == 1)
        n_portions = sum(1 for e in entries if len(e.tokens) > 1)
        n_singles = len(entries) - n_portions
        Tp_real = sum(len(e.tokens) for e in entries if len(e.tokens) > 1)
        R_real = sum(len(e.want) for e in entries)
        Tp, P, ND, R = Tp_real, n_portions, n_singles, R_real
        if shape is not None:
            Tp, P, ND, R = shape
            if Tp < Tp_real or Tp % 16 or P < n_portions or ND < n_singles or R < R_real:
                raise StepError(f"a step of {(Tp_real, n_portions, n_singles, R_real)} does not fit the shape {shape}")
        S = P + ND
        T = Tp + ND
        widths = []
        for e in entries:
            if not e.tokens:
                raise StepError(f"{e.cache.request_id}: an entry needs at least one token")
            if e.start < 0 or e.start + len(e.tokens) > self.max_positions:
                raise StepError(f"{e.cache.request_id}: positions {e.start}..{e.start + len(e.tokens) - 1} "
                                f"exceed the model's {self.max_positions}")
            end = e.start + len(e.tokens)
            need = -(-end // page)
            for g in range(n_groups):
                if len(e.cache.tables[g]) < need:
                    raise StepError(f"{e.cache.request_id}: {len(e.cache.tables[g])} pages do not hold {end} tokens")
            widths.append(need)
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise StepError(f"{e.cache.request_id}: wanted place {w} is not among its {len(e.tokens)} tokens")
        W = max(widths)
        if table_width is not None:
            if table_width < W:
                raise StepError(f"block tables of {W} pages do not fit the width {table_width}")
            W = table_width
        n_tiles_real = sum(-(-len(e.tokens) // 16) for e in entries if len(e.tokens) > 1)
        n_tiles = self.padded_tiles(Tp, P) if (shape is not None and n_tiles_real) else n_tiles_real
        n_ints = 3 * T + (S + 1) + 2 * S + max(R, 1) + n_groups * (T + S * W) + 4 * n_tiles
        buf = self._staging(n_ints)
        off = 0

        def take(n):
            nonlocal off
            view = buf[off:off + n]
            span = (off, n)
            off += n
            return view, span

        ids, ids_s = take(T)
        pos, pos_s = take(T)
        seq_of, seq_s = take(T)
        cu, cu_s = take(S + 1)
        ctx_lens, ctx_s = take(S)
        slots_state, st_s = take(S)
        rows, rows_s = take(max(R, 1))
        g_slot, g_tab = [], []
        for _ in range(n_groups):
            g_slot.append(take(T))
            g_tab.append(take(S * W))

        tiles, tiles_s = take(4 * n_tiles)
        if shape is not None:                               # what no entry fills is padding
            ids[:] = 0
            pos[:] = 0
            seq_of[:] = 0
            ctx_lens[:] = 1
            slots_state[:] = self.pools.padding_state_slot
            rows[:] = 0
            for g in range(n_groups):
                g_slot[g][0][:] = -1
                g_tab[g][0][:] = 0
        tile_i = 0
        row0 = 0
        first_row = [0] * S
        q_lens, starts = [], []
        cu[0] = 0
        for s, i in enumerate(order[:n_portions]):
            e = entries[i]
            n = len(e.tokens)
            toks = np.asarray(e.tokens, dtype=np.int64)
            if toks.min() < 0 or toks.max() >= self.vocab:
                raise StepError(f"{e.cache.request_id}: a token id is outside the vocabulary of {self.vocab}")
            ids[row0:row0 + n] = toks
            p = np.arange(e.start, e.start + n, dtype=np.int64)
            pos[row0:row0 + n] = p
            seq_of[row0:row0 + n] = s
            cu[s + 1] = row0 + n
            ctx_lens[s] = e.start + n
            slots_state[s] = e.cache.state_slot
            for g in range(n_groups):
                table = np.asarray(e.cache.tables[g][:widths[i]], dtype=np.int64)
                pages = table[p // page]
                if (pages == RELEASED).any():
                    raise StepError(f"{e.cache.request_id}: a token would be written to a page already given back")
                g_slot[g][0][row0:row0 + n] = pages * page + p % page
                tab = g_tab[g][0][s * W:(s + 1) * W]
                tab[:widths[i]] = np.where(table == RELEASED, 0, table)   # never read: below the window
                tab[widths[i]:] = 0                                       # padding: never read either
            if n > 1:
                first = np.arange(0, n, 16, dtype=np.int64)                      # first token of each tile
                t = tiles[4 * tile_i:4 * (tile_i + len(first))].reshape(len(first), 4)
                t[:, 0] = s
                t[:, 1] = row0 + first
                t[:, 2] = np.minimum(16, n - first)
                t[:, 3] = e.start + first
                tile_i += len(first)
            first_row[i] = row0
            q_lens.append(n)
            starts.append(e.start)
            row0 += n
        # single tokens: the same rows, written with a few bulk assignments instead of a dozen array
        # operations each (a mixed step may hold a hundred of them)
        cu[n_portions + 1:P + 1] = Tp_real                  # portions without tokens
        row0 = Tp                                           # the single tokens stand behind the portions' rows
        singles = [entries[i] for i in order[n_portions:]]
        cu[P + 1:] = np.arange(Tp + 1, Tp + ND + 1)
        if singles:
            n1 = len(singles)
            s0 = P
            toks = np.asarray([e.tokens[0] for e in singles], dtype=np.int64)
            if toks.min() < 0 or toks.max() >= self.vocab:
                raise StepError(f"a token id is outside the vocabulary of {self.vocab}")
            p1 = [e.start for e in singles]
            ids[row0:row0 + n1] = toks
            pos[row0:row0 + n1] = p1
            seq_of[row0:row0 + n1] = np.arange(s0, s0 + n1)
            cu[s0 + 1:s0 + n1 + 1] = np.arange(row0 + 1, row0 + n1 + 1)
            ctx_lens[s0:s0 + n1] = [p + 1 for p in p1]
            slots_state[s0:s0 + n1] = [e.cache.state_slot for e in singles]
            for g in range(n_groups):
                tabs = g_tab[g][0][s0 * W:(s0 + n1) * W].reshape(n1, W)
                windowed = self.pools.groups[g].window is not None
                new_slots = []
                for j, (e, p) in enumerate(zip(singles, p1)):
                    table = e.cache.tables[g]
                    last = p // page
                    if table[last] == RELEASED:
                        raise StepError(f"{e.cache.request_id}: a token would be written to a page already given back")
                    new_slots.append(table[last] * page + p % page)
                    row = tabs[j]
                    row[:last + 1] = table[:last + 1]
                    row[last + 1:] = 0                                        # padding: never read
                    if windowed:
                        row[row == RELEASED] = 0                              # never read: below the window
                g_slot[g][0][row0:row0 + n1] = new_slots
            for j, i in enumerate(order[n_portions:]):
                first_row[i] = row0 + j
            q_lens.extend([1] * n1)
            starts.extend(p1)
            row0 += n1
        if n_tiles > n_tiles_real:                                            # repeats of the last real tile
            t = tiles.reshape(n_tiles, 4)
            t[n_tiles_real:] = t[n_tiles_real - 1]
        if n_tiles > 1:
            # the tiles that see the most keys first: the long ones start early and the short ones fill
            # the end of the launch (a tile's result does not depend on where in the table it stands)
            t = tiles.reshape(n_tiles, 4)
            t[:] = t[np.argsort(-(t[:, 3] + t[:, 2]), kind="stable")]
        r = 0
        for i, e in enumerate(entries):
            for w in e.want:
                rows[r] = first_row[i] + w
                r += 1
        if R_real == 0:
            rows[0] = 0
        elif R > R_real:
            rows[R_real:R] = rows[0]

        if into is None:
            dev = self._pinned[:off].to(self.device, non_blocking=True)
        else:
            if into.numel() < off or into.dtype != torch.int32:
                raise StepError("the metadata buffer is too small for this step")
            dev = into[:off]
            dev.copy_(self._pinned[:off], non_blocking=True)
        self._copied.record()
        self._copy_pending = True

        def d(span):
            return dev[span[0]:span[0] + span[1]]

        groups = [GroupStep(block_tables=d(g_tab[g][1]).view(S, W), slot_mapping=d(g_slot[g][1]))
                  for g in range(n_groups)]
        ctx = StepContext(
            num_tokens=T, num_seqs=S, token_ids=d(ids_s), positions=d(pos_s), seq_of_token=d(seq_s),
            cu_q_lens=d(cu_s), context_lens=d(ctx_s), state_slots=d(st_s), logit_rows=d(rows_s)[:R], groups=groups,
            q_lens=q_lens, start_positions=starts, max_q_len=max(q_lens),
            max_context_len=self.max_positions if shape is not None else max(s0 + n for s0, n in zip(starts, q_lens)),
            num_logit_rows=R, num_decode=ND,
            max_decode_context=(self.max_positions if ND else 0) if shape is not None else
            max([s0 + 1 for s0, n in zip(starts, q_lens) if n == 1], default=0),
            prefill_tiles=d(tiles_s).view(n_tiles, 4))
        return ctx, list(range(R_real))

    @staticmethod
    def padded_tiles(portion_rows: int, portions: int) -> int:
        """Tiles of 16 tokens that any ``portions`` portions (or fewer) with at most ``portion_rows`` (a multiple
        of 16) tokens in all can need: every portion but one may add a tile that is not full. One portion
        needs no more tiles than its rows: a 2,048-token prompt stays at 128 tiles, a block for every CU."""
        return portion_rows // 16 + max(portions - 1, 0)

    def metadata_ints(self, shape: tuple[int, int, int, int], table_width: int) -> int:
        """Size of the metadata buffer ``prepare`` fills for a step of this shape."""
        Tp, P, ND, R = shape
        S, T = P + ND, Tp + ND
        return (3 * T + (S + 1) + 2 * S + max(R, 1) + len(self.pools.groups) * (T + S * table_width)
                + 4 * self.padded_tiles(Tp, P))

    @torch.inference_mode()
    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Run one step. Returns float32 logits [R, vocab] on the device: one row per wanted place,
        entries in the given order and each entry's ``want`` in its order."""
        for e in entries:
            if e.cache.fresh:                     # per-request state starts from zero at (re)admission
                self.pools.reset_state_slot(e.cache.state_slot)
                e.cache.fresh = False
        if self.graphs is not None and self.graphs.can_run(entries):
            logits = self.graphs.run(entries)
            if logits is not None:
                return logits
        if self.step_graphs is not None and self.step_graphs.can_run(entries):
            logits = self.step_graphs.run(entries)
            if logits is not None:
                return logits
        ctx, _ = self.prepare(entries)
        return self.forward(ctx)

    def step_behind(self, entries: list[StepEntry], ids_from: torch.Tensor) -> torch.Tensor | None:
        """A step of single tokens queued behind the step whose sampled ids ``ids_from`` holds on the device (one per
        entry, in the entries' order; the entries' own ``tokens`` are placeholders). Only as a graph replay: None if
        this batch has no graph, and nothing was queued then."""
        if self.graphs is None or not self.graphs.can_run(entries) or any(e.cache.fresh for e in entries):
            return None
        bucket = self.graphs._bucket(len(entries))
        if bucket.graph is None:                  # a capture runs the step outside the graph first: not behind another
            return None
        return self.graphs.run(entries, ids_from=ids_from)

    def forward(self, step: StepContext, about_to_be_captured: bool = False) -> torch.Tensor:
        """The step's float32 logits [R, vocab], by the model's step program."""
        return self.program.run(step, at_once=about_to_be_captured)

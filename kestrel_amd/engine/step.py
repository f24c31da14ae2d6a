"""The step function: one batch of (request, its next tokens) through the model.

A step takes, for any number of live requests, the next tokens of each: a portion of
a prompt (cut anywhere) or one decoded token, all packed into one token stream. It
runs only these tokens, reading what earlier steps left in the cache, and returns the
logits at the places asked for. The reference runs either padded whole prompts
(``kestrel/models/moondream/runtime.py:1999-2157``) or one token per row
(``runtime.py:2479-2586``); its metadata (slot mapping ``kv_cache.py:524-551``, per-row
block table and key counts ``runtime.py:2283-2290``) is what is built here per token.

Steps that hold one token per request are replayed as HIP graphs, one graph per batch
size bucket (1, 2, 4, 8, 16, 32, 48, ... as in ``kestrel/runtime/decode_graph.py:18-23``): the
metadata lives at fixed addresses, rows that pad the bucket see no keys and write nothing. A graph
is captured, and run once before that, on padding rows alone: no live request is touched by
anything but the replays, so a mixer that keeps state is advanced once a step.

Steps of any other shape (a prompt portion, alone or beside decoded tokens) of up to
``MIXED_GRAPH_MAX_TOKENS`` tokens are replayed as well where every part of the model allows it
(``Part.replays_every_step``), one graph per bucket of tokens and of rows: launching a layer's kernels
one by one costs the host about 0.13 ms, which is more than the kernels of a short portion take.
Their layout is fixed by the bucket (``ModelRunner.build_batch`` with ``pad_tokens``); longer steps, and
steps that want more logits than the largest bucket of rows, are launched kernel by kernel.
"""

from __future__ import annotations

import operator
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..models.decoder import DecoderModel
from .batch import GroupBatch, StepBatch, Workspace


PENDING_TOKEN = -2     # "the token that sampling last left for this request on the device"
GIVEN_TOKEN = -1       # "the embedding of this place is given"


class StepRefused(ValueError):
    """An entry of a step is not what the step function takes. It is raised before any page is
    taken or any kernel runs, so the other entries of the step can be run again without it;
    ``entry_index`` names the entry."""

    def __init__(self, entry_index: int, message: str) -> None:
        super().__init__(message)
        self.entry_index = entry_index


@dataclass
class StepEntry:
    """The next tokens of one request.

    ``tokens``: ids; ``-1`` marks a place whose embedding is given in ``embeds`` (rows in
    order of the ``-1`` places); ``PENDING_TOKEN`` stands for the id that the sampler last
    stored for this request in ``ModelRunner.pending`` (it need not have reached the host,
    ``kestrel/scheduler/scheduler.py:2289-2290``). ``want``: indices into ``tokens`` whose logits are returned.
    ``bidirectional``: position ranges ``[lo, hi)`` whose tokens see each other both ways
    (an image block); each must lie wholly inside this portion. ``start``: position of the
    first token; ``None`` means right after what the request already holds. ``positions``: for models
    with a position encoding of several axes (``PositionEncoding.axes``), the numbers of every token,
    ``[tokens, axes]``; ``None``: the place in the sequence on every axis.
    """

    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()
    embeds: Optional[torch.Tensor] = None
    bidirectional: Sequence[Tuple[int, int]] = ()
    start: Optional[int] = None
    positions: Optional[Sequence[Sequence[int]]] = None


def _align(n: int) -> int:
    return (n + 3) & ~3


def graph_buckets(max_batch: int) -> List[int]:
    """Batch sizes graphs are captured for: 1, 2, 4, 8, then every multiple of 16, then
    ``max_batch`` itself (``kestrel/runtime/decode_graph.py:18-23``; 33 -> 1, 2, 4, 8, 16, 32, 33;
    64 -> 1, 2, 4, 8, 16, 32, 48, 64)."""
    max_batch = max(1, max_batch)
    sizes = {size for size in (1, 2, 4, 8) if size <= max_batch}
    sizes.update(range(16, max_batch + 1, 16))
    sizes.add(max_batch)
    return sorted(sizes)


# Steps of any shape are captured up to this many tokens. Up to some 1,500 tokens the host needs longer to
# launch a step's kernels one by one than the kernels take; beyond, a replay still saves what passes
# between two launched kernels (0.4 ms of a 2,048-token prompt's 6.9).
MIXED_GRAPH_MAX_TOKENS = 2048


def mixed_graph_buckets(max_tokens: int) -> List[int]:
    """Token counts that steps of any shape are captured for: 16, 32, every multiple of 64 up to 512, every
    multiple of 128 up to ``MIXED_GRAPH_MAX_TOKENS``, and the step's token limit itself where that is less."""
    top = max(1, min(int(max_tokens), MIXED_GRAPH_MAX_TOKENS))
    sizes = {size for size in (16, 32, *range(64, 513, 64), *range(640, MIXED_GRAPH_MAX_TOKENS + 1, 128)) if size <= top}
    sizes.add(top)
    return sorted(sizes)


def mixed_graph_rows(max_requests: int) -> List[int]:
    """Numbers of rows (requests, and wanted places) that steps of any shape are captured for."""
    top = max(1, int(max_requests))
    return sorted({min(8, top), min(64, top), top})


class _Column:
    """The int32 values of one section of a step's metadata, gathered piece by piece: lists from
    rows of a few tokens, arrays from prompt portions (thousands of tokens, which are never
    turned into Python integers)."""

    def __init__(self) -> None:
        self.pieces: list = []
        self.count = 0

    def __len__(self) -> int:
        return self.count

    def extend(self, values) -> None:
        if isinstance(values, np.ndarray):
            self.pieces.append(values)
        else:
            values = list(values)
            if self.pieces and isinstance(self.pieces[-1], list):
                self.pieces[-1].extend(values)
            else:
                self.pieces.append(values)
        self.count += len(values)

    def append(self, value: int) -> None:
        self.extend((value,))

    def write(self, host: np.ndarray, offset: int) -> None:
        for piece in self.pieces:
            host[offset:offset + len(piece)] = piece
            offset += len(piece)


class _GraphState:
    """A captured step of one bucket size: its metadata, scratch and graph."""

    def __init__(self, device: torch.device) -> None:
        self.workspace = Workspace(device)
        self.meta: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None


class _PageRuns:
    """The packed tokens of a step cut into runs for the kernels that write the cache: a run is
    either the tokens that fill one page of their row in order (``page_size`` of them, the first at a
    page's start), or up to ``page_size`` neighbouring tokens of any kind (a prompt's first or last few,
    single decoded tokens of different rows)."""

    def __init__(self, page_size: int) -> None:
        self.ps = page_size
        self._first: List[int] = []
        self._count: List[int] = []
        self._loose_first = 0
        self._loose = 0

    def _close(self) -> None:
        if self._loose:
            self._first.append(self._loose_first)
            self._count.append(self._loose)
            self._loose = 0

    def _add_loose(self, at: int, n: int) -> None:
        if self._loose and (self._loose_first + self._loose != at or self._loose + n > self.ps):
            self._close()
        if not self._loose:
            self._loose_first = at
        self._loose += n

    def add(self, base: int, start: int, q: int) -> None:
        """``q`` tokens of one row at positions ``start...``, the first of them token ``base`` of the step."""
        ps = self.ps
        lead = min(q, (-start) % ps)               # up to the next page's start
        if lead:
            self._add_loose(base, lead)
        pages = (q - lead) // ps
        if pages:
            self._close()
            self._first.extend(range(base + lead, base + lead + pages * ps, ps))
            self._count.extend([ps] * pages)
        tail = q - lead - pages * ps
        if tail:
            self._add_loose(base + lead + pages * ps, tail)

    def first(self) -> List[int]:
        self._close()
        return self._first

    def count(self) -> List[int]:
        self._close()
        return self._count


class ModelRunner:
    """Owns the model, its cache and the scratch memory; ``step`` is the only way in."""

    STAGING_RING = 4
    SCALAR_ROW = 16          # rows of at most this many tokens are laid out token by token, longer ones as arrays

    def __init__(self, model: DecoderModel, cache: CacheManager, device: torch.device,
                 max_tokens_per_step: int = 4096, enable_graphs: bool = False,
                 max_graph_batch: Optional[int] = None) -> None:
        self.model, self.cache, self.device = model, cache, device
        self.max_tokens_per_step = max_tokens_per_step
        self.workspace = Workspace(device)
        self.layer_caches = cache.layer_caches()
        self.held: Dict[int, int] = {}            # slot -> tokens the request holds in the cache
        self._staging: List[Optional[torch.Tensor]] = [None] * self.STAGING_RING
        self._staging_events: List[Optional[torch.cuda.Event]] = [None] * self.STAGING_RING
        self._staging_next = 0
        self._meta_device: Optional[torch.Tensor] = None
        self.enable_graphs = enable_graphs
        self._buckets = graph_buckets(min(max_graph_batch or cache.max_requests, cache.max_requests))
        self._graphs: Dict[int, _GraphState] = {}
        self._pages_cap = -(-model.plan.max_positions // cache.page_size)
        self.graph_replays = 0
        # steps of any shape (prompt portions, beside decoded tokens or not) are replayed too, if every
        # part of the model can be (``Part.replays_every_step``): per bucket of tokens and of rows
        every = getattr(model, "replays_every_step", None)
        self.mixed_graphs = bool(enable_graphs and callable(every) and every())
        self._mixed_tokens = mixed_graph_buckets(max_tokens_per_step)
        self._mixed_rows = mixed_graph_rows(cache.max_requests)
        self._mixed: Dict[Tuple[int, int], _GraphState] = {}      # (tokens, rows) -> the captured step
        self._mixed_workspace: Optional[Workspace] = None         # their scratch tensors, shared
        self._mixed_given: Optional[torch.Tensor] = None          # where given embeddings are copied to before a replay
        self.mixed_graph_replays = 0
        self.logit_slots: Optional[torch.Tensor] = None     # of the last step: the slot per row of logits, on the device
        # the latest sampled token of every request slot, written by the sampling kernels
        self.pending = torch.zeros(max(1, cache.max_requests), dtype=torch.int32, device=device)
        # Sizes of the blocks of queries that the mixers' kernels want a row cut into (a mixer says
        # so through ``query_tile()``): the step lists the blocks of each size, most keys first.
        tiles = getattr(model, "query_tiles", None)
        self.query_tiles: List[int] = sorted(tiles()) if callable(tiles) else []
        axes = getattr(model, "position_axes", None)
        self.position_axes: int = int(axes()) if callable(axes) else 1

    # ------------------------------------------------------------------ requests
    def admit(self, reserve_length: int = 0, portion: int = 1) -> int:
        slot = self.cache.admit(reserve_length, portion)
        self.held[slot] = 0
        return slot

    def release(self, slot: int) -> None:
        self.cache.release(slot)
        del self.held[slot]

    # ------------------------------------------------------------------ metadata
    def _stage(self, count: int) -> Tuple[torch.Tensor, int]:
        index = self._staging_next
        self._staging_next = (index + 1) % self.STAGING_RING
        event = self._staging_events[index]
        if event is not None:
            event.synchronize()
        buf = self._staging[index]
        if buf is None or buf.numel() < count:
            buf = torch.empty(max(count, 4096), dtype=torch.int32, pin_memory=True)
            self._staging[index] = buf
        return buf, index

    def _check_entries(self, entries: Sequence[StepEntry]) -> List[int]:
        """Everything that can be wrong with an entry is found here, before the step touches the
        cache: its slot, its start, its token ids, its embeddings, its block and the places wanted.
        Returns the entries' start positions."""
        plan = self.model.plan
        seen = set()
        starts: List[int] = []
        n_tokens = 0
        for index, e in enumerate(entries):
            def refuse(message: str, index=index, e=e):
                return StepRefused(index, f"slot {e.slot}: {message}")
            if e.slot in seen:
                raise refuse("it appears twice in one step")
            seen.add(e.slot)
            if e.slot not in self.held:
                raise refuse("it is not live")
            q = len(e.tokens)
            if q == 0:
                raise refuse("an entry needs at least one token")
            start = self.held[e.slot] if e.start is None else int(e.start)
            if start != self.held[e.slot]:
                raise refuse(f"portion starts at {start} but the request holds {self.held[e.slot]} tokens")
            if start + q > plan.max_positions:
                raise refuse(f"{start + q} tokens exceed the model's {plan.max_positions} positions")
            if q <= self.SCALAR_ROW:
                n_given = 0
                for tok in e.tokens:
                    try:
                        tok = operator.index(tok)
                    except TypeError:
                        raise refuse("token ids must be a flat sequence of integers") from None
                    if tok >= plan.vocab_size or tok < PENDING_TOKEN:
                        raise refuse(f"token id {tok} outside the vocabulary of {plan.vocab_size}")
                    n_given += tok == GIVEN_TOKEN
            else:
                tok_a = np.asarray(e.tokens)
                if tok_a.ndim != 1 or tok_a.dtype.kind not in "iu":
                    raise refuse("token ids must be a flat sequence of integers")
                bad = (tok_a >= plan.vocab_size) | (tok_a < PENDING_TOKEN)
                if bad.any():
                    raise refuse(f"token id {int(tok_a[bad][0])} outside the vocabulary of {plan.vocab_size}")
                n_given = int((tok_a == GIVEN_TOKEN).sum())
            if n_given:
                if not isinstance(e.embeds, torch.Tensor) or e.embeds.dim() != 2 \
                        or tuple(e.embeds.shape) != (n_given, plan.dim) or not e.embeds.is_floating_point():
                    raise refuse(f"{n_given} places need floating-point embeddings of shape [{n_given}, {plan.dim}]")
            elif e.embeds is not None and e.embeds.numel():
                raise refuse("embeddings given but no token id is -1")
            for lo_b, hi_b in e.bidirectional:
                if not (start <= lo_b < hi_b <= start + q):
                    raise refuse(f"the bidirectional block [{lo_b}, {hi_b}) must lie inside one portion, this one "
                                 f"covers [{start}, {start + q})")
            for w in e.want:
                if not 0 <= int(w) < q:
                    raise refuse(f"wanted place {w} outside its {q} tokens")
            if e.positions is not None:
                if self.position_axes == 1:
                    raise refuse("positions given, but the model's encodings take the place in the sequence")
                given_axes = np.asarray(e.positions)
                if given_axes.shape != (q, self.position_axes) or given_axes.dtype.kind not in "iu":
                    raise refuse(f"positions must be integers of shape [{q}, {self.position_axes}]")
            starts.append(start)
            n_tokens += q
        if n_tokens > self.max_tokens_per_step:
            raise ValueError(f"{n_tokens} tokens in one step exceed the limit of {self.max_tokens_per_step}")
        return starts

    def build_batch(self, entries: Sequence[StepEntry], pad_rows: int = 0, fixed_pages: int = 0,
                    meta: Optional[torch.Tensor] = None, workspace: Optional[Workspace] = None,
                    pad_tokens: int = 0) -> StepBatch:
        """Checks the entries, backs their positions with pages and lays the metadata out.

        ``pad_rows`` > number of entries adds rows of one token that see no keys and write
        nothing; ``fixed_pages`` fixes the width of the block tables; ``meta`` is the device
        buffer the metadata is copied into. With all three the layout depends on ``pad_rows``
        alone, which is what a captured graph needs.

        ``pad_tokens`` > 0 (with ``pad_rows`` and ``fixed_pages``) lays out a step of any shape so that the
        layout depends on ``pad_tokens`` and ``pad_rows`` alone: ``pad_rows + 1`` rows, of which those
        behind the entries hold no token and the last holds the tokens that fill the step up to
        ``pad_tokens`` (they see no keys and write nothing); ``pad_rows`` wanted places (those behind
        the entries' name token 0, for nobody); as many places for given rows as tokens (-1 behind
        the entries'); the lists of runs and of blocks of queries at the most entries any such step
        can have (runs without tokens and blocks without queries behind the step's own).
        """
        cache, plan = self.cache, self.model.plan
        ps = cache.page_size
        if not entries and pad_rows <= 0:
            raise ValueError("a step needs at least one entry")
        starts = self._check_entries(entries)
        for e, start in zip(entries, starts):
            cache.ensure(e.slot, start + len(e.tokens))

        n_groups = len(cache.groups)
        ids, positions, token_row, kv_hi = _Column(), _Column(), _Column(), _Column()
        n_axes = self.position_axes
        axes = _Column() if n_axes > 1 else None       # row-major [tokens, axes]
        # blocks of queries, per size: row, first token, most keys any of them sees
        blocks: Dict[int, List[Tuple[int, int, int]]] = {tile: [] for tile in self.query_tiles}
        logit_rows: List[int] = []
        logit_slot: List[int] = []            # the request's slot, per row of logits
        given_rows: List[int] = []
        given: List[torch.Tensor] = []
        row_slot: List[int] = []
        cu_q = [0]
        kv_len: List[int] = []
        slots = [_Column() for _ in range(n_groups)]
        kv_lo = [_Column() if g.spec.window is not None else None for g in cache.groups]
        max_pages = max(1, fixed_pages)
        max_q = max_kv = 1
        causal_only = True
        runs = _PageRuns(ps)
        for r, (e, start) in enumerate(zip(entries, starts)):
            q = len(e.tokens)
            base = len(ids)
            runs.add(base, start, q)
            if e.bidirectional:
                causal_only = False
            if q <= self.SCALAR_ROW:
                hi = [start + i + 1 for i in range(q)]
                for lo_b, hi_b in e.bidirectional:
                    for p in range(lo_b, hi_b):
                        hi[p - start] = max(hi[p - start], hi_b)
                row_ids, row_given = [], []
                for i, tok in enumerate(e.tokens):
                    tok = int(tok)
                    if tok == PENDING_TOKEN:
                        tok = PENDING_TOKEN - e.slot      # the embedding kernel reads pending[slot]
                    elif tok == GIVEN_TOKEN:
                        row_given.append(base + i)
                    row_ids.append(tok)
            else:
                # a prompt portion has thousands of tokens: a loop over them in Python would take
                # longer than some of the kernels that follow
                hi_a = np.arange(start + 1, start + q + 1, dtype=np.int64)
                for lo_b, hi_b in e.bidirectional:
                    np.maximum(hi_a[lo_b - start:hi_b - start], hi_b, out=hi_a[lo_b - start:hi_b - start])
                tok_a = np.array(e.tokens, dtype=np.int64).reshape(-1)     # a copy: it is edited below
                pending = tok_a == PENDING_TOKEN
                is_given = tok_a == GIVEN_TOKEN
                tok_a[pending] = PENDING_TOKEN - e.slot
                row_given = (base + np.nonzero(is_given)[0]).tolist()
                row_ids, hi = tok_a, hi_a
            n_given = len(row_given)
            given_rows.extend(row_given)
            ids.extend(row_ids)
            if n_given:
                given.append(e.embeds)
            if q <= self.SCALAR_ROW:
                positions.extend(range(start, start + q))
                token_row.extend([r] * q)
            else:
                positions.extend(np.arange(start, start + q, dtype=np.int64))
                token_row.extend(np.full(q, r, dtype=np.int64))
            kv_hi.extend(hi)
            if axes is not None:
                if e.positions is not None:
                    axes.extend(np.asarray(e.positions, dtype=np.int64).reshape(-1))
                else:
                    axes.extend(np.repeat(np.arange(start, start + q, dtype=np.int64), n_axes))
            for tile, listed in blocks.items():
                if isinstance(hi, np.ndarray):
                    # most keys any query of a block sees: the blocks' maxima in one go
                    tops = np.pad(hi, (0, (-q) % tile)).reshape(-1, tile).max(axis=1).tolist()
                    listed.extend((r, base + i * tile, top) for i, top in enumerate(tops))
                else:
                    for first in range(0, q, tile):
                        listed.append((r, base + first, max(hi[first:first + tile])))
            logit_rows.extend(base + int(w) for w in e.want)
            logit_slot.extend(e.slot for _ in e.want)
            cu_q.append(base + q)
            kv_len.append(start + q)
            row_slot.append(e.slot)
            max_q, max_kv = max(max_q, q), max(max_kv, start + q)
            for g in range(n_groups):
                table = cache.block_table(g, e.slot)
                if fixed_pages and len(table) > fixed_pages:
                    raise ValueError(f"slot {e.slot}: {len(table)} pages exceed the fixed table width {fixed_pages}")
                max_pages = max(max_pages, len(table))
                if q <= self.SCALAR_ROW:
                    slots[g].extend(table[p // ps] * ps + p % ps for p in range(start, start + q))
                else:
                    places = np.arange(start, start + q, dtype=np.int64)
                    slots[g].extend(np.asarray(table, dtype=np.int64)[places // ps] * ps + places % ps)
                if kv_lo[g] is not None:
                    kv_lo[g].extend(cache.window_start(g, p) for p in range(start, start + q))
        n_real = len(entries)
        n_wanted = len(logit_rows)
        if pad_tokens:
            n_live = len(ids)
            if n_live > pad_tokens or n_real > pad_rows or n_wanted > pad_rows or not fixed_pages:
                raise ValueError(f"{n_live} tokens of {n_real} rows with {n_wanted} wanted places do not fit a step "
                                 f"laid out for {pad_tokens} tokens and {pad_rows} rows")
            fill = pad_tokens - n_live
            cu_q.extend([n_live] * (pad_rows - n_real))            # rows without a token
            kv_len.extend([0] * (pad_rows - n_real))
            row_slot.extend([-1] * (pad_rows - n_real))
            if fill:                                               # the last row: what fills the step up
                zeros = np.zeros(fill, dtype=np.int64)
                runs.add(n_live, 0, fill)
                ids.extend(zeros)
                positions.extend(zeros)
                token_row.extend(np.full(fill, pad_rows, dtype=np.int64))
                kv_hi.extend(zeros)
                if axes is not None:
                    axes.extend(np.zeros(fill * n_axes, dtype=np.int64))
                for tile, listed in blocks.items():
                    listed.extend((pad_rows, n_live + first, 0) for first in range(0, fill, tile))
                for g in range(n_groups):
                    slots[g].extend(np.full(fill, -1, dtype=np.int64))
                    if kv_lo[g] is not None:
                        kv_lo[g].extend(zeros)
            cu_q.append(pad_tokens)
            kv_len.append(0)
            row_slot.append(-1)
            logit_rows.extend([0] * (pad_rows - n_wanted))
            logit_slot.extend([-1] * (pad_rows - n_wanted))
            given_rows = given_rows + [-1] * (pad_tokens - len(given_rows))
            pad_rows += 1                                          # (the last row is one of the step's rows)
        for r in range(n_real, 0 if pad_tokens else pad_rows):     # rows that only fill the bucket, a token each
            runs.add(len(ids), 0, 1)
            ids.append(0)
            positions.append(0)
            token_row.append(r)
            kv_hi.append(0)
            if axes is not None:
                axes.extend([0] * n_axes)
            for listed in blocks.values():
                listed.append((r, len(ids) - 1, 0))
            logit_rows.append(len(ids) - 1)
            logit_slot.append(-1)
            cu_q.append(len(ids))
            kv_len.append(0)
            row_slot.append(-1)                    # no request: a mixer with state must pass these rows over
            for g in range(n_groups):
                slots[g].append(-1)
                if kv_lo[g] is not None:
                    kv_lo[g].append(0)
        n_rows = max(n_real, pad_rows)
        n_tokens = len(ids)

        # the blocks that see the most keys first: a launch then ends with short ones
        for listed in blocks.values():
            listed.sort(key=lambda b: -b[2])
        run_first, run_count = runs.first(), runs.count()
        if pad_tokens:
            # every row with tokens has at most one block that is not full, and at most two runs that are no whole page
            most_runs = pad_tokens // ps + 2 * n_rows
            run_first = run_first + [0] * (most_runs - len(run_first))
            run_count = run_count + [0] * (most_runs - len(run_count))
            for tile, listed in blocks.items():
                # (a block of the last row that starts behind its last token: no query in it is live)
                listed.extend([(n_rows - 1, pad_tokens, 0)] * (pad_tokens // tile + n_rows - len(listed)))
        # one packed int32 buffer, every section starting on a 16-byte boundary
        sections: List[Tuple[str, object]] = [
            ("ids", ids), ("positions", positions), ("token_row", token_row), ("kv_hi", kv_hi),
            ("row_slot", row_slot), ("cu_q", cu_q), ("kv_len", kv_len), ("logit_rows", logit_rows),
            ("logit_slot", logit_slot),
            ("given_rows", given_rows), ("run_first", run_first), ("run_count", run_count),
        ]
        if axes is not None:
            sections.append(("position_axes", axes))
        for tile, listed in blocks.items():
            sections.append((f"qblk_row{tile}", [b[0] for b in listed]))
            sections.append((f"qblk_tok{tile}", [b[1] for b in listed]))
        for g in range(n_groups):
            sections.append((f"slots{g}", slots[g]))
            if kv_lo[g] is not None:
                sections.append((f"kv_lo{g}", kv_lo[g]))
            tables = np.zeros((n_rows, max_pages), dtype=np.int32)     # (rows without a request: page 0, never read)
            for r, e in enumerate(entries):
                table = cache.block_table(g, e.slot)
                tables[r, :len(table)] = table
                tables[r, len(table):] = -1
            sections.append((f"table{g}", tables.reshape(-1)))
        offsets: Dict[str, Tuple[int, int]] = {}
        total = 0
        for name, values in sections:
            offsets[name] = (total, len(values))
            total += _align(len(values))
        staging, ring = self._stage(total)
        host = staging.numpy()
        for name, values in sections:
            off, count = offsets[name]
            if count and isinstance(values, _Column):
                values.write(host, off)
            elif count:
                host[off:off + count] = values
        if meta is None:
            if self._meta_device is None or self._meta_device.numel() < total:
                self._meta_device = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
            meta = self._meta_device
        elif meta.numel() < total:
            raise ValueError("the metadata buffer of the graph is too small")
        meta[:total].copy_(staging[:total], non_blocking=True)
        event = self._staging_events[ring] or torch.cuda.Event()
        event.record()
        self._staging_events[ring] = event

        def view(name: str) -> torch.Tensor:
            off, count = offsets[name]
            return meta[off:off + count]

        groups: Dict[int, GroupBatch] = {}
        for g in range(n_groups):
            groups[g] = GroupBatch(block_table=view(f"table{g}").view(n_rows, max_pages), slots=view(f"slots{g}"),
                                   kv_lo=view(f"kv_lo{g}") if kv_lo[g] is not None else None, page_size=ps)
        given_embeds = None
        if given:
            given_embeds = torch.cat([t.to(self.device) for t in given], dim=0).contiguous()
            if given_embeds.dtype not in (torch.float32, torch.bfloat16):
                given_embeds = given_embeds.float()
        return StepBatch(
            n_tokens=n_tokens, n_rows=n_rows, token_ids=view("ids"), positions=view("positions"),
            token_row=view("token_row"), kv_hi=view("kv_hi"), row_slot=view("row_slot"), cu_q=view("cu_q"),
            kv_len=view("kv_len"), logit_rows=view("logit_rows"), logit_slot=view("logit_slot"), groups=groups,
            workspace=workspace or self.workspace,
            query_blocks={tile: (view(f"qblk_row{tile}"), view(f"qblk_tok{tile}")) for tile in blocks},
            position_axes=view("position_axes").view(n_tokens, n_axes) if axes is not None else None,
            pending=self.pending, given_embeds=given_embeds, given_rows=view("given_rows") if given or pad_tokens else None,
            max_q=max_q, max_kv=max_kv, decode_only=max_q == 1 and not pad_tokens, causal_only=causal_only and not pad_tokens,
            wants_every_token=not pad_tokens and logit_rows == list(range(n_tokens)),
            page_runs=(view("run_first"), view("run_count")),
            host={"starts": starts, "q_lens": [len(e.tokens) for e in entries], "kv_len": kv_len, "meta_ints": total},
        )

    # ------------------------------------------------------------------ graphs
    def _graph_bucket(self, entries: Sequence[StepEntry]) -> Optional[int]:
        """The bucket a step can be replayed in, or ``None``: every entry one token with its
        logits wanted, no given embedding, at most the largest bucket."""
        if not self.enable_graphs or len(entries) > self._buckets[-1]:
            return None
        for e in entries:
            # (anything odd about an entry is left to ``_check_entries``, which names it: the eager path)
            if len(e.tokens) != 1 or list(e.want) != [0] or e.embeds is not None:
                return None
            try:
                token = operator.index(e.tokens[0])
            except TypeError:
                return None
            if token < 0 and token != PENDING_TOKEN:
                return None
        return next(b for b in self._buckets if b >= len(entries))

    def _capture(self, bucket: int) -> _GraphState:
        """The graph of a decode step of ``bucket`` rows, made if it is not there yet.

        Warm-up and capture run on padding rows alone (no slot, no keys, nothing written): the
        layout of the metadata depends on the bucket only, and nothing of a live request,
        per-request state included, is touched before the first replay."""
        state = self._graphs.get(bucket)
        if state is None:
            state = self._graphs[bucket] = _GraphState(self.device)
        if state.graph is None:
            probe = self.build_batch([], pad_rows=bucket, fixed_pages=self._pages_cap)
            state.meta = torch.empty(probe.host["meta_ints"], dtype=torch.int32, device=self.device)
            blank = self.build_batch([], pad_rows=bucket, fixed_pages=self._pages_cap, meta=state.meta,
                                     workspace=state.workspace)
            # the decode attention kernel cuts a row's keys by the longest context of the batch: a
            # graph must cut the same way on every replay, so it is captured for the longest possible
            blank.max_kv = self.model.plan.max_positions
            self._run_aside(blank)
            state.workspace.freeze()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                state.logits = self.model.forward(blank, self.layer_caches)
            state.graph = graph
        return state

    def _mixed_bucket(self, entries: Sequence[StepEntry]) -> Optional[Tuple[int, int]]:
        """``(tokens, rows)`` of the captured layout that a step of any shape fits in, or ``None``."""
        if not self.mixed_graphs:
            return None
        try:
            n_tokens = sum(len(e.tokens) for e in entries)
            n_wanted = sum(len(e.want) for e in entries)
        except TypeError:
            return None                  # (``_check_entries`` names what is odd: the eager path)
        n_rows = max(len(entries), n_wanted)
        if n_tokens > self._mixed_tokens[-1] or n_rows > self._mixed_rows[-1]:
            return None
        return (next(t for t in self._mixed_tokens if t >= n_tokens), next(r for r in self._mixed_rows if r >= n_rows))

    def _blank_step(self, tokens: int, rows: int, meta: Optional[torch.Tensor], workspace: Optional[Workspace] = None) -> StepBatch:
        """A step of the layout ``(tokens, rows)`` whose tokens belong to no request."""
        blank = self.build_batch([], pad_rows=rows, pad_tokens=tokens, fixed_pages=self._pages_cap, meta=meta,
                                 workspace=workspace or self._mixed_workspace)
        blank.max_kv = self.model.plan.max_positions       # (kernels that size themselves by the longest row)
        blank.given_embeds = self._mixed_given[:tokens]
        return blank

    def _run_aside(self, batch: StepBatch) -> None:
        """A run outside any capture, on a stream of its own: every buffer and plan that the run needs comes into being."""
        current = torch.cuda.current_stream()
        side = torch.cuda.Stream()
        side.wait_stream(current)
        with torch.cuda.stream(side):
            self.model.forward(batch, self.layer_caches)
        current.wait_stream(side)
        torch.cuda.synchronize()

    def _capture_mixed(self, tokens: int, rows: int) -> _GraphState:
        """The graph of a step of up to ``tokens`` tokens of up to ``rows`` requests, made if it is not
        there yet: as for decode steps, on tokens that belong to no request. All these graphs run one
        after the other on one stream and share one set of scratch tensors: before the first of them
        is captured, every bucket of tokens (at the most rows) and of rows (at the most tokens) is run
        once, kernel by kernel, largest first, which brings every tensor that any of them asks for to
        the size that serves them all. (Which tensors a step asks for depends on its number of tokens:
        the kernels of few rows have scratch tensors of their own.)"""
        if self._mixed_workspace is None:
            self._mixed_workspace = Workspace(self.device)
            self._mixed_given = torch.zeros(self._mixed_tokens[-1], self.model.plan.dim, dtype=torch.float32, device=self.device)
            shapes = [(t, self._mixed_rows[-1]) for t in reversed(self._mixed_tokens)]
            shapes += [(self._mixed_tokens[-1], r) for r in reversed(self._mixed_rows[:-1])]
            for shape in shapes:
                self._run_aside(self._blank_step(*shape, None))
            self._mixed_workspace.freeze()
        state = self._mixed.get((tokens, rows))
        if state is None:
            state = self._mixed[(tokens, rows)] = _GraphState(self.device)
            state.workspace = self._mixed_workspace
        if state.graph is None:
            probe = self.build_batch([], pad_rows=rows, pad_tokens=tokens, fixed_pages=self._pages_cap)
            state.meta = torch.empty(probe.host["meta_ints"], dtype=torch.int32, device=self.device)
            try:
                blank = self._blank_step(tokens, rows, state.meta, state.workspace)
                self._run_aside(blank)             # (the vendor library's plans for this number of rows)
            except RuntimeError as error:
                if "after freeze()" not in str(error):
                    raise
                # a layout that asks for a tensor none of the runs above has made: scratch tensors of its own
                state.workspace = Workspace(self.device)
                blank = self._blank_step(tokens, rows, state.meta, state.workspace)
                self._run_aside(blank)
                state.workspace.freeze()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                state.logits = self.model.forward(blank, self.layer_caches)
            state.graph = graph
        return state

    def _step_mixed(self, entries: Sequence[StepEntry], tokens: int, rows: int) -> Tuple[torch.Tensor, List[int]]:
        if (tokens, rows) not in self._mixed:
            self._check_entries(entries)           # (no graph is made for a step that is refused)
        state = self._capture_mixed(tokens, rows)
        batch = self.build_batch(entries, pad_rows=rows, pad_tokens=tokens, fixed_pages=self._pages_cap, meta=state.meta,
                                 workspace=state.workspace)
        if batch.given_embeds is not None:
            self._mixed_given[:batch.given_embeds.shape[0]].copy_(batch.given_embeds)
        state.graph.replay()
        self.mixed_graph_replays += 1
        wanted = sum(len(e.want) for e in entries)
        self.logit_slots = batch.logit_slot[:wanted]
        return state.logits[:wanted], batch.host["starts"]

    def _step_graph(self, entries: Sequence[StepEntry], bucket: int) -> torch.Tensor:
        state = self._capture(bucket)
        batch = self.build_batch(entries, pad_rows=bucket, fixed_pages=self._pages_cap, meta=state.meta,
                                 workspace=state.workspace)
        state.graph.replay()
        self.graph_replays += 1
        self.logit_slots = batch.logit_slot[:len(entries)]
        return state.logits[:len(entries)]

    # ------------------------------------------------------------------ everything made at start
    @torch.no_grad()
    def prepare(self, prompt_tokens: Optional[int] = None, wanted_rows: int = 1, tune_linears: int = 0) -> Dict[str, float]:
        """Make now what steps would otherwise make when they first need it, with live requests
        waiting (``kestrel/runtime/decode_graph.py:70-93``, ``kestrel/models/moondream/runtime.py:886-888``,
        ``kestrel/engine/core.py:458-484``): the kernels' scratch buffers, the graph of every bucket of
        decode rows and, where steps of any shape are replayed, of every bucket of tokens and rows up to
        ``prompt_tokens`` (captured on padding rows), the metadata buffer at its largest, and the scratch
        tensors and vendor-library plans of prompt steps, by running prompts of ids 0 of every
        multiple of 64 tokens up to ``prompt_tokens`` (default: the step's token limit) through a slot
        that is given back. ``tune_linears`` > 0: the vendor-library linears of these prompts time the algorithms
        the library offers, that many products each, and keep the fastest per bucket of rows. No request may be
        live. Returns what was done and how long it took."""
        if self.held:
            raise RuntimeError("prepare() runs before the first request is admitted")
        import time

        done: Dict[str, float] = {}
        started = time.perf_counter()
        if self.model.dtype == torch.bfloat16:
            from ..ops import fast
            done["kernel_scratch_bytes"] = fast.prepare(self.device)
        cache, plan = self.cache, self.model.plan
        limit = self.max_tokens_per_step if prompt_tokens is None else min(prompt_tokens, self.max_tokens_per_step)
        rows = max(cache.max_requests, 1)
        per_token = 8 + 2 * len(cache.groups) + 2 * max(len(self.query_tiles), 1) + self.position_axes
        ints = per_token * (limit + rows) + rows * (8 + len(cache.groups) * (self._pages_cap + 4)) + 4096
        if self._meta_device is None or self._meta_device.numel() < ints:
            self._meta_device = torch.empty(ints, dtype=torch.int32, device=self.device)
        # (plans of the vendor library made from here on, by the runs before a capture or by the prompts below,
        # time their candidates)
        tuning = tune_linears > 0 and self.model.dtype == torch.bfloat16
        if tuning:
            fast.set_library_tuning(tune_linears)
        try:
            return self._prepare(done, started, limit, rows, wanted_rows)
        finally:
            if tuning:
                fast.set_library_tuning(0)
                done.update({f"library_{k}": v for k, v in fast.library_stats().items()})

    def _prepare(self, done: Dict[str, float], started: float, limit: int, rows: int, wanted_rows: int) -> Dict[str, float]:
        import time

        cache, plan = self.cache, self.model.plan
        if self.enable_graphs:
            for bucket in self._buckets:
                self._capture(bucket)
            done["graphs"] = len(self._buckets)
            if self.mixed_graphs:
                shapes = [(t, r) for t in self._mixed_tokens if t <= max(limit, self._mixed_tokens[0]) for r in self._mixed_rows]
                for tokens, rows_here in shapes:
                    self._capture_mixed(tokens, rows_here)
                done["step_graphs"] = len(shapes)
            done["capture_s"] = time.perf_counter() - started
        # prompts: the largest first (every scratch tensor at its largest), then one per bucket of rows of
        # the vendor library's plans, the smallest (64 tokens: the kernels of few rows) last
        fits = min(limit, plan.max_positions - 1, min(g.pool.free_count for g in cache.groups) * cache.page_size
                   if cache.groups else limit)
        sizes = sorted({fits} | set(range(64, fits, 64)), reverse=True) if fits >= 1 else []
        if self.model.dtype != torch.bfloat16:
            sizes = sizes[:1] + ([64] if fits > 64 else [])      # no library plans on the 32-bit path
        prompt_started = time.perf_counter()
        for tokens in sizes:
            if not cache.can_admit(tokens, tokens):
                continue
            slot = self.admit(tokens, tokens)
            try:
                self.step([StepEntry(slot, np.zeros(tokens, dtype=np.int64), want=list(range(min(tokens, wanted_rows, rows))))])
            finally:
                self.release(slot)
        torch.cuda.synchronize(self.device)
        done["prompt_steps"] = len(sizes)
        done["prompt_s"] = time.perf_counter() - prompt_started
        done["seconds"] = time.perf_counter() - started
        return done

    # ------------------------------------------------------------------ the step
    # (no_grad, not inference_mode: at a graph capture torch makes tensors of its own, the random
    # generator's state, which a later capture by the caller, outside inference mode, has to update:
    # tensors made inside inference mode would refuse that)
    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the entries as one batch. Returns fp32 logits ``[wanted, vocab]`` in the order of
        the entries and of their ``want``; the tensor is scratch memory and is overwritten by
        the next step. ``logit_slots`` then holds, on the device, the slot of the request that each
        row of logits belongs to (until the next step, like the logits)."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        bucket = self._graph_bucket(entries)
        mixed = self._mixed_bucket(entries) if bucket is None else None
        if bucket is not None:
            logits = self._step_graph(entries, bucket)
            starts = [self.held[e.slot] for e in entries]
        elif mixed is not None:
            logits, starts = self._step_mixed(entries, *mixed)
        else:
            batch = self.build_batch(entries)
            logits = self.model.forward(batch, self.layer_caches)
            self.logit_slots = batch.logit_slot
            starts = batch.host["starts"]
        for e, start in zip(entries, starts):
            self.held[e.slot] = start + len(e.tokens)
            self.cache.trim(e.slot, self.held[e.slot])
        return logits

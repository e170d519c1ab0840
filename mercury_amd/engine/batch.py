"""The batch of one step: flat tokens plus per-sequence bookkeeping, on the device.

A step runs, as one batch, the next tokens of any number of requests: portions of prompts of
any length beside single decoded tokens.  Activations are flat [T, H]; everything that knows
which token belongs to which request lives here
(reference: the flat token layout of mercury/model/qwen2.py:118-122 and the per-request
tensors of mercury/runner.py:112-160, which run prompts and decoding as separate forwards).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


class BatchError(ValueError):
    """A step that cannot be run as given: a token id or position out of range, a wanted
    place outside a sequence's tokens, pages missing from a block table."""


@dataclass
class SeqChunk:
    """The next tokens of one request.

    key     the request's key in the cache manager
    tokens  token ids to run now, at absolute positions start .. start + len - 1
    start   how many tokens of the request earlier steps have run (they are in the cache)
    want    indices into `tokens` whose logits the caller wants
    """

    key: object
    tokens: list
    start: int
    want: list = field(default_factory=list)


class StepContext:
    """Device-side description of a step (all index tensors int32).

    token_ids, positions, token_seq   per token: id, absolute position, index of its sequence
    cu_q        [S+1] prefix sums of the sequences' token counts (sequence s owns tokens
                cu_q[s] .. cu_q[s+1]-1, in order)
    kv_len      [S] tokens of the sequence in the cache once this step's are written
    state_slots [S] the sequence's state slot
    logit_rows  [n] flat token indices whose logits are returned, in caller order
    block_tables  per cache group: [S, W] page ids (-1 = none / given back)
    spans       host list of (first token, count, start position) per sequence
    """

    def __init__(self):
        self.num_tokens = self.num_seqs = self.num_logit_rows = 0
        self.token_ids = self.positions = self.token_seq = None
        self.cu_q = self.kv_len = self.state_slots = self.logit_rows = None
        self.block_tables: list = []
        self.spans: list = []
        self.max_q_len = self.max_kv_len = 0
        self.all_decode = False
        self.fresh_slots: list = []
        self._tiles: dict = {}

    def tiles(self, group: int, rows: int = 16):
        """(tile_seq, tile_row0, count) for attention tiles of `rows` rows, a row being a
        (token, head within a group of `group` query heads) pair: sequence s with n tokens
        this step has ceil(n * group / rows) tiles."""
        cached = self._tiles.get((group, rows))
        if cached is None:
            seqs, firsts = [], []
            for s, (_first, count, _start) in enumerate(self.spans):
                n = -(-count * group // rows)
                seqs.extend([s] * n)
                firsts.extend(range(0, rows * n, rows))
            device = self.token_ids.device
            both = torch.tensor([seqs, firsts], dtype=torch.int32).to(device, non_blocking=True)
            cached = (both[0], both[1], len(seqs))
            self._tiles[(group, rows)] = cached
        return cached


class PackedStep:
    """A step flattened into one int32 host buffer (pinned when a GPU will read it), with the
    offsets of its parts: token ids, positions, token -> sequence, prefix sums of the
    sequences' token counts, lengths, state slots, wanted rows, one block table per group."""

    def __init__(self, host, sizes, num_tokens, num_seqs, num_rows, widths, spans, max_q_len,
                 max_kv_len, fresh_slots):
        self.host, self.sizes = host, sizes
        self.num_tokens, self.num_seqs, self.num_rows = num_tokens, num_seqs, num_rows
        self.widths, self.spans = widths, spans
        self.max_q_len, self.max_kv_len, self.fresh_slots = max_q_len, max_kv_len, fresh_slots

    def layout(self):
        """What must be equal for two steps to share device buffers (and a captured graph)."""
        return (self.num_tokens, self.num_seqs, self.num_rows, tuple(self.widths))


def pack_step(chunks: list, manager, vocab_size: int, max_positions: int, pinned: bool = True,
              table_width: int | None = None) -> PackedStep:
    """Flatten `chunks` into one packed int32 host buffer.  `table_width` fixes the number of
    columns of every block table (default: as many as the longest sequence needs)."""
    if not chunks:
        raise BatchError("a step needs at least one sequence")
    num_seqs = len(chunks)
    counts = [len(c.tokens) for c in chunks]
    if min(counts) <= 0:
        raise BatchError("every sequence of a step needs at least one token")
    total = sum(counts)
    n_groups = len(manager.groups)
    ps = manager.page_size

    cu = np.zeros(num_seqs + 1, dtype=np.int64)
    np.cumsum(counts, out=cu[1:])
    if total == num_seqs:
        ids = np.fromiter((c.tokens[0] for c in chunks), dtype=np.int64, count=num_seqs)
    else:
        ids = np.concatenate([np.asarray(c.tokens, dtype=np.int64) for c in chunks])
    if ids.min() < 0 or ids.max() >= vocab_size:
        raise BatchError(f"token id outside [0, {vocab_size})")
    starts = np.asarray([c.start for c in chunks], dtype=np.int64)
    kv_len = starts + np.asarray(counts, dtype=np.int64)
    if starts.min() < 0 or kv_len.max() > max_positions:
        raise BatchError(f"a sequence would reach {int(kv_len.max())} tokens; the limit is {max_positions}")
    token_seq = np.repeat(np.arange(num_seqs, dtype=np.int64), counts)
    positions = np.arange(total, dtype=np.int64) - cu[token_seq] + starts[token_seq]
    rows = []
    for s, c in enumerate(chunks):
        for w in c.want:
            if not 0 <= w < counts[s]:
                raise BatchError(f"wanted index {w} outside the {counts[s]} tokens of a sequence")
            rows.append(int(cu[s]) + w)
        if len(set(c.want)) != len(c.want):
            # The final norm folds the last projection's partial sums into a wanted row of the
            # residual stream; a row named twice would receive them twice.
            raise BatchError(f"sequence {c.key!r} wants the same place twice: {sorted(c.want)}")
    slots = [manager.sequence(c.key).state_slot for c in chunks]

    needed = max(-(-int(kv) // ps) for kv in kv_len)
    width = needed if table_width is None else table_width
    if width < needed:
        raise BatchError(f"block tables of width {width} cannot hold {needed} pages")
    tables = []
    needs = (-(-kv_len // ps)).tolist()
    for g in range(n_groups):
        t = np.full((num_seqs, width), -1, dtype=np.int64)
        for s, c in enumerate(chunks):
            pages = manager.table(c.key, g)
            need = needs[s]
            if len(pages) < need:
                raise BatchError(
                    f"sequence {c.key!r} holds {len(pages)} pages in group {g} but needs {need}")
            t[s, :need] = pages if len(pages) == need else pages[:need]
        tables.append(t)

    parts = [ids, positions, token_seq, cu, kv_len, np.asarray(slots, dtype=np.int64),
             np.asarray(rows, dtype=np.int64)] + [t.reshape(-1) for t in tables]
    sizes = [p.size for p in parts]
    host = torch.empty(sum(sizes), dtype=torch.int32, pin_memory=pinned)
    np.concatenate(parts, out=host.numpy().reshape(-1), casting="unsafe")
    spans = [(int(cu[s]), counts[s], int(starts[s])) for s in range(num_seqs)]
    fresh = [slots[s] for s in range(num_seqs) if starts[s] == 0]
    return PackedStep(host, sizes, total, num_seqs, len(rows), [width] * n_groups, spans,
                      max(counts), int(kv_len.max()), fresh)


def context_from_packed(packed: PackedStep, on_device: torch.Tensor) -> StepContext:
    """Slice a step context out of the device copy of a packed step."""
    views, offset = [], 0
    for size in packed.sizes:
        views.append(on_device[offset:offset + size])
        offset += size
    step = StepContext()
    step.num_tokens, step.num_seqs, step.num_logit_rows = packed.num_tokens, packed.num_seqs, packed.num_rows
    (step.token_ids, step.positions, step.token_seq, step.cu_q, step.kv_len, step.state_slots,
     step.logit_rows) = views[:7]
    step.block_tables = [views[7 + g].view(packed.num_seqs, w) for g, w in enumerate(packed.widths)]
    step.spans = packed.spans
    step.max_q_len, step.max_kv_len = packed.max_q_len, packed.max_kv_len
    step.all_decode = step.max_q_len == 1
    step.fresh_slots = packed.fresh_slots
    step._packed_host = packed.host  # keeps the pinned buffer alive until the copy has run
    return step


def build_step(chunks: list, manager, vocab_size: int, max_positions: int, device,
               pinned: bool = True) -> StepContext:
    """Pack `chunks`, copy the buffer to the device once, and slice the context out of it."""
    packed = pack_step(chunks, manager, vocab_size, max_positions,
                       pinned and torch.device(device).type == "cuda")
    return context_from_packed(packed, packed.host.to(device, non_blocking=True))

"""The batch of one step: flat tokens plus per-sequence bookkeeping, on the device.

A step runs, as one batch, the next tokens of any number of requests: portions of prompts of
any length beside single decoded tokens.  Activations are flat [T, H]; everything that knows
which token belongs to which request lives here.  The host core packs a step into one int32
buffer (``csrc/host/step_batch.*``) that a single copy takes to the device; this module
describes what goes in (:class:`SeqChunk`) and gives Python-run layers and tests a view of
what came out (:class:`StepContext`).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..hostcore import core as _core

BatchError = _core.BatchError
"""A step that cannot be run as given: a token id or position out of range, a wanted place
outside a sequence's tokens or named twice, pages missing from a block table."""


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
            seqs, firsts = _core.build_tiles([count for _f, count, _s in self.spans], group, rows)
            device = self.token_ids.device
            both = torch.tensor([seqs, firsts], dtype=torch.int32).to(device, non_blocking=True)
            cached = (both[0], both[1], len(seqs))
            self._tiles[(group, rows)] = cached
        return cached


    def as_view(self, program=None) -> dict:
        """The step by device address, as ``Program.run_on`` takes it; with the row-tile lists
        `program` needs for a step of this shape."""
        ptr = lambda t: 0 if t is None else t.data_ptr()
        counts = [count for _first, count, _start in self.spans]
        tiles = []
        if program is not None:
            for group, rows in program.tile_needs(counts, self.max_q_len, self.max_kv_len):
                seq, row0, count = self.tiles(group, rows)
                tiles.append((group, rows, ptr(seq), ptr(row0), count))
        return {
            "counts": counts, "num_rows": self.num_logit_rows,
            "max_q_len": self.max_q_len, "max_kv_len": self.max_kv_len,
            "token_ids": ptr(self.token_ids), "positions": ptr(self.positions),
            "token_seq": ptr(self.token_seq), "cu_q": ptr(self.cu_q), "kv_len": ptr(self.kv_len),
            "state_slots": ptr(self.state_slots), "logit_rows": ptr(self.logit_rows),
            "tables": [(ptr(t), t.shape[1]) for t in self.block_tables],
            "tiles": tiles,
        }


def context_from_packed(packed, ints: torch.Tensor) -> StepContext:
    """A step context over `ints`, the int32 tensor (on the device, or on the host for tests)
    that holds the packed step."""
    offsets = packed.offsets

    def part(name):
        offset, count = offsets[name]
        return ints[offset:offset + count]

    step = StepContext()
    step.num_tokens, step.num_seqs = packed.num_tokens, packed.num_seqs
    step.num_logit_rows = packed.num_rows
    step.token_ids, step.positions = part("token_ids"), part("positions")
    step.token_seq, step.cu_q, step.kv_len = part("token_seq"), part("cu_q"), part("kv_len")
    step.state_slots, step.logit_rows = part("state_slots"), part("logit_rows")
    step.block_tables = [ints[offset:offset + rows * width].view(rows, width)
                         for offset, rows, width in offsets["tables"]]
    for group, tile_rows, count, off_seq, off_row0 in offsets["tiles"]:
        step._tiles[(group, tile_rows)] = (ints[off_seq:off_seq + count],
                                           ints[off_row0:off_row0 + count], count)
    step.spans = packed.spans
    step.max_q_len, step.max_kv_len = packed.max_q_len, packed.max_kv_len
    step.all_decode = step.max_q_len == 1
    step.fresh_slots = packed.fresh_slots
    return step


def host_ints(packed) -> torch.Tensor:
    """The packed step's buffer as an int32 tensor on the host (a copy)."""
    return torch.tensor(packed.host_list(), dtype=torch.int32)


def build_step(chunks: list, manager, vocab_size: int, max_positions: int, device) -> StepContext:
    """Pack `chunks` against `manager` and copy them to `device`: a step context for running
    a part or a layer by itself, outside a model's program."""
    device = torch.device(device)
    packer = _core.StepPacker(manager, vocab_size, max_positions, pinned=device.type == "cuda")
    packed = packer.pack(chunks)
    ints = torch.empty(packed.total, dtype=torch.int32, device=device)
    if device.type == "cuda":
        packer.upload(packed, ints.data_ptr(), torch.cuda.current_stream(device).cuda_stream)
        torch.cuda.current_stream(device).synchronize()
    else:
        ints.copy_(host_ints(packed))
    return context_from_packed(packed, ints)

"""The step function: run a batch of next tokens through the model, from the cache, and
return the logits at the wanted places.

`ModelRunner` owns the device memory that outlives a step: the paged key/value tensors of
every cache slot and the per-request state tensors.  It runs only the tokens it is given;
everything earlier comes from the cache that earlier steps left
(reference: mercury/runner.py:106-178 runs prompts and decoding as separate forwards and
returns sampled tokens; here one forward takes any mix and returns logits).
"""

from __future__ import annotations

import numpy as np
import torch

from ..parts.base import LayerCache
from .batch import (BatchError, SeqChunk, StepContext, build_step, context_from_packed,
                    pack_step)


class DecodeGraph:
    """One captured HIP graph of a decode-only step (one token per sequence) for a fixed
    number of sequences and a fixed bound on their length.

    The step's index tensors live in one static device buffer that every replay refills with a
    single copy; block tables have the full width of the longest sequence the engine allows,
    and the number of key splits of the attention kernel is the one chosen for the length
    bound, so any shorter step replays the same launches.
    """

    def __init__(self, runner, packed, kv_bound: int):
        self.layout = packed.layout()
        self.static = torch.empty(packed.host.shape, dtype=torch.int32, device=runner.device)
        self.static.copy_(packed.host, non_blocking=True)
        self.ctx = context_from_packed(packed, self.static)
        self.ctx.max_kv_len = kv_bound
        self.ctx.fresh_slots = []
        # The host's copy of the step, kept between replays: a replay rewrites the few
        # numbers that change (token ids, positions, lengths, new pages) and copies it whole.
        self.host = torch.empty(packed.host.shape, dtype=torch.int32, pin_memory=True)
        self.host.copy_(packed.host)
        views, offset = [], 0
        for size in packed.sizes:
            views.append(self.host.numpy()[offset:offset + size])
            offset += size
        self.ids, self.positions, _seq, _cu, self.kv_len, self.slots, _rows = views[:7]
        n = packed.num_seqs
        self.tables = [views[7 + g].reshape(n, w) for g, w in enumerate(packed.widths)]
        self.copied = None                                 # the last copy of `host` to the device
        self.row_record = [None] * n                       # whose pages a table row mirrors
        self.row_pages = [[0] * n for _ in packed.widths]  # and how many of them
        self.appendable = [g.window is None for g in runner.manager.groups]
        # Once outside the capture: loads libraries, fills the context's tile tables.
        side = torch.cuda.Stream(device=runner.device)
        side.wait_stream(torch.cuda.current_stream(runner.device))
        with torch.cuda.stream(side):
            runner.model.forward(self.ctx, runner.caches, runner.states)
        torch.cuda.current_stream(runner.device).wait_stream(side)
        torch.cuda.synchronize(runner.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.model.forward(self.ctx, runner.caches, runner.states)

    def refill(self, chunks: list, manager, vocab_size: int, max_positions: int,
               ids_on_device: bool = False) -> None:
        """Write this step's numbers into the host copy, once the previous replay's copy to
        the device has finished.  With `ids_on_device` the token ids are not the chunks'."""
        if self.copied is not None:
            self.copied.synchronize()
        n = len(chunks)
        if not ids_on_device:
            self.ids[:] = [c.tokens[0] for c in chunks]
            if self.ids.min() < 0 or self.ids.max() >= vocab_size:
                raise BatchError(f"token id outside [0, {vocab_size})")
        self.positions[:] = [c.start for c in chunks]
        if self.positions.min() < 0 or self.positions.max() >= max_positions:
            raise BatchError(f"a sequence would pass the limit of {max_positions} tokens")
        np.add(self.positions, 1, out=self.kv_len)
        ps = manager.page_size
        for s in range(n):
            c = chunks[s]
            record = manager.sequence(c.key)
            need = c.start // ps + 1
            # a key stands for one admission: its state slot and pages change only by growing
            same = (c.key, record.state_slot) == self.row_record[s]
            if not same:
                self.row_record[s] = (c.key, record.state_slot)
                self.slots[s] = record.state_slot
            for g, table in enumerate(self.tables):
                have = self.row_pages[g][s]
                if same and self.appendable[g] and have == need:
                    continue
                pages = record.tables[g]
                if len(pages) < need:
                    raise BatchError(
                        f"sequence {c.key!r} holds {len(pages)} pages in group {g} but needs {need}")
                if same and self.appendable[g] and have < need:
                    table[s, have:need] = pages[have:need]
                else:
                    table[s, :need] = pages[:need]
                    table[s, need:] = -1
                self.row_pages[g][s] = need

    def replay(self, ids: torch.Tensor | None = None) -> torch.Tensor:
        """Copy the step to the device and run the graph; `ids` (int32 on the device, one per
        sequence) replace the token ids of the host copy."""
        self.static.copy_(self.host, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()
        if ids is not None:
            self.ctx.token_ids.copy_(ids)
        self.graph.replay()
        return self.logits


def require_gpu(device: torch.device) -> None:
    if device.type != "cuda":
        raise RuntimeError(
            f"the step function runs hand-written GPU kernels only; device {device} is not a GPU")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to this process; there is no CPU path")


class ModelRunner:
    def __init__(self, model, manager, dtype: torch.dtype, device, max_model_len: int,
                 use_graphs: bool = True, max_graph_batch: int = 256):
        device = torch.device(device)
        require_gpu(device)
        self.graphs: dict = {}
        self.use_graphs = bool(use_graphs) and all(
            getattr(layer, "graph_safe", False) for layer in model.layers)
        self.max_graph_batch = int(max_graph_batch)
        self.last_prepare_seconds = 0.0
        self.model, self.manager = model, manager
        self.dtype, self.device = dtype, device
        self.max_model_len = int(max_model_len)
        self.page_size = manager.page_size
        model.prepare(self.max_model_len, device)

        # Paged keys [pages, kv_heads, page, head_dim] and values [pages, kv_heads, head_dim,
        # page] per cache slot.
        self.kv = {}
        for slot, spec in model.cache_slots.items():
            pages = manager.groups[manager.group_of(slot)].pool.num_pages
            kv_dtype = spec.dtype or dtype
            self.kv[slot] = (
                torch.zeros((pages, spec.kv_heads, self.page_size, spec.head_dim), dtype=kv_dtype, device=device),
                torch.zeros((pages, spec.kv_heads, spec.v_dim, self.page_size), dtype=kv_dtype, device=device))
        self.caches = {}
        for n, call in enumerate(model.calls):
            if call.cache is None:
                continue
            k, v = self.kv[call.cache]
            self.caches[n] = LayerCache(k, v, manager.group_of(call.cache), self.page_size,
                                        call.writes)
        # Per-request state of fixed size, one tensor per layer that declares it.
        self.states = {}
        for i, layer in enumerate(model.layers):
            spec = layer.mixer.state_spec()
            if spec is not None:
                self.states[i] = torch.zeros((manager.state_slots.num_slots, *spec.shape),
                                             dtype=spec.dtype, device=device)

    @property
    def kv_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for kv in self.kv.values() for t in kv)

    def kv_bytes_per_token(self) -> int:
        return sum(k.shape[1] * (k.shape[3] + v.shape[2]) * k.element_size()
                   for k, v in self.kv.values())

    def build(self, chunks: list) -> StepContext:
        return build_step(chunks, self.manager, self.model.vocab_size, self.max_model_len,
                          self.device)

    @torch.inference_mode()
    def step(self, chunks: list) -> torch.Tensor:
        """Run the chunks' tokens as one batch.  Returns float32 logits [wanted, V] in the
        order of the chunks and of each chunk's `want`.  The tensor may be overwritten by the
        next step."""
        import time

        started = time.perf_counter()
        if self._graphable(chunks):
            return self.step_graphed(chunks, started)
        ctx = self.build(chunks)
        self.last_prepare_seconds = time.perf_counter() - started
        return self.run(ctx)

    def captured(self, chunks: list) -> bool:
        """Whether `step_graphed` would replay a graph it already has for these chunks."""
        return self._graphable(chunks) and self._graph_key(chunks) in self.graphs

    @staticmethod
    def _graph_key(chunks: list) -> tuple:
        bound = 256
        longest = max(c.start for c in chunks) + 1
        while bound < longest:
            bound *= 2
        return len(chunks), bound

    def _graphable(self, chunks: list) -> bool:
        return (self.use_graphs and len(chunks) <= self.max_graph_batch
                and all(len(c.tokens) == 1 and c.want == [0] and c.start > 0 for c in chunks))

    @torch.inference_mode()
    def step_graphed(self, chunks: list, started: float | None = None,
                     ids: torch.Tensor | None = None) -> torch.Tensor:
        """A decode-only step through a captured graph (captured on first use for this number
        of sequences and length bound).  `ids`: the token ids, on the device, when the host
        does not know them yet."""
        key = self._graph_key(chunks)
        bound = key[1]
        graph = self.graphs.get(key)
        if graph is None:
            width = -(-self.max_model_len // self.page_size)
            packed = pack_step(chunks, self.manager, self.model.vocab_size, self.max_model_len,
                               pinned=True, table_width=width)
            graph = self.graphs[key] = DecodeGraph(self, packed, bound)
        graph.refill(chunks, self.manager, self.model.vocab_size, self.max_model_len,
                     ids_on_device=ids is not None)
        if started is not None:
            import time

            self.last_prepare_seconds = time.perf_counter() - started
        return graph.replay(ids)

    @torch.inference_mode()
    def run(self, ctx: StepContext) -> torch.Tensor:
        if self.states and ctx.fresh_slots:
            index = torch.tensor(ctx.fresh_slots, device=self.device)
            for state in self.states.values():
                state.index_fill_(0, index, 0)
        return self.model.forward(ctx, self.caches, self.states)


__all__ = ["ModelRunner", "SeqChunk", "StepContext"]

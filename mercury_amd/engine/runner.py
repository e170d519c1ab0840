"""The step function: run a batch of next tokens through the model, from the cache, and
return the logits at the wanted places.

`ModelRunner` owns the device memory that outlives a step: the paged key/value tensors of
every cache slot, the per-request state tensors, the step's index buffer and the workspace its
operations write into.  A step is packed by the host core into one int32 buffer, copied to the
device once, and launched by the host core as one walk over the model's program; parts that
do not hand their work over (parts defined outside the package without operations of their
own) are run from here in between, on the same registers.  It runs only the tokens it is given; everything
earlier comes from the cache that earlier steps left
(reference: mercury/runner.py:106-178 runs prompts and decoding as separate forwards and
returns sampled tokens; here one forward takes any mix and returns logits).
"""

from __future__ import annotations

import time

import torch

from ..hostcore import core as _core
from ..kernels import lib as _lib
from ..kernels import ops
from collections import OrderedDict

from ..parts.base import LayerCache
from ..parts.model import Registers
from .batch import BatchError, SeqChunk, StepContext, context_from_packed


def require_gpu(device: torch.device) -> None:
    if device.type != "cuda":
        raise RuntimeError(
            f"the step function runs hand-written GPU kernels only; device {device} is not a GPU")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to this process; there is no CPU path")


class _Buffers:
    """The device memory one in-flight step uses: its index buffer and its workspace, grown
    when a larger step comes."""

    def __init__(self, device, num_ints: int = 1 << 14, num_bytes: int = 1 << 20):
        self.device = device
        self.ints = torch.empty(num_ints, dtype=torch.int32, device=device)
        self.workspace = torch.empty(num_bytes, dtype=torch.uint8, device=device)

    def fits(self, num_ints: int, num_bytes: int) -> bool:
        return self.ints.numel() >= num_ints and self.workspace.numel() >= num_bytes

    def fit(self, num_ints: int, num_bytes: int) -> None:
        if self.ints.numel() < num_ints:
            self.ints = torch.empty(num_ints + num_ints // 4, dtype=torch.int32, device=self.device)
        if self.workspace.numel() < num_bytes:
            self.workspace = torch.empty(num_bytes + num_bytes // 4, dtype=torch.uint8,
                                         device=self.device)

    @property
    def nbytes(self) -> int:
        return self.ints.numel() * 4 + self.workspace.numel()

    def view(self, address: int, shape: tuple, dtype=torch.float32) -> torch.Tensor:
        """The tensor of `shape` at device address `address` inside the workspace."""
        offset = address - self.workspace.data_ptr()
        count = 1
        for n in shape:
            count *= n
        size = count * torch.empty((), dtype=dtype).element_size()
        if offset < 0 or offset + size > self.workspace.numel():
            raise RuntimeError("a step's result lies outside its workspace")
        return self.workspace[offset:offset + size].view(dtype).view(*shape)


class DecodeGraph:
    """One captured HIP graph of a decode-only step (one token per sequence) for a fixed
    number of sequences and a fixed bound on their length.

    Block tables have the full width of the longest sequence the engine allows, and the
    number of key splits of the attention kernel is the one chosen for the length bound, so
    any shorter step packs into the same layout and replays the same launches.  The index
    buffer and the workspace are the runner's, shared by all its graphs: replays are serial on
    one stream, and whoever reads a replay's logits does so on that stream before the next.
    """

    def __init__(self, runner, packed, buffers: _Buffers):
        self.layout = packed.layout()
        self.buffers = buffers
        self.ids_at = packed.offsets["token_ids"][0]
        self.num_seqs = packed.num_seqs
        stream = torch.cuda.current_stream(runner.device)
        runner.packer.upload(packed, buffers.ints.data_ptr(), stream.cuda_stream)
        # Once outside the capture (loads libraries, warms the kernels), then captured.
        side = torch.cuda.Stream(device=runner.device)
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            runner.launch(packed, buffers)
        stream.wait_stream(side)
        torch.cuda.synchronize(runner.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.launch(packed, buffers)

    def replay(self, runner, packed, ids: torch.Tensor | None = None) -> torch.Tensor:
        """Copy the step to the device and run the graph; `ids` (int32 on the device, one per
        sequence) replace the token ids of the packed step."""
        if packed.layout() != self.layout:
            raise BatchError("a step of another shape was given to a captured graph")
        stream = torch.cuda.current_stream(runner.device).cuda_stream
        runner.packer.upload(packed, self.buffers.ints.data_ptr(), stream)
        if ids is not None:
            self.buffers.ints[self.ids_at:self.ids_at + self.num_seqs].copy_(ids)
        self.graph.replay()
        return self.logits


def sizing_caches(model, manager_groups: dict, page_size: int, dtype: torch.dtype, device) -> dict:
    """Caches without pages, for a program that is only measured: execution-list index ->
    LayerCache over empty tensors.  `manager_groups` maps a cache slot to its group."""
    caches = {}
    for n, call in enumerate(model.calls):
        if call.cache is None:
            continue
        spec = model.cache_slots[call.cache]
        kv_dtype = spec.dtype or dtype
        k = torch.empty((0, spec.kv_heads, page_size, spec.head_dim), dtype=kv_dtype, device=device)
        v = torch.empty((0, spec.kv_heads, spec.v_dim, page_size), dtype=kv_dtype, device=device)
        caches[n] = LayerCache(k, v, manager_groups[call.cache], page_size, call.writes)
    return caches


class ModelRunner:
    def __init__(self, model, manager, dtype: torch.dtype, device, max_model_len: int,
                 use_graphs: bool = True, max_graph_batch: int = 256, max_graphs: int = 96):
        device = torch.device(device)
        require_gpu(device)
        _lib.load("core")
        if dtype == torch.bfloat16:
            _lib.load("mfma")
        # captured decode graphs, least recently used first; at most `max_graphs` are kept
        self.graphs: OrderedDict = OrderedDict()
        self.max_graphs = max(2, int(max_graphs))
        self.graph_stats = {"captured": 0, "dropped": 0, "resets": 0}
        self.use_graphs = bool(use_graphs) and all(
            getattr(layer, "graph_safe", False) for layer in model.layers)
        self.max_graph_batch = int(max_graph_batch)
        self.last_prepare_seconds = 0.0
        self.model, self.manager = model, manager
        self.dtype, self.device = dtype, device
        self.max_model_len = int(max_model_len)
        self.page_size = manager.page_size
        model.prepare(self.max_model_len, device)

        # Paged keys [pages, kv_heads, page, key width] and values [pages, kv_heads, value
        # width, page] per cache slot, in the slot's own dtype or the model's.
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
        # The model as a program of the host core; parts that do not hand their work over
        # are steps this runner runs in between (model.caller_steps).
        self.program = model.compile(self.caches, self.states)
        self.packer = _core.StepPacker(manager, model.vocab_size, self.max_model_len, pinned=True)
        self.buffers = _Buffers(device)
        self.graph_buffers: _Buffers | None = None

    @property
    def kv_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for kv in self.kv.values() for t in kv)

    def kv_bytes_per_token(self) -> int:
        return sum(k.shape[1] * (k.shape[3] + v.shape[2]) * k.element_size()
                   for k, v in self.kv.values())

    # ---- what a runner needs beside weights and cache

    @staticmethod
    def step_needs(program, num_groups: int, page_size: int, max_model_len: int,
                   prefill_tokens: int, max_seqs: int, graph_batch: int) -> dict:
        """Bytes of index buffer and workspace for the largest step a scheduler with these
        limits can plan (a portion of `prefill_tokens` beside single tokens of the other
        sequences) and for the largest captured decode step."""
        width = -(-max_model_len // page_size)

        def ints_for(tokens, seqs):
            return 4 * (3 * tokens + 5 * seqs + 2 + num_groups * seqs * width + 2 * (tokens + seqs))

        tokens = prefill_tokens + max(0, max_seqs - 1)
        counts = [prefill_tokens] + [1] * max(0, max_seqs - 1)
        eager = program.workspace_bytes_for(counts, max_seqs, max_model_len, num_groups)
        graph, batch = 0, 1
        while graph_batch > 0:
            batch = min(batch, graph_batch)
            graph = max(graph, program.workspace_bytes_for([1] * batch, batch, max_model_len, num_groups))
            if batch == graph_batch:
                break
            batch *= 2
        return {"eager_workspace": eager, "eager_ints": ints_for(tokens, max_seqs),
                "graph_workspace": graph,
                "graph_ints": ints_for(graph_batch, graph_batch) if graph_batch > 0 else 0}

    def memory_report(self) -> dict:
        """Device memory this runner holds beside the weights."""
        return {
            "kv_bytes": self.kv_bytes,
            "state_bytes": sum(t.numel() * t.element_size() for t in self.states.values()),
            "step_buffer_bytes": self.buffers.nbytes,
            "graph_buffer_bytes": self.graph_buffers.nbytes if self.graph_buffers else 0,
            "graphs": len(self.graphs), "max_graphs": self.max_graphs, **self.graph_stats,
        }

    # ---- one step

    @torch.inference_mode()
    def step(self, chunks: list) -> torch.Tensor:
        """Run the chunks' tokens as one batch.  Returns float32 logits [wanted, V] in the
        order of the chunks and of each chunk's `want`.  The tensor may be overwritten by the
        next step."""
        started = time.perf_counter()
        if self._graphable([(len(c.tokens), c.start, c.want == [0]) for c in chunks]):
            key = self._graph_key(len(chunks), max(c.start for c in chunks) + 1)
            packed = self.packer.pack(chunks, self.program, self._full_width(), kv_bound=key[1])
            return self._replay(key, packed, started)
        packed = self.packer.pack(chunks, self.program)
        return self._run(packed, started)

    @torch.inference_mode()
    def step_plan(self, plan) -> torch.Tensor:
        """The same for a scheduler's plan: the logits of every work item that emits."""
        started = time.perf_counter()
        if self._graphable([(w.count, w.start, w.emits) for w in plan.work]):
            key = self._graph_key(len(plan.work), max(w.start for w in plan.work) + 1)
            packed = self.packer.pack_plan(plan, self.program, self._full_width(), kv_bound=key[1])
            return self._replay(key, packed, started)
        packed = self.packer.pack_plan(plan, self.program)
        return self._run(packed, started)

    def _run(self, packed, started: float) -> torch.Tensor:
        self.buffers.fit(packed.total, self.program.workspace_bytes(packed))
        stream = torch.cuda.current_stream(self.device).cuda_stream
        self.packer.upload(packed, self.buffers.ints.data_ptr(), stream)
        self.last_prepare_seconds = time.perf_counter() - started
        return self.launch(packed, self.buffers)

    def launch(self, packed, buffers: _Buffers) -> torch.Tensor:
        """Launch the step whose indices lie in `buffers.ints`."""
        if self.states and packed.fresh_slots:
            index = torch.tensor(packed.fresh_slots, device=self.device)
            for state in self.states.values():
                state.index_fill_(0, index, 0)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        program, ws = self.program, buffers.workspace
        tokens, hidden, vocab = packed.num_tokens, self.model.hidden_size, self.model.vocab_size
        begin, regs = 0, None
        logits = None
        while True:
            x, pending = (regs.x, regs.pending) if regs is not None else (None, None)
            stopped, h_at, logits_at, x_at, x_rows, pending_at, pending_count = program.run(
                packed, buffers.ints.data_ptr(), ws.data_ptr(), ws.numel(), stream, begin,
                0 if x is None else x.data_ptr(), 0 if x is None else x.shape[0],
                0 if pending is None else pending.data_ptr(),
                0 if pending is None else pending.shape[0])
            if logits_at:
                logits = buffers.view(logits_at, (packed.num_rows, vocab))
            if stopped >= program.num_ops:
                break
            # A step that stays with the caller: run it on the same registers.
            if regs is None:
                regs = Registers(None, None, None, context_from_packed(packed, buffers.ints))
            regs.h = buffers.view(h_at, (tokens, hidden))
            regs.x = buffers.view(x_at, (x_rows, hidden), self.dtype) if x_at else None
            regs.pending = (buffers.view(pending_at, (pending_count, tokens, hidden))
                            if pending_count else None)
            with ops.on_current_stream():
                self.model.caller_steps[program.host_index(stopped)].run(regs)
            if regs.logits is not None:
                logits = regs.logits
            begin = stopped + 1
        if packed.num_rows == 0 or logits is None:
            return torch.empty((0, vocab), dtype=torch.float32, device=self.device)
        return logits

    # ---- decode steps through captured graphs

    def _full_width(self) -> int:
        return -(-self.max_model_len // self.page_size)

    def _graphable(self, items: list) -> bool:
        """items: (count, start, wants its one token's logits) per sequence."""
        return (self.use_graphs and len(items) <= self.max_graph_batch
                and all(count == 1 and wanted and start > 0 for count, start, wanted in items))

    @staticmethod
    def _graph_key(num_seqs: int, longest: int) -> tuple:
        bound = 256
        while bound < longest:
            bound *= 2
        return num_seqs, bound

    def captured(self, num_seqs: int, longest: int) -> bool:
        """Whether a decode step of `num_seqs` sequences, the longest reaching `longest`
        tokens, would replay a graph that exists already."""
        return self.use_graphs and self._graph_key(num_seqs, longest) in self.graphs

    def _buffers_for_graphs(self, packed) -> _Buffers:
        """The one index buffer and workspace all captured graphs share, made for the largest
        decode step the runner captures.  Should a step need more after all, every graph is
        dropped (their launches hold the old addresses) and the buffers grow."""
        need = self.program.workspace_bytes(packed)
        if self.graph_buffers is None:
            sizes = self.step_needs(self.program, self.manager.num_groups, self.page_size,
                                    self.max_model_len, 1, 1, self.max_graph_batch)
            self.graph_buffers = _Buffers(self.device, max(sizes["graph_ints"] // 4, packed.total),
                                          max(sizes["graph_workspace"], need))
        elif not self.graph_buffers.fits(packed.total, need):
            torch.cuda.synchronize(self.device)
            self.graphs.clear()
            self.graph_stats["resets"] += 1
            self.graph_buffers.fit(packed.total, need)
        return self.graph_buffers

    def _replay(self, key: tuple, packed, started: float | None,
                ids: torch.Tensor | None = None) -> torch.Tensor:
        """Through the graph for `key` (captured on first use).  The step was packed with the
        key's length bound as its longest length, so that the attention's key splits, chosen at
        capture, suit every step that replays the graph."""
        graph = self.graphs.get(key)
        if graph is None:
            graph = DecodeGraph(self, packed, self._buffers_for_graphs(packed))
            self.graphs[key] = graph
            self.graph_stats["captured"] += 1
            while len(self.graphs) > self.max_graphs:
                # the least recently used; the newest and whatever ran last stay
                self.graphs.popitem(last=False)
                self.graph_stats["dropped"] += 1
        else:
            self.graphs.move_to_end(key)
        if started is not None:
            self.last_prepare_seconds = time.perf_counter() - started
        return graph.replay(self, packed, ids)

    @torch.inference_mode()
    def step_ahead(self, chunks: list, ids: torch.Tensor) -> torch.Tensor:
        """A decode step whose token ids the host does not know yet: they are `ids`, int32 on
        the device, one per chunk.  Only through a graph that exists."""
        key = self._graph_key(len(chunks), max(c.start for c in chunks) + 1)
        packed = self.packer.pack(chunks, self.program, self._full_width(), check_ids=False,
                                  kv_bound=key[1])
        return self._replay(key, packed, None, ids)


__all__ = ["ModelRunner", "SeqChunk", "StepContext"]

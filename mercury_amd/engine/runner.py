"""The step function: run a batch of next tokens through the model, from the cache, and
return the logits at the wanted places.

`ModelRunner` owns the device memory that outlives a step: the paged key/value tensors of
every cache slot, the per-request state tensors, the step's index buffer and the workspace its
operations write into.  A step is packed by the host core into one int32 buffer, copied to the
device once, and launched by the host core as one walk over the model's program; layers whose
parts do not hand their work over (parts defined outside the package, mixers with state of
their own) are run from here in between.  It runs only the tokens it is given; everything
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
from ..parts.base import LayerCache
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

    def __init__(self, device):
        self.device = device
        self.ints = torch.empty(1 << 14, dtype=torch.int32, device=device)
        self.workspace = torch.empty(1 << 20, dtype=torch.uint8, device=device)

    def fit(self, num_ints: int, num_bytes: int) -> None:
        if self.ints.numel() < num_ints:
            self.ints = torch.empty(num_ints + num_ints // 4, dtype=torch.int32, device=self.device)
        if self.workspace.numel() < num_bytes:
            self.workspace = torch.empty(num_bytes + num_bytes // 4, dtype=torch.uint8,
                                         device=self.device)

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

    The step's index buffer and workspace are the graph's own; block tables have the full
    width of the longest sequence the engine allows, and the number of key splits of the
    attention kernel is the one chosen for the length bound, so any shorter step packs into
    the same layout and replays the same launches.
    """

    def __init__(self, runner, packed, kv_bound: int):
        self.layout = packed.layout()
        self.buffers = _Buffers(runner.device)
        self.buffers.fit(packed.total, runner.program.workspace_bytes(packed))
        self.ids_at = packed.offsets["token_ids"][0]
        self.num_seqs = packed.num_seqs
        stream = torch.cuda.current_stream(runner.device)
        runner.packer.upload(packed, self.buffers.ints.data_ptr(), stream.cuda_stream)
        # Once outside the capture (loads libraries, warms the kernels), then captured.
        side = torch.cuda.Stream(device=runner.device)
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            runner.launch(packed, self.buffers)
        stream.wait_stream(side)
        torch.cuda.synchronize(runner.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = runner.launch(packed, self.buffers)

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


class ModelRunner:
    def __init__(self, model, manager, dtype: torch.dtype, device, max_model_len: int,
                 use_graphs: bool = True, max_graph_batch: int = 256):
        device = torch.device(device)
        require_gpu(device)
        _lib.load("core")
        if dtype == torch.bfloat16:
            _lib.load("mfma")
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
        # The model as a program of the host core (None: every layer is run from here).
        self.program = model.compile(self.caches, self.states)
        self.packer = _core.StepPacker(manager, model.vocab_size, self.max_model_len, pinned=True)
        self.buffers = _Buffers(device)

    @property
    def kv_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for kv in self.kv.values() for t in kv)

    def kv_bytes_per_token(self) -> int:
        return sum(k.shape[1] * (k.shape[3] + v.shape[2]) * k.element_size()
                   for k, v in self.kv.values())

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
        need = self.program.workspace_bytes(packed) if self.program is not None else 0
        self.buffers.fit(packed.total, need)
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
        if self.program is None:
            ctx = context_from_packed(packed, buffers.ints)
            return self.model.forward(ctx, self.caches, self.states)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        program, ws = self.program, buffers.workspace
        begin, pending, ctx = 0, None, None
        tokens, hidden = packed.num_tokens, self.model.hidden_size
        while True:
            stopped, h_at, logits_at, pending_at, pending_count = program.run(
                packed, buffers.ints.data_ptr(), ws.data_ptr(), ws.numel(), stream, begin,
                0 if pending is None else pending.data_ptr(),
                0 if pending is None else pending.shape[0])
            if stopped >= program.num_ops:
                break
            # A layer that stays with the caller: run it on the same residual stream.
            if ctx is None:
                ctx = context_from_packed(packed, buffers.ints)
            h = buffers.view(h_at, (tokens, hidden))
            if pending_count:
                pending = buffers.view(pending_at, (pending_count, tokens, hidden))
            else:
                pending = None
            n = program.host_index(stopped)
            call = self.model.calls[n]
            with ops.on_current_stream():
                pending = self.model.layers[call.layer].forward(
                    h, ctx, self.caches.get(n), self.states.get(call.layer), self.dtype, pending)
            begin = stopped + 1
        if packed.num_rows == 0:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        return buffers.view(logits_at, (packed.num_rows, self.model.vocab_size))

    # ---- decode steps through captured graphs

    def _full_width(self) -> int:
        return -(-self.max_model_len // self.page_size)

    def _graphable(self, items: list) -> bool:
        """items: (count, start, wants its one token's logits) per sequence."""
        return (self.use_graphs and self.program is not None and len(items) <= self.max_graph_batch
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

    def _replay(self, key: tuple, packed, started: float | None,
                ids: torch.Tensor | None = None) -> torch.Tensor:
        """Through the graph for `key` (captured on first use).  The step was packed with the
        key's length bound as its longest length, so that the attention's key splits, chosen at
        capture, suit every step that replays the graph."""
        graph = self.graphs.get(key)
        if graph is None:
            graph = self.graphs[key] = DecodeGraph(self, packed, key[1])
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

"""The engine: the public entry point around the host core's loop.

The host core (C++) keeps the requests, the scheduler, the cache bookkeeping and the step log;
it decides, and reports what happened as a list of events.  This class owns what is Python's
to own: the command queue through which other threads talk to the engine thread, the optional
engine thread itself, the per-request sinks the events are delivered to, and the executor that
runs a plan on the GPU (reference for the API and its meanings: mercury/engine.py:28-300).

    engine = Engine(EngineConfig(model=folder))
    engine.submit(rid, prompt_ids, max_tokens, sink)      # from any thread
    engine.step()                                         # or engine.start() for a thread
    tokens = engine.generate([[1, 2, 3]], SamplingParams(), max_tokens=16)   # blocking
"""

from __future__ import annotations

import threading
import time
from collections import deque
from typing import Callable

from ..cache import CacheManager, PageHasher
from ..config.engine_config import EngineConfig
from ..hostcore import core as _core

StreamEvent = _core.StreamEvent
SamplingParams = _core.SamplingParams
Sink = Callable[[StreamEvent], None]


# What the captured decode graphs may cost beside the buffers they share: the launch records
# of a few hundred kernels each (measured well under a megabyte a graph).
GRAPH_RECORD_BYTES = 2 << 20


def autosize_blocks(cfg: EngineConfig, kv_bytes_per_token: int, device, reserve_bytes: int = 0) -> int:
    """Pages that fit in the memory that is free once the weights are resident, after
    `reserve_bytes` are set aside for what is allocated later: the workspace and index buffer
    of the largest step, the buffers the captured graphs share, and the graphs themselves
    (reference: mercury/config.py:164-185, which reserves for weights not yet loaded; here
    the weights are loaded when this is called, and the reservation is for the rest)."""
    import torch

    free, _total = torch.cuda.mem_get_info(torch.device(device))
    budget = int(max(0, free - reserve_bytes) * cfg.gpu_memory_fraction)
    per_page = max(1, kv_bytes_per_token * cfg.block_size)
    pages = budget // per_page
    if pages < 1:
        raise RuntimeError(
            f"only {free / 2**30:.1f} GiB are free and {reserve_bytes / 2**30:.1f} GiB are set "
            f"aside for the steps' buffers; there is no room for a cache")
    return pages


class _Inbox:
    """What other threads ask of the loop, in the order they asked: the loop takes everything
    at once at the top of a pass, and sleeps on the inbox when it has nothing to run."""

    def __init__(self):
        self._items: deque = deque()
        self._ready = threading.Condition()

    def post(self, kind: str, payload) -> None:
        with self._ready:
            self._items.append((kind, payload))
            self._ready.notify()

    def take_all(self) -> list:
        with self._ready:
            items = list(self._items)
            self._items.clear()
        return items

    def wait(self, timeout: float) -> None:
        with self._ready:
            if not self._items:
                self._ready.wait(timeout)


class Engine:
    """`Engine(cfg)` loads the model folder `cfg.model` onto the GPU, or, with
    `cfg.random_weights`, builds the model that `model_config` (a ``config.json`` as a dict) or
    the ``config.json`` at `cfg.model` describes and draws its weights from `cfg.weight_seed`.
    Tests pass `executor` (anything with `execute(plan)`) and, with it, the cache manager it
    checks against.

    One pass of the loop is `step()`.  Whoever calls it owns the loop: the caller's own
    thread (`step`, `run_until_idle`, `generate`), or, after `start()`, a thread of the
    engine's that runs passes until `shutdown()`.  `submit` and `abort` may come from any
    thread either way; they only post to the inbox."""

    def __init__(self, cfg: EngineConfig, executor=None, manager: CacheManager | None = None,
                 clock: Callable[[], float] = time.perf_counter, eos_token_ids=None,
                 model_config: dict | None = None):
        self.cfg = cfg
        self.clock = clock
        self.hasher = PageHasher(cfg.block_size, cfg.cryptographic_hashes)
        if executor is None:
            executor, manager, eos = self._load(cfg, model_config)
            eos_token_ids = eos if eos_token_ids is None else eos_token_ids
        elif manager is None:
            raise ValueError("an engine with its own executor needs the cache manager it uses")
        self.executor, self.manager = executor, manager
        self.runner = executor  # the reference's name for this seam
        self.core = _core.EngineCore(
            manager, self.hasher, policy=cfg.policy, max_running=cfg.max_running,
            prefill_budget=cfg.prefill_budget, aging_tokens_per_s=cfg.aging_tokens_per_s,
            max_wait_s=cfg.max_wait_s, scan_limit=cfg.scan_limit,
            max_model_len=cfg.max_model_len, eos_ids=sorted(eos_token_ids or ()),
            max_step_records=cfg.max_step_records)
        self.sched = self.core.scheduler
        self.metrics = self.core      # counters, summary(), step_records()
        self._inbox = _Inbox()
        self._listeners: dict = {}                  # request id -> sink
        self._listeners_guard = threading.Lock()
        self._accepted = 0                          # requests submit() has queued so far
        self._worker: threading.Thread | None = None
        self._serving = threading.Event()
        self._worker_error: BaseException | None = None

    @property
    def eos_ids(self) -> set:
        """Token ids that end a request (unless it asked to ignore them)."""
        return set(self.core.eos_ids)

    @eos_ids.setter
    def eos_ids(self, ids) -> None:
        self.core.eos_ids = sorted(ids)

    @staticmethod
    def _load(cfg: EngineConfig, model_config: dict | None):
        import torch

        from ..config.model_config import read_config_json
        from ..config.registry import build_model
        from ..sampling.sampler import Sampler
        from ..weights.loader import load_model_folder, load_weights
        from ..weights.random_init import RandomSource
        from .executor import GpuExecutor
        from .runner import ModelRunner, require_gpu

        device = torch.device(cfg.device)
        require_gpu(device)
        if cfg.random_weights:
            model = build_model(model_config if model_config is not None
                                else read_config_json(cfg.model))
            from ..config.engine_config import _DTYPE_BY_NAME

            stored = _DTYPE_BY_NAME[cfg.weight_dtype]
            load_weights(model, RandomSource(model, cfg.weight_seed, cfg.weight_std, stored, device),
                         cfg.torch_dtype, device)
        elif model_config is not None:
            raise ValueError("model_config is only for random_weights; a model folder brings its own")
        else:
            model = load_model_folder(cfg.model, cfg.torch_dtype, device)
        if model.max_positions:
            cfg.validate_against(model.max_positions)
        has_state = any(layer.mixer.state_spec() is not None for layer in model.layers)
        graph_batch = min(cfg.max_graph_batch, cfg.max_running)
        if cfg.num_blocks < 0:
            reserve = Engine.reserve_bytes(model, cfg, device, graph_batch)
            cfg.extra["reserved_bytes"] = reserve
            cfg.num_blocks = autosize_blocks(cfg, model.kv_bytes_per_token(cfg.torch_dtype), device,
                                             reserve)
            cfg.validate_against(model.max_positions or cfg.max_model_len)
        manager = CacheManager(model.cache_slots, cfg.num_blocks, cfg.block_size, cfg.max_running,
                               has_state)
        runner = ModelRunner(model, manager, cfg.torch_dtype, device, cfg.max_model_len,
                             use_graphs=cfg.use_graphs, max_graph_batch=graph_batch,
                             max_graphs=cfg.max_graphs)
        return (GpuExecutor(runner, Sampler(cfg.seed), lookahead=cfg.lookahead), manager,
                model.eos_token_ids)

    @staticmethod
    def reserve_bytes(model, cfg: EngineConfig, device, graph_batch: int) -> int:
        """Device memory the engine will allocate after the cache: measured on the model's
        program, built over caches without pages, for the largest step the scheduler can plan
        under `prefill_budget` and `max_running` and for the largest captured decode step."""
        import torch

        from ..kernels import lib as kernel_lib
        from .runner import ModelRunner, sizing_caches

        kernel_lib.load("core")
        if cfg.torch_dtype == torch.bfloat16:
            kernel_lib.load("mfma")
        # the groups as the cache manager will form them, from a manager of one page
        has_state = any(layer.mixer.state_spec() is not None for layer in model.layers)
        sizing = CacheManager(model.cache_slots, 1, cfg.block_size, cfg.max_running, has_state)
        groups = {slot: sizing.group_of(slot) for slot in model.cache_slots}
        model.prepare(cfg.max_model_len, device)
        caches = sizing_caches(model, groups, cfg.block_size, cfg.torch_dtype, device)
        states = {i: torch.empty((0, *layer.mixer.state_spec().shape),
                                 dtype=layer.mixer.state_spec().dtype, device=device)
                  for i, layer in enumerate(model.layers) if layer.mixer.state_spec() is not None}
        program = model.compile(caches, states)
        needs = ModelRunner.step_needs(program, max(1, sizing.num_groups), cfg.block_size,
                                       cfg.max_model_len, min(cfg.prefill_budget, cfg.max_model_len),
                                       cfg.max_running, graph_batch if cfg.use_graphs else 0)
        graphs = cfg.max_graphs * GRAPH_RECORD_BYTES if cfg.use_graphs else 0
        # buffers grow by a quarter beyond what a step asks for
        return int(1.25 * (needs["eager_workspace"] + needs["eager_ints"])
                   + needs["graph_workspace"] + needs["graph_ints"] + graphs)

    # ---------------------------------------------------------------- lifecycle

    def start(self) -> None:
        """Hand the loop to a thread of the engine's own, until `shutdown`."""
        if self._worker is not None:
            return
        self._serving.set()
        self._worker_error = None
        self._worker = threading.Thread(target=self._serve, name="mercury-amd-loop", daemon=True)
        self._worker.start()

    def shutdown(self, timeout: float = 5.0) -> None:
        """Stop the engine's thread after the pass it is in.  Raises what the thread died of,
        if it died, and TimeoutError when it does not come back in `timeout` seconds."""
        worker, self._worker = self._worker, None
        self._serving.clear()
        if worker is None:
            return
        self._inbox.post("wake", None)
        worker.join(timeout)
        if worker.is_alive():
            self._worker = worker
            raise TimeoutError(f"the engine's thread did not stop within {timeout} s")
        if self._worker_error is not None:
            raise self._worker_error

    def _serve(self) -> None:
        try:
            while self._serving.is_set():
                if self.step() is None:
                    self._inbox.wait(self.cfg.idle_sleep_s)
        except BaseException as error:      # kept for shutdown() to raise on the caller's thread
            self._worker_error = error
            self._serving.clear()

    # ---------------------------------------------------------------- client side

    def submit(self, rid: str, prompt_ids: list, max_tokens: int, sink: Sink,
               params: SamplingParams | None = None, session_id: str | None = None,
               arrival: float | None = None) -> None:
        """Queue a request; its events go to `sink`, called on the loop's thread.  A request
        that can never run (an empty prompt, more tokens than one request may hold) gets an
        "error" event here and now, and is not queued."""
        now = self.clock()
        refusal = self.core.refusal(len(prompt_ids), max_tokens)
        if refusal is not None:
            self.core.count_rejected()
            sink(StreamEvent(rid=rid, kind="error", message=refusal, t=now))
            return
        request = self.core.make_request(rid, prompt_ids, max_tokens,
                                         now if arrival is None else arrival, params, session_id)
        with self._listeners_guard:
            self._listeners[rid] = sink
            self._accepted += 1
        self._inbox.post("add", request)

    def abort(self, rid: str) -> None:
        """Ask the loop to end request `rid`; its sink receives the closing event."""
        self._inbox.post("abort", rid)

    def run_until_idle(self) -> int:
        """On the caller's thread: passes until nothing is queued or running.  Returns how many
        passes ran a step."""
        if self._worker is not None:
            raise RuntimeError("the engine's own thread runs the loop; shutdown() first")
        ran = 0
        self._take_commands()
        while self.sched.has_work():
            if self.step() is not None:
                ran += 1
        return ran

    def generate(self, prompts: list, params=None, max_tokens: int = 16) -> list:
        """Blocking: run every prompt (a list of token ids each) to completion and return the
        generated token ids, one list per prompt.  `params` is one SamplingParams for all or a
        list with one per prompt; `max_tokens` likewise an int or a list."""
        if self._worker is not None:
            raise RuntimeError("generate() drives the loop itself; do not call it after start()")
        n = len(prompts)
        params = params if isinstance(params, list) else [params] * n
        budgets = max_tokens if isinstance(max_tokens, list) else [max_tokens] * n
        outputs, errors = [[] for _ in range(n)], {}
        first = self._accepted

        def sink_for(i):
            def sink(event):
                if event.kind == "token":
                    outputs[i].append(event.token)
                elif event.kind == "error":
                    errors[i] = event.message
            return sink

        for i, prompt in enumerate(prompts):
            self.submit(f"gen-{first + i}", prompt, budgets[i], sink_for(i), params=params[i])
        if errors:
            raise ValueError("; ".join(f"prompt {i}: {m}" for i, m in sorted(errors.items())))
        self.run_until_idle()
        return outputs

    # ---------------------------------------------------------------- the loop

    def step(self):
        """One pass: take commands, plan, run the plan, apply its results.  Returns the step's
        record, or None when there was nothing to run."""
        started = time.perf_counter()
        self._take_commands()
        plan, events = self.core.schedule(self.clock())
        self._deliver(events)
        if not plan:
            self.core.count_idle()
            return None
        result = self.executor.execute(plan)
        now = self.clock()
        self._deliver(self.core.advance(plan, result.tokens, now))
        if self.cfg.debug_invariants:
            self.manager.check_invariants()
        return self.core.log_step(plan, now, result.prepare_seconds, result.forward_seconds,
                                  getattr(result, "device_seconds", 0.0),
                                  time.perf_counter() - started)

    def _take_commands(self) -> None:
        for kind, payload in self._inbox.take_all():
            if kind == "add":
                self.core.add(payload)
            elif kind == "abort":
                events = self.core.abort(payload, self.clock())
                if not events:
                    # finished already, or never queued: nobody to tell
                    with self._listeners_guard:
                        self._listeners.pop(payload, None)
                self._deliver(events)

    def _deliver(self, events: list) -> None:
        for event in events:
            with self._listeners_guard:
                if event.kind == "done":
                    sink = self._listeners.pop(event.rid, None)
                else:
                    sink = self._listeners.get(event.rid)
            if sink is None:
                continue
            try:
                sink(event)
            except Exception:
                # a sink that raises has stopped listening: end its request
                self.abort(event.rid)

    # ---------------------------------------------------------------- reporting

    def snapshot(self) -> dict:
        c = self.cfg
        return {
            "config": {
                "policy": c.policy, "block_size": c.block_size, "num_blocks": c.num_blocks,
                "kv_capacity_tokens": self.manager.capacity_tokens(), "max_running": c.max_running,
                "prefill_budget": c.prefill_budget, "aging_tokens_per_s": c.aging_tokens_per_s,
                "max_wait_s": c.max_wait_s, "scan_limit": c.scan_limit, "model": c.model,
                "dtype": c.dtype,
            },
            "allocator": self.manager.snapshot(),
            "scheduler": self.sched.snapshot(),
            "engine": self.core.summary(),
            "submitted": self._accepted,
            "executor": self.executor.snapshot() if hasattr(self.executor, "snapshot") else {},
        }

    def leaked_blocks(self) -> int:
        """Pages held although no request is live (0 when the bookkeeping is whole)."""
        return self.manager.leaked_pages()

    def drain_request_records(self) -> list:
        """The records of requests finished since the last call."""
        return self.core.drain_finished()

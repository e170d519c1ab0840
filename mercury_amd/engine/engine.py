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

import queue
import threading
import time
from typing import Callable

from ..cache import CacheManager, PageHasher
from ..config.engine_config import EngineConfig
from ..hostcore import core as _core

StreamEvent = _core.StreamEvent
SamplingParams = _core.SamplingParams
Sink = Callable[[StreamEvent], None]


def autosize_blocks(cfg: EngineConfig, kv_bytes_per_token: int, device) -> int:
    """Pages that fit in the memory that is free once the weights are resident
    (reference: mercury/config.py:164-185)."""
    import torch

    free, _total = torch.cuda.mem_get_info(torch.device(device))
    budget = int(free * cfg.gpu_memory_fraction)
    per_page = max(1, kv_bytes_per_token * cfg.block_size)
    pages = budget // per_page
    if pages < 1:
        raise RuntimeError(f"only {free / 2**30:.1f} GiB are free; there is no room for a cache")
    return pages


class Engine:
    """`Engine(cfg)` loads the model folder `cfg.model` onto the GPU, or, with
    `cfg.random_weights`, builds the model that `model_config` (a ``config.json`` as a dict) or
    the ``config.json`` at `cfg.model` describes and draws its weights from `cfg.weight_seed`.
    Tests pass `executor` (anything with `execute(plan)`) and, with it, the cache manager it
    checks against."""

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
        self._commands: queue.Queue = queue.Queue()
        self._sinks: dict = {}
        self._wake, self._stop = threading.Event(), threading.Event()
        self._thread = None
        self._lock = threading.Lock()
        self._submitted = 0

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
        if cfg.num_blocks < 0:
            cfg.num_blocks = autosize_blocks(cfg, model.kv_bytes_per_token(cfg.torch_dtype), device)
            cfg.validate_against(model.max_positions or cfg.max_model_len)
        manager = CacheManager(model.cache_slots, cfg.num_blocks, cfg.block_size, cfg.max_running,
                               has_state)
        runner = ModelRunner(model, manager, cfg.torch_dtype, device, cfg.max_model_len,
                             use_graphs=cfg.use_graphs)
        return (GpuExecutor(runner, Sampler(cfg.seed), lookahead=cfg.lookahead), manager,
                model.eos_token_ids)

    # ---------------------------------------------------------------- lifecycle

    def start(self) -> None:
        """Run the loop on a thread of its own until `shutdown`."""
        if self._thread is not None:
            return
        self._thread = threading.Thread(target=self._run, name="mercury-amd-engine", daemon=True)
        self._thread.start()

    def shutdown(self, timeout: float = 5.0) -> None:
        self._stop.set()
        self._wake.set()
        if self._thread is not None:
            self._thread.join(timeout)
            self._thread = None

    def _run(self) -> None:
        while not self._stop.is_set():
            if self.step() is None:
                self._wake.wait(self.cfg.idle_sleep_s)
                self._wake.clear()

    # ---------------------------------------------------------------- client side

    def submit(self, rid: str, prompt_ids: list, max_tokens: int, sink: Sink,
               params: SamplingParams | None = None, session_id: str | None = None,
               arrival: float | None = None) -> None:
        """Queue a request.  A request that can never run (an empty prompt, more tokens than
        one request may hold) is answered at once with an "error" event and not queued."""
        arrival = self.clock() if arrival is None else arrival
        why = self.core.refusal(len(prompt_ids), max_tokens)
        if why is not None:
            self.core.count_rejected()
            sink(StreamEvent(rid=rid, kind="error", message=why, t=self.clock()))
            return
        request = self.core.make_request(rid, prompt_ids, max_tokens, arrival, params, session_id)
        with self._lock:
            self._sinks[rid] = sink
            self._submitted += 1
        self._commands.put(("add", request))
        self._wake.set()

    def abort(self, rid: str) -> None:
        self._commands.put(("abort", rid))
        self._wake.set()

    def generate(self, prompts: list, params=None, max_tokens: int = 16) -> list:
        """Blocking: run every prompt (a list of token ids each) to completion and return the
        generated token ids, one list per prompt.  `params` is one SamplingParams for all or a
        list with one per prompt; `max_tokens` likewise an int or a list."""
        if self._thread is not None:
            raise RuntimeError("generate() drives the loop itself; do not call it after start()")
        n = len(prompts)
        params = params if isinstance(params, list) else [params] * n
        budgets = max_tokens if isinstance(max_tokens, list) else [max_tokens] * n
        outputs, errors = [[] for _ in range(n)], {}
        base = self._submitted

        def sink_for(i):
            def sink(event):
                if event.kind == "token":
                    outputs[i].append(event.token)
                elif event.kind == "error":
                    errors[i] = event.message
            return sink

        for i, prompt in enumerate(prompts):
            self.submit(f"gen-{base + i}", prompt, budgets[i], sink_for(i),
                        params=params[i])
        if errors:
            raise ValueError("; ".join(f"prompt {i}: {m}" for i, m in sorted(errors.items())))
        self._drain_commands()
        while self.sched.has_work():
            self.step()
        return outputs

    # ---------------------------------------------------------------- the loop

    def step(self):
        """One pass: take commands, plan, run the plan, apply its results.  Returns the step's
        record, or None when there was nothing to run."""
        started = time.perf_counter()
        self._drain_commands()
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

    def _drain_commands(self) -> None:
        while True:
            try:
                kind, payload = self._commands.get_nowait()
            except queue.Empty:
                return
            if kind == "add":
                self.core.add(payload)
                continue
            events = self.core.abort(payload, self.clock())
            if not events:
                with self._lock:
                    self._sinks.pop(payload, None)    # already finished, or never queued
            self._deliver(events)

    def _deliver(self, events: list) -> None:
        for event in events:
            closing = event.kind == "done"
            with self._lock:
                sink = self._sinks.pop(event.rid, None) if closing else self._sinks.get(event.rid)
            if sink is None:
                continue
            try:
                sink(event)
            except Exception:
                self.abort(event.rid)   # a sink that raises means nobody is listening any more

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
            "submitted": self._submitted,
        }

    def leaked_blocks(self) -> int:
        return self.manager.leaked_pages()

    def drain_request_records(self) -> list:
        return self.core.drain_finished()

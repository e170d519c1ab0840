"""The engine loop: take commands, schedule, execute, route tokens, finish and free
(reference: mercury/engine.py:28-300).

One thread owns everything that touches the cache.  Clients talk to it through `submit` and
`abort` (a queue) and hear back through a per-request `sink` callable that receives
:class:`StreamEvent` objects; `generate` wraps that into a blocking call that returns token
lists.
"""

from __future__ import annotations

import queue
import threading
import time
from dataclasses import dataclass
from typing import Callable

from ..cache.hashing import PageHasher
from ..cache.manager import CacheManager
from ..config.engine_config import EngineConfig
from .metrics import EngineMetrics, StepRecord
from .request import Request, RequestState, SamplingParams
from .scheduler import Scheduler


@dataclass(slots=True)
class StreamEvent:
    """kind: "token" (token, index), "done" (finish_reason: "length" | "stop" | "abort"),
    "preempted", or "error" (message)."""

    rid: str
    kind: str
    token: int | None = None
    index: int = 0
    finish_reason: str | None = None
    message: str | None = None
    t: float = 0.0


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
    """`Engine(cfg)` loads the model folder `cfg.model` onto the GPU.  Tests pass `executor`
    (anything with `execute(plan)`) and, with it, the cache manager it checks against."""

    def __init__(self, cfg: EngineConfig, executor=None, manager: CacheManager | None = None,
                 clock: Callable[[], float] = time.perf_counter, eos_token_ids=None):
        self.cfg = cfg
        self.clock = clock
        self.hasher = PageHasher(cfg.block_size, cfg.cryptographic_hashes)
        if executor is None:
            executor, manager, eos = self._load(cfg)
            eos_token_ids = eos if eos_token_ids is None else eos_token_ids
        elif manager is None:
            raise ValueError("an engine with its own executor needs the cache manager it uses")
        self.executor, self.manager = executor, manager
        self.runner = executor  # the reference's name for this seam
        self.eos_ids = set(eos_token_ids or ())
        self.sched = Scheduler(
            manager, self.hasher, policy=cfg.policy, max_running=cfg.max_running,
            prefill_budget=cfg.prefill_budget, aging_tokens_per_s=cfg.aging_tokens_per_s,
            max_wait_s=cfg.max_wait_s, scan_limit=cfg.scan_limit)
        self.metrics = EngineMetrics(max_steps=cfg.max_step_records)
        self._commands: queue.Queue = queue.Queue()
        self._sinks: dict = {}
        self._wake, self._stop = threading.Event(), threading.Event()
        self._thread = None
        self._lock = threading.Lock()
        self._submitted = 0

    @staticmethod
    def _load(cfg: EngineConfig):
        from ..sampling.sampler import Sampler
        from ..weights.loader import load_model_folder
        from .executor import GpuExecutor
        from .runner import ModelRunner, require_gpu

        import torch

        device = torch.device(cfg.device)
        require_gpu(device)
        model = load_model_folder(cfg.model, cfg.torch_dtype, device)
        if model.max_positions:
            cfg.validate_against(model.max_positions)
        has_state = any(layer.mixer.state_spec() is not None for layer in model.layers)
        if cfg.num_blocks < 0:
            elem = torch.empty((), dtype=cfg.torch_dtype).element_size()
            per_token = sum(2 * s.kv_heads * s.head_dim * elem for s in model.cache_slots.values())
            cfg.num_blocks = autosize_blocks(cfg, per_token, device)
            cfg.validate_against(model.max_positions or cfg.max_model_len)
        manager = CacheManager(model.cache_slots, cfg.num_blocks, cfg.block_size, cfg.max_running,
                               has_state)
        runner = ModelRunner(model, manager, cfg.torch_dtype, device, cfg.max_model_len,
                             use_graphs=cfg.use_graphs)
        return (GpuExecutor(runner, Sampler(cfg.seed), lookahead=cfg.lookahead), manager,
                model.eos_token_ids)

    # ---------------------------------------------------------------- lifecycle

    def start(self) -> None:
        if self._thread is not None:
            return
        self.metrics.started_at = self.clock()
        self._thread = threading.Thread(target=self._run, name="mercury-engine", daemon=True)
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
        params = params or SamplingParams()
        arrival = self.clock() if arrival is None else arrival
        ceiling = min(self.cfg.max_model_len, self.manager.capacity_tokens())
        if not prompt_ids:
            self._reject(rid, sink, "prompt must contain at least one token")
            return
        if len(prompt_ids) + max_tokens > ceiling:
            self._reject(rid, sink,
                         f"prompt ({len(prompt_ids)}) + max_tokens ({max_tokens}) exceeds the "
                         f"{ceiling}-token ceiling of this engine")
            return
        r = Request(rid=rid, prompt=list(prompt_ids), max_tokens=max_tokens, arrival=arrival,
                    hashes=self.hasher.hashes(prompt_ids), params=params, session_id=session_id)
        with self._lock:
            self._sinks[rid] = sink
            self._submitted += 1
        self._commands.put(("add", r))
        self._wake.set()

    def abort(self, rid: str) -> None:
        self._commands.put(("abort", rid))
        self._wake.set()

    def _reject(self, rid: str, sink: Sink, message: str) -> None:
        self.metrics.counters["rejected_requests"] += 1
        sink(StreamEvent(rid=rid, kind="error", message=message, t=self.clock()))

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
            self.submit(f"gen-{base + i}", prompt, budgets[i], sink_for(i), params=params[i])
        if errors:
            raise ValueError("; ".join(f"prompt {i}: {m}" for i, m in sorted(errors.items())))
        self._drain_commands()
        while self.sched.has_work():
            self.step()
        return outputs

    # ---------------------------------------------------------------- the loop

    def step(self):
        t_start = time.perf_counter()
        self._drain_commands()
        plan = self.sched.schedule(self.clock())
        for r in plan.preempted:
            self._emit(r, StreamEvent(rid=r.rid, kind="preempted", t=self.clock()))
        if not plan:
            self.metrics.counters["idle_steps"] += 1
            return None

        result = self.executor.execute(plan)
        now = self.clock()
        for work, token in zip(plan.work, result.tokens):
            self._advance(work, token, now)

        if self.cfg.debug_invariants:
            self.manager.check_invariants()

        record = StepRecord(
            t=now, num_prefill=len(plan.prefill), num_decode=len(plan.decode),
            prefill_tokens=plan.num_prefill_tokens, sched_s=plan.sched_seconds,
            prepare_s=result.prepare_seconds, forward_s=result.forward_seconds,
            step_s=time.perf_counter() - t_start, waiting=len(self.sched.waiting),
            running=len(self.sched.running), free_blocks=self.manager.num_available(),
            preempted=len(plan.preempted))
        self.metrics.add_step(record)
        return record

    def _drain_commands(self) -> None:
        while True:
            try:
                kind, payload = self._commands.get_nowait()
            except queue.Empty:
                return
            if kind == "add":
                self.sched.add(payload)
                continue
            r = self.sched.abort(payload)
            if r is None:
                with self._lock:
                    self._sinks.pop(payload, None)
                continue
            self.metrics.counters["aborted_requests"] += 1
            r.finished_at = self.clock()
            self.metrics.add_finished(r.record())
            self._emit(r, StreamEvent(rid=r.rid, kind="done", finish_reason="abort",
                                      t=r.finished_at), close=True)

    def _advance(self, work, token, now: float) -> None:
        """The step wrote keys and values for the work's tokens: note it, offer the pages that
        became full to the prefix cache, give back what a window passed, and, when the work
        completed the sequence, take the sampled token."""
        r = work.request
        r.num_computed = work.start + work.count
        full = r.num_computed // self.cfg.block_size
        if self.manager.prefix_sharing and full > len(r.hashes):
            self.hasher.extend(r.hashes, r.tokens[:r.num_computed])
        self.manager.commit(r.rid, r.hashes, full)
        self.manager.trim(r.rid, r.num_computed)
        if token is None:
            return
        index = len(r.out)
        r.append(int(token))
        if r.first_token_at is None:
            r.first_token_at = now
        self._emit(r, StreamEvent(rid=r.rid, kind="token", token=int(token), index=index, t=now))
        if len(r.out) >= r.max_tokens:
            self._finish(r, "length", now)
        elif not r.params.ignore_eos and int(token) in self.eos_ids:
            self._finish(r, "stop", now)

    def _finish(self, r: Request, reason: str, now: float) -> None:
        r.state = RequestState.FINISHED
        r.finish_reason = reason
        r.finished_at = now
        self.sched.drop(r)
        self.metrics.counters["finished_requests"] += 1
        self.metrics.add_finished(r.record())
        self._emit(r, StreamEvent(rid=r.rid, kind="done", finish_reason=reason, t=now), close=True)

    def _emit(self, r: Request, event: StreamEvent, close: bool = False) -> None:
        with self._lock:
            sink = self._sinks.pop(r.rid, None) if close else self._sinks.get(r.rid)
        if sink is None:
            return
        try:
            sink(event)
        except Exception:
            self.abort(r.rid)  # a sink that raises means nobody is listening any more

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
            "engine": self.metrics.summary(),
            "submitted": self._submitted,
        }

    def leaked_blocks(self) -> int:
        return self.manager.leaked_pages()

    def drain_request_records(self) -> list:
        return self.metrics.drain_finished()

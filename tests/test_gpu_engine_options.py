"""Engine options that only a GPU run exercises: the automatic pool size, the loop on a thread
of the engine's own with requests from another thread, and the bound on what captured decode
graphs hold (reference: mercury/config.py:164-185, mercury/engine.py:81-100)."""

from __future__ import annotations

import threading

import pytest
import torch

from tests import helpers
from tests.test_gpu_replay import sized_folder

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def free_bytes() -> int:
    torch.cuda.synchronize(DEV)
    torch.cuda.empty_cache()
    return torch.cuda.mem_get_info(DEV)[0]


def test_automatic_pool_size_leaves_room_for_what_comes_after_it():
    """num_blocks = -1: the pool is sized to a fraction of the free memory after setting aside
    what the steps and the captured graphs will need; the engine then generates, leaks nothing,
    and what it allocated after the cache stays within what was set aside."""
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = sized_folder("S64")
    before = free_bytes()
    cfg = EngineConfig(model=str(folder), dtype="bfloat16", num_blocks=-1, gpu_memory_fraction=0.02,
                       max_running=16, prefill_budget=512, max_model_len=1024)
    engine = Engine(cfg)
    reserved = cfg.extra["reserved_bytes"]
    memory = engine.snapshot()["executor"]["memory"]
    assert cfg.num_blocks > 1024 // 16 and reserved > 0
    assert engine.snapshot()["config"]["num_blocks"] == cfg.num_blocks
    # the pool is the stated fraction of what was free beyond the reservation (the weights
    # were resident when it was measured)
    per_page = engine.executor.runner.kv_bytes_per_token() * cfg.block_size
    assert memory["kv_bytes"] == cfg.num_blocks * per_page
    assert memory["kv_bytes"] <= 0.02 * before
    assert memory["kv_bytes"] >= 0.02 * (before - reserved) - 2 * 10**9 * 0.02 - per_page
    # the largest steps the scheduler can plan under these options: portions of 512 beside
    # decoded tokens, then sixteen requests decoding through captured graphs
    prompts = [helpers.random_tokens(5003, 700 + 11 * i, seed=i) for i in range(16)]
    out = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=40)
    assert [len(o) for o in out] == [40] * 16 and engine.leaked_blocks() == 0
    memory = engine.snapshot()["executor"]["memory"]
    assert memory["graphs"] >= 1 and memory["graph_buffer_bytes"] > 0
    later = memory["step_buffer_bytes"] + memory["graph_buffer_bytes"] + memory["graphs"] * (2 << 20)
    assert later <= reserved, (memory, reserved)
    # and on the card: everything the engine holds beside its weights is pool + reservation
    weights = sum(t.numel() * t.element_size() for t in
                  {id(t): t for t in _tensors(engine.executor.runner.model)}.values())
    used = before - free_bytes()
    assert used <= weights + memory["kv_bytes"] + reserved + (256 << 20), (used, weights, memory, reserved)


def _tensors(model):
    seen = []

    def walk(obj, depth=0):
        if isinstance(obj, torch.Tensor):
            seen.append(obj)
        elif isinstance(obj, (list, tuple)):
            for item in obj:
                walk(item, depth + 1)
        elif isinstance(obj, dict):
            for item in obj.values():
                walk(item, depth + 1)
        elif hasattr(obj, "__dict__") and depth < 6 and type(obj).__module__.startswith("mercury_amd"):
            for item in vars(obj).values():
                walk(item, depth + 1)

    walk(model)
    return seen


def test_autosize_refuses_a_card_without_room():
    from mercury_amd.config import EngineConfig
    from mercury_amd.engine.engine import autosize_blocks

    cfg = EngineConfig(model="x", gpu_memory_fraction=0.5)
    free = torch.cuda.mem_get_info(DEV)[0]
    with pytest.raises(RuntimeError, match="no room for a cache"):
        autosize_blocks(cfg, 256, DEV, reserve_bytes=free)
    assert autosize_blocks(cfg, 256, DEV, reserve_bytes=free // 2) > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_loop_on_its_own_thread_with_requests_from_another(dtype):
    """start() / submit from a second thread / shutdown(): the tokens are those of generate()
    on the caller's thread, captured graphs and lookahead included."""
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = helpers.model_folder("A")
    prompts = [helpers.random_tokens(512, n, seed=n) for n in (5, 17, 33, 64, 9, 40)]
    params = SamplingParams(ignore_eos=True)

    def make():
        return Engine(EngineConfig(model=str(folder), dtype=dtype, num_blocks=64, max_model_len=256,
                                   max_running=4, prefill_budget=48))

    want = make().generate(prompts, params, max_tokens=24)

    engine = make()
    got = {i: [] for i in range(len(prompts))}
    finished = {i: threading.Event() for i in range(len(prompts))}

    def sink_for(i):
        def sink(event):
            if event.kind == "token":
                got[i].append(event.token)
            elif event.kind == "done":
                finished[i].set()
        return sink

    def client():
        for i, prompt in enumerate(prompts):
            engine.submit(f"req-{i}", prompt, 24, sink_for(i), params=params)

    engine.start()
    with pytest.raises(RuntimeError, match="own thread"):
        engine.run_until_idle()
    sender = threading.Thread(target=client)
    sender.start()
    sender.join(30)
    assert all(flag.wait(60) for flag in finished.values()), "requests did not finish"
    engine.shutdown()
    assert [got[i] for i in range(len(prompts))] == want
    assert engine.leaked_blocks() == 0
    assert engine.executor.runner.graphs, "decoding did not go through captured graphs"
    # the thread is gone and the caller may drive the loop again
    assert engine.generate([prompts[0]], params, max_tokens=24)[0] == want[0]


def test_a_failure_on_the_engine_thread_reaches_shutdown():
    from mercury_amd import Engine, EngineConfig

    folder = helpers.model_folder("A")
    engine = Engine(EngineConfig(model=str(folder), dtype="float32", num_blocks=64, max_model_len=256))

    class Broken:
        def execute(self, plan):
            raise RuntimeError("executor made to fail")

    engine.executor = Broken()
    engine.start()
    engine.submit("r", [1, 2, 3], 4, lambda event: None)
    engine._worker.join(30)
    with pytest.raises(RuntimeError, match="made to fail"):
        engine.shutdown()


def test_captured_graphs_share_their_buffers_and_are_bounded():
    """Decoding through every number of sequences from 1 to 64 at two length bounds captures
    128 graphs.  They share one index buffer and one workspace, at most `max_graphs` are kept,
    and the card's memory after the sweep stays within a stated bound of what it was when the
    first graph existed."""
    from mercury_amd.engine.replay import ReplaySession

    folder = sized_folder("S64")
    tokens = helpers.random_tokens(5003, 420, 1)
    per_graph = 2 << 20          # what the engine sets aside per graph (GRAPH_RECORD_BYTES)

    def sweep(max_graphs):
        s = ReplaySession(folder, "bfloat16", 64 * 448, page_size=16, max_live=64)
        runner = s.runner
        runner.max_graphs = max_graphs
        done = [100] * 64
        for i in range(64):
            s.step([{"id": f"r{i}", "tokens": tokens[:100], "want": []}], [])

        def decode(batch):
            out = s.step([{"id": f"r{i}", "tokens": tokens[done[i]:done[i] + 1], "want": [0]}
                          for i in range(batch)], [])
            for i in range(batch):
                done[i] += 1
            return out

        decode(1)
        start = free_bytes()
        buffers = runner.graph_buffers
        address = (buffers.ints.data_ptr(), buffers.workspace.data_ptr())
        for batch in range(1, 65):              # every length below 256: one bound
            decode(batch)
        assert max(done) < 256
        while min(done) <= 256:                 # all of them past 256: the next bound
            decode(64)
        for batch in range(1, 65):
            decode(batch)
        assert max(done) < 512
        report = runner.memory_report()
        assert {bound for _n, bound in runner.graphs} <= {256, 512}
        assert report["captured"] >= 127 and report["resets"] == 0
        assert report["graphs"] <= max_graphs
        assert report["dropped"] == report["captured"] - report["graphs"]
        assert (buffers.ints.data_ptr(), buffers.workspace.data_ptr()) == address
        return start - free_bytes(), report

    grown, report = sweep(96)
    assert grown <= 96 * per_graph, (grown, report)
    grown_small, report_small = sweep(8)
    assert report_small["graphs"] == 8
    assert grown_small <= 8 * per_graph + (8 << 20), (grown_small, report_small)

"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

A "step" is one decode step of the whole engine (schedule, run the batch through the model from
the cache, sample), at the layer sizes of Qwen2.5-0.5B with random weights, synthetic uniform
random token ids, a batch of 8 and a context that reaches 4,096 tokens at the last timed step.
One JSON line is printed: `value` is decoded tokens per second; `prefill` times one 2,048-token
prompt as one step; `roofline` divides the bytes a decode step has to read (every weight it
uses once, and the cache of the live requests) by its time and by the HBM peak; `points`
holds decode throughput at batch 1 and 64 and, at the default batch, at half the context, and
the tokens a second of one 8,192-token prompt as one step.
Beside the published peaks both fractions are also given against what this machine reaches in
the same run: a streaming read of a 2 GiB matrix by the engine's one-row projection, and a
8192 x 8192 x 8192 bfloat16 product by its tiled matrix-core kernel (`measured`).

    python bench.py --attention

times the prompt attention kernel alone at the models' head shapes, and

    python bench.py --shape 32b --serve

runs a whole workload through the scheduler instead (64 requests with prompts of 2,048 tokens,
admitted in portions of 512 beside the decoding of the others, each decoded to 4,096) and
prints the generated tokens per second of the whole run.
"""

from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

# Qwen2.5-0.5B layer sizes (the model this benchmark names).
QWEN25_05B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 896, "intermediate_size": 4864, "num_hidden_layers": 24,
    "num_attention_heads": 14, "num_key_value_heads": 2, "head_dim": 64,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 32768,
}
# The larger models of the family, for `--shape`.
QWEN25_7B = dict(QWEN25_05B, hidden_size=3584, intermediate_size=18944, num_hidden_layers=28,
                 num_attention_heads=28, num_key_value_heads=4, head_dim=128, vocab_size=152064,
                 tie_word_embeddings=False)
QWEN25_32B = dict(QWEN25_05B, hidden_size=5120, intermediate_size=27648, num_hidden_layers=64,
                  num_attention_heads=40, num_key_value_heads=8, head_dim=128, vocab_size=152064,
                  tie_word_embeddings=False)
SHAPES = {"0.5b": ("Qwen2.5-0.5B", QWEN25_05B), "7b": ("Qwen2.5-7B", QWEN25_7B),
          "32b": ("Qwen2.5-32B", QWEN25_32B)}
CONTEXT = 4096
PREFILL_TOKENS = 2048
LONG_PREFILL_TOKENS = 8192   # a second prompt length, in `points`
BLOCK_SIZE = 16
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--shape", default="0.5b", choices=sorted(SHAPES),
                   help="layer sizes of which model of the family")
    p.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    p.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    p.add_argument("--context", type=int, default=CONTEXT)
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 runs")
    p.add_argument("--no-lookahead", action="store_true",
                   help="never start a decode step before the previous one's tokens are read")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--serve", action="store_true",
                   help="instead of the decode steps: --serve-requests requests with prompts of "
                        "half the context through the scheduler, prompts in portions of "
                        "--serve-chunk tokens beside the others' decoding, each decoded to the "
                        "context; one line with the generated tokens a second")
    p.add_argument("--attention", action="store_true",
                   help="instead of the engine's steps: the prompt attention kernel alone at the "
                        "head shapes of the three models, a table of times and PFLOP/s")
    p.add_argument("--serve-requests", type=int, default=64)
    p.add_argument("--serve-chunk", type=int, default=512)
    return p.parse_args(argv)


def prefill_flops(cfg: dict, tokens: int) -> float:
    """Multiply-adds times two of one whole-prompt step: the projections of every layer for
    every token, causal attention (scores and weighted sum), and the head for one row."""
    h, i = cfg["hidden_size"], cfg["intermediate_size"]
    n_q, n_kv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    linear = 2.0 * (h * (n_q + 2 * n_kv) * d + n_q * d * h + 3 * h * i)
    attention = 4.0 * n_q * d * tokens * (tokens + 1) / 2
    layers = cfg["num_hidden_layers"]
    return layers * (linear * tokens + attention) + 2.0 * h * cfg["vocab_size"]


class Bench:
    def __init__(self, cfg: dict, dtype: str, max_batch: int, context: int, seed: int,
                 lookahead: bool = True, prefill_budget: int = 8192):
        import torch

        from mercury_amd import Engine, EngineConfig

        self.torch = torch
        self.cfg = cfg
        t0 = time.time()
        pages = max_batch * (-(-(context + 128) // BLOCK_SIZE) + 1) + LONG_PREFILL_TOKENS // BLOCK_SIZE + 8
        self.engine_cfg = EngineConfig(
            model="random", random_weights=True, weight_seed=seed, weight_std=0.02,
            device="cuda:0", dtype=dtype, block_size=BLOCK_SIZE, num_blocks=pages,
            max_running=max_batch + 1, prefill_budget=prefill_budget,
            max_model_len=min(max(context, LONG_PREFILL_TOKENS) + 128,
                              cfg.get("max_position_embeddings", 1 << 30)), seed=seed,
            lookahead=lookahead)
        self.engine = Engine(self.engine_cfg, model_config=cfg, eos_token_ids=())
        self.runner, self.manager = self.engine.executor.runner, self.engine.manager
        self.model = model = self.runner.model
        self.rng = torch.Generator().manual_seed(seed)
        self.counter = 0
        print(f"[bench] model ready in {time.time() - t0:.1f} s: "
              f"{model.decode_weight_bytes() / 1e9:.3f} GB of weights a step reads, "
              f"{pages} pages", file=sys.stderr, flush=True)

    def tokens(self, count: int) -> list:
        return self.torch.randint(0, self.cfg["vocab_size"], (count,), generator=self.rng).tolist()

    def sync(self):
        self.torch.cuda.synchronize()

    def decode(self, batch: int, context: int, steps: int, warmup: int) -> dict:
        """Time `steps` decode steps of `batch` requests whose context reaches `context` at
        the last timed step."""
        from mercury_amd import SamplingParams

        # Prompts enter a few per step (the token budget), so the first admitted request is
        # some tokens ahead of the last; the untimed steps are counted so that the longest
        # request reaches `context` exactly at the last timed step.
        stagger = -(-batch * context // self.engine_cfg.prefill_budget) + 1
        prompt_len = context - steps - warmup - stagger
        rids = []
        for _ in range(batch):
            rid = f"bench-{self.counter}"
            self.counter += 1
            self.engine.submit(rid, self.tokens(prompt_len), steps + warmup + stagger + batch + 8,
                               lambda e: None, params=SamplingParams(ignore_eos=True))
            rids.append(rid)
        self.engine._take_commands()
        t0 = time.time()
        while any(r.remaining > 1 for r in self.engine.sched.running) or self.engine.sched.waiting:
            self.engine.step()          # prompts, in portions under the token budget
        self.sync()
        fill_s = time.time() - t0
        assert len(self.engine.sched.running) == batch
        longest = max(r.num_computed for r in self.engine.sched.running)
        untimed = context - steps - longest
        assert untimed >= warmup, (untimed, warmup)
        for _ in range(untimed):
            self.engine.step()
        self.sync()
        # The device's own clock over the same steps: one pair of events around all of them
        # (a pair per step costs tens of microseconds a step, which a short step feels).
        began, ended = (self.torch.cuda.Event(enable_timing=True) for _ in range(2))
        start = time.perf_counter()
        began.record()
        for _ in range(steps):
            record = self.engine.step()
            assert record.num_decode == batch and record.num_prefill == 0
        ended.record()
        self.sync()
        elapsed = time.perf_counter() - start
        assert max(r.num_computed for r in self.engine.sched.running) == context
        kv_tokens = sum(r.num_computed for r in self.engine.sched.running)
        kv_bytes = kv_tokens * self.runner.kv_bytes_per_token()
        for rid in rids:
            self.engine.abort(rid)
        self.engine._take_commands()
        assert self.engine.leaked_blocks() == 0
        ms = 1e3 * elapsed / steps
        device_ms = began.elapsed_time(ended) / steps
        return {"tok_s": batch * steps / elapsed, "ms": ms, "fill_s": fill_s, "device_ms": device_ms,
                "prompt_len": prompt_len, "bytes": self.model.decode_weight_bytes() + kv_bytes}

    def measured_peaks(self) -> dict:
        """What this machine reaches, by the engine's own kernels: GB/s of a streaming read
        (a 2 GiB matrix times one row, the projection every decode step is made of) and
        FLOP/s of a large bfloat16 product (8192 x 8192 x 8192 through the tiled matrix-core
        kernel)."""
        torch = self.torch
        from mercury_amd.kernels import ops

        def best(fn, repeats=5):
            fn()
            times = []
            for _ in range(repeats):
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                fn()
                stop.record()
                stop.synchronize()
                times.append(1e-3 * start.elapsed_time(stop))
            return min(times)

        dtype = torch.bfloat16 if self.engine_cfg.dtype == "bfloat16" else torch.float32
        rows = (1 << 31) // (4096 * torch.empty((), dtype=dtype).element_size())
        big = torch.empty((rows, 4096), dtype=dtype, device="cuda:0").normal_()
        one = torch.empty((1, 4096), dtype=dtype, device="cuda:0").normal_()
        read_s = best(lambda: ops.linear(one, big, out_dtype=torch.float32))
        gbs = big.numel() * big.element_size() / read_s / 1e9
        del big
        out = {"hbm_read_gbs": round(gbs, 1)}
        if self.engine_cfg.dtype == "bfloat16":
            n = 8192
            a = torch.empty((n, n), dtype=torch.bfloat16, device="cuda:0").normal_()
            b = torch.empty((n, n), dtype=torch.bfloat16, device="cuda:0").normal_()
            gemm_s = best(lambda: ops.linear(a, b))
            out["gemm_flops"] = round(2.0 * n ** 3 / gemm_s, -9)
        return out

    def prefill(self, tokens: int, repeats: int = 9) -> dict:
        from mercury_amd import SamplingParams

        times = []
        for _ in range(repeats + 1):
            rid = f"bench-{self.counter}"
            self.counter += 1
            self.engine.submit(rid, self.tokens(tokens), 1, lambda e: None,
                               params=SamplingParams(ignore_eos=True))
            self.sync()
            start = time.perf_counter()
            record = self.engine.step()
            self.sync()
            times.append(time.perf_counter() - start)
            assert record.prefill_tokens == tokens and not self.engine.sched.has_work()
        seconds = statistics.median(times[1:])
        return {"tok_s": tokens / seconds, "ms": 1e3 * seconds}


    def serve(self, requests: int, prompt_len: int, new_tokens: int) -> dict:
        """All requests submitted at once and run to their last token by the engine's own
        loop: prompts enter in portions under the token budget beside the decoding of the
        requests already in."""
        from mercury_amd import SamplingParams

        generated = [0]

        def sink(event):
            if event.kind == "token":
                generated[0] += 1

        for _ in range(requests):
            rid = f"bench-{self.counter}"
            self.counter += 1
            self.engine.submit(rid, self.tokens(prompt_len), new_tokens, sink,
                               params=SamplingParams(ignore_eos=True))
        self.engine._take_commands()
        self.sync()
        start = time.perf_counter()
        steps = mixed = 0
        split = {"sched": 0.0, "prepare": 0.0, "forward": 0.0}
        first_all_decoding = None
        while self.engine.sched.has_work():
            record = self.engine.step()
            steps += 1
            mixed += bool(record.num_prefill and record.num_decode)
            split["sched"] += record.sched_s
            split["prepare"] += record.prepare_s
            split["forward"] += record.forward_s
            if first_all_decoding is None and not record.num_prefill and not self.engine.sched.waiting:
                self.sync()
                first_all_decoding = time.perf_counter() - start
            if steps % 256 == 0:
                print(f"[bench] serve: step {steps}, {generated[0]} tokens", file=sys.stderr, flush=True)
        self.sync()
        elapsed = time.perf_counter() - start
        assert self.engine.leaked_blocks() == 0
        assert generated[0] == requests * new_tokens, (generated[0], requests * new_tokens)
        return {"tok_s": generated[0] / elapsed, "seconds": elapsed, "steps": steps, "mixed": mixed,
                "generated": generated[0], "prompt_seconds": first_all_decoding or 0.0,
                "preemptions": self.engine.metrics.summary().get("preemptions", 0),
                "split": {k: round(v, 3) for k, v in split.items()}}


def serve_main(args, model_name: str, cfg: dict, full_layers: int) -> int:
    prompt_len = args.context // 2
    new_tokens = args.context - prompt_len
    bench = Bench(cfg, args.dtype, args.serve_requests, args.context, args.seed,
                  not args.no_lookahead, prefill_budget=args.serve_chunk)
    run = bench.serve(args.serve_requests, prompt_len, new_tokens)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": f"generated tok/s, {args.serve_requests} requests of {prompt_len} prompt tokens "
                  f"in portions of {args.serve_chunk} beside decoding, to a context of "
                  f"{args.context} ({model_name} shapes)",
        "value": round(run["tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": run["steps"],
        "warmup": 0, "ms_per_step": round(1e3 * run["seconds"] / run["steps"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic: seeded uniform-random token ids, random weights N(0, 0.02) drawn on the GPU",
        "config": {"model": f"{model_name} shapes", "layers": cfg["num_hidden_layers"],
                   "layers_full": full_layers, "requests": args.serve_requests,
                   "prompt_len": prompt_len, "new_tokens": new_tokens,
                   "prefill_budget": args.serve_chunk, "seq_len": args.context,
                   "block_size": BLOCK_SIZE, "parallelism": "single GPU"},
        "seconds": round(run["seconds"], 3), "generated": run["generated"],
        "steps_with_prompt_and_decode": run["mixed"],
        "seconds_until_all_decode": round(run["prompt_seconds"], 3),
        "preemptions": run["preemptions"], "host_seconds": run["split"],
    }), flush=True)
    return 0


def attention_main(args) -> int:
    """The attention kernel by itself, as the model's layers call it: queries of prompt
    portions over a filled paged cache, the kernel and its shape chosen by the planner."""
    import numpy as np
    import torch

    from mercury_amd.engine.batch import StepContext
    from mercury_amd.kernels import ops

    dev = "cuda:0"

    def context(spans):
        step = StepContext()
        counts, starts = [c for c, _ in spans], [s for _, s in spans]
        cu = np.zeros(len(spans) + 1, dtype=np.int64)
        np.cumsum(counts, out=cu[1:])
        seq = np.repeat(np.arange(len(spans)), counts)
        positions = np.arange(int(cu[-1])) - cu[seq] + np.asarray(starts)[seq]
        put = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)
        step.num_tokens, step.num_seqs = int(cu[-1]), len(spans)
        step.token_ids = put(np.zeros(int(cu[-1])))
        step.positions, step.token_seq, step.cu_q = put(positions), put(seq), put(cu)
        step.kv_len = put(np.asarray(starts) + np.asarray(counts))
        step.state_slots = put(np.arange(len(spans)))
        step.spans = [(int(cu[i]), counts[i], starts[i]) for i in range(len(spans))]
        step.max_q_len, step.max_kv_len = max(counts), max(s + c for c, s in spans)
        step.all_decode = step.max_q_len == 1
        return step

    def run(spans, n_q, n_kv, d, repeats=10):
        step = context(spans)
        per = -(-max(c + s for c, s in spans) // BLOCK_SIZE)
        table = torch.arange(len(spans) * per, dtype=torch.int32, device=dev).view(len(spans), per)
        k_cache = torch.randn(len(spans) * per, n_kv, BLOCK_SIZE, d, device=dev).bfloat16()
        v_cache = torch.randn(len(spans) * per, n_kv, d, BLOCK_SIZE, device=dev).bfloat16()
        q = torch.randn(step.num_tokens, n_q * d, device=dev).bfloat16()
        call = lambda: ops.attention(q, n_q * d, k_cache, v_cache, step, table, n_q, n_kv, d,
                                     d ** -0.5, kernel="mfma")
        for _ in range(3):
            call()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(repeats):
            call()
        end.record()
        end.synchronize()
        us = begin.elapsed_time(end) / repeats * 1e3
        flops = sum(4.0 * n_q * d * (c * s + c * (c + 1) / 2) for c, s in spans)
        return us, flops / us / 1e9

    print("| heads x size (kv heads) | tokens (over a prefix) | sequences | us | PFLOP/s | of 2.5 |")
    print("|---|---|---|---|---|---|")
    for n_q, n_kv, d in ((14, 2, 64), (28, 4, 64), (28, 4, 128), (40, 8, 128)):
        for count, prefix, seqs in ((2048, 0, 1), (8192, 0, 1), (2048, 0, 4), (2048, 30720, 1),
                                    (1024, 15360, 16)):
            us, rate = run([(count, prefix)] * seqs, n_q, n_kv, d)
            print(f"| {n_q} x {d} ({n_kv}) | {count} ({prefix}) | {seqs} | {us:.0f} | {rate:.3f} | "
                  f"{100 * rate / 2.5:.0f} % |", flush=True)
    return 0


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine "
              "has no multi-GPU path)")
        return 2
    if args.attention:
        return attention_main(args)
    model_name, shape = SHAPES[args.shape]
    cfg = dict(shape)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    if args.serve:
        return serve_main(args, model_name, cfg, full_layers)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    # requests are given a little room beyond the context they are measured at
    limit = cfg.get("max_position_embeddings", 1 << 30) - max_batch - 16
    if args.context > limit:
        print(f"[bench] context {args.context} leaves no room below the model's "
              f"{cfg['max_position_embeddings']} positions: measuring at {limit}",
              file=sys.stderr, flush=True)
        args.context = limit
    bench = Bench(cfg, args.dtype, max_batch, args.context, args.seed, not args.no_lookahead)

    main_run = bench.decode(args.batch, args.context, args.steps, args.warmup)
    print(f"[bench] decode b{args.batch}: {main_run['ms']:.3f} ms/step "
          f"(cache filled in {main_run['fill_s']:.1f} s)", file=sys.stderr, flush=True)
    pre = bench.prefill(PREFILL_TOKENS)
    print(f"[bench] prefill {PREFILL_TOKENS}: {pre['ms']:.2f} ms", file=sys.stderr, flush=True)
    points = {}
    if not args.no_points:
        half = bench.decode(args.batch, args.context // 2, max(8, args.steps // 2), min(args.warmup, 4))
        points[f"decode_b{args.batch}_ctx{args.context // 2}"] = round(half["tok_s"], 1)
        print(f"[bench] decode b{args.batch} at context {args.context // 2}: {half['ms']:.3f} ms/step",
              file=sys.stderr, flush=True)
        for b in (1, 64):
            steps = max(8, args.steps // 2)
            run = bench.decode(b, args.context, steps, min(args.warmup, 4))
            points[f"decode_b{b}"] = round(run["tok_s"], 1)
            print(f"[bench] decode b{b}: {run['ms']:.3f} ms/step", file=sys.stderr, flush=True)
        long = bench.prefill(LONG_PREFILL_TOKENS, repeats=3)
        points[f"prefill_{LONG_PREFILL_TOKENS}"] = round(long["tok_s"], 1)
        long_rate = prefill_flops(cfg, LONG_PREFILL_TOKENS) / (long["ms"] * 1e-3)
        print(f"[bench] prefill {LONG_PREFILL_TOKENS}: {long['ms']:.2f} ms "
              f"({long_rate / 1e15:.3f} PFLOP/s)", file=sys.stderr, flush=True)

    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    achieved = main_run["bytes"] / (main_run["ms"] * 1e-3) / 1e9
    peaks = bench.measured_peaks()
    print(f"[bench] this machine: {peaks}", file=sys.stderr, flush=True)
    prefill_rate = prefill_flops(cfg, PREFILL_TOKENS) / (pre["ms"] * 1e-3)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} ({model_name} shapes)",
        "value": round(main_run["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms"], 4),
        "device_ms_per_step": round(main_run["device_ms"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic: seeded uniform-random token ids, random weights N(0, 0.02) drawn on the GPU",
        "config": {
            "model": f"{model_name} shapes", "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"],
            "vocab": cfg["vocab_size"], "tied_embeddings": cfg["tie_word_embeddings"],
            "global_batch": args.batch, "seq_len": args.context,
            "prompt_len": main_run["prompt_len"], "block_size": BLOCK_SIZE,
            "prefill_tokens": PREFILL_TOKENS, "parallelism": "single GPU",
        },
        "prefill": {"value": round(pre["tok_s"], 1), "tokens": PREFILL_TOKENS,
                    "ms": round(pre["ms"], 4),
                    "frac": round(prefill_rate / PEAK_FLOPS[short], 5),
                    "measured_peak": peaks.get("gemm_flops"),
                    "frac_of_measured": (round(prefill_rate / peaks["gemm_flops"], 5)
                                         if peaks.get("gemm_flops") else None)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 5),
                     "measured_peak": peaks["hbm_read_gbs"],
                     "frac_of_measured": round(achieved / peaks["hbm_read_gbs"], 5)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

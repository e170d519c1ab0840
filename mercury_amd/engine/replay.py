"""Trace replay: feed given token ids through a model step by step and write logits.

Nothing is sampled and nothing is scheduled: each input line names, for every request of the
step, its next tokens and the places whose logits are wanted.  The replay drives the same
model, step function, cache manager and kernels that generation uses; it owns no forward
pass, cache or loader.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
              [--block-size B] [--max-live R]

``--max-tokens`` is the most tokens that live requests hold at any time, each request's count
rounded up to a multiple of 64 (of the page size, if that is larger); the cache pool is made
for exactly this many, so that pages are used again.  ``--block-size`` is the page size of the
cache (a power of two, default 16), ``--max-live`` the most requests live at a time.

Input (standard input, one JSON object per line):

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``DIR/<step>.f32`` receives the logits at the wanted
places, in the order of the entries and of ``want``, as little-endian float32 [wanted, vocab].
After every step a line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

DEFAULT_PAGE_SIZE = 16     # the engine's default block_size
DEFAULT_MAX_LIVE = 8
ROUNDING = 64              # a live request counts as its length rounded up to this many tokens


class ReplaySession:
    """Requests by id over one runner; `step` runs one input line."""

    def __init__(self, model_dir, dtype_name: str, max_tokens: int, device="cuda:0",
                 page_size: int = DEFAULT_PAGE_SIZE, max_live: int = DEFAULT_MAX_LIVE):
        import torch

        from ..cache import CacheManager
        from ..config.engine_config import _DTYPE_BY_NAME
        from ..weights.loader import load_model_folder
        from .runner import ModelRunner

        if dtype_name not in _DTYPE_BY_NAME:
            raise SystemExit(f"--dtype must be bfloat16 or float32, got {dtype_name!r}")
        dtype = _DTYPE_BY_NAME[dtype_name]
        self.torch = torch
        self.model = load_model_folder(model_dir, dtype, device)
        if page_size <= 0 or page_size & (page_size - 1):
            raise SystemExit(f"--block-size must be a power of two, got {page_size}")
        # Every live request counts as a multiple of max(64, page) tokens, so this many pages
        # hold whatever the trace keeps live, and not one page more.
        unit = max(ROUNDING, page_size)
        pages = max(1, -(-int(max_tokens) // unit) * (unit // page_size))
        has_state = any(layer.mixer.state_spec() is not None for layer in self.model.layers)
        self.manager = CacheManager(self.model.cache_slots, pages, page_size, int(max_live), has_state)
        limit = min(self.model.max_positions or pages * page_size, pages * page_size)
        self.runner = ModelRunner(self.model, self.manager, dtype, device, limit)
        self.progress: dict = {}

    def step(self, entries: list, end: list):
        """Returns float32 logits [wanted, V] on the host, or None when nothing is wanted."""
        from .batch import SeqChunk

        chunks, picks, repeated = [], [], False
        for entry in entries:
            key, tokens = entry["id"], list(entry["tokens"])
            want = list(entry.get("want", []))
            if not tokens:
                continue
            # A place wanted twice is computed once and written twice.
            once = sorted(set(want))
            repeated = repeated or len(once) != len(want)
            base = sum(len(c.want) for c in chunks)
            picks.extend(base + once.index(w) for w in want)
            want = once
            if key not in self.progress:
                if self.manager.admit(key, [], len(tokens)) is None:
                    raise RuntimeError(f"step cannot admit request {key!r}: the cache pool is full")
                self.progress[key] = 0
            start = self.progress[key]
            if not self.manager.grow(key, start, start + len(tokens)):
                raise RuntimeError(f"request {key!r} needs pages the cache pool does not have")
            chunks.append(SeqChunk(key, tokens, start, want))
        logits = None
        if chunks:
            out = self.runner.step(chunks)
            if out.shape[0]:
                logits = out.float().cpu()
                if repeated:
                    logits = logits[picks]
            for chunk in chunks:
                self.progress[chunk.key] += len(chunk.tokens)
                self.manager.trim(chunk.key, self.progress[chunk.key])
        for key in end:
            if key in self.progress:
                self.manager.free(key)
                del self.progress[key]
        return logits


def main(argv=None) -> int:
    parser = argparse.ArgumentParser("trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    parser.add_argument("--out", required=True, help="folder that receives <step>.f32")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (sizes the cache pool)")
    parser.add_argument("--block-size", type=int, default=DEFAULT_PAGE_SIZE,
                        help="tokens per cache page, a power of two")
    parser.add_argument("--max-live", type=int, default=DEFAULT_MAX_LIVE,
                        help="most requests live at a time")
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    session = ReplaySession(args.model, args.dtype, args.max_tokens, args.device,
                            page_size=args.block_size, max_live=args.max_live)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        logits = session.step(record.get("entries", []), record.get("end", []))
        if logits is not None:
            logits.numpy().astype("<f4", copy=False).tofile(out_dir / f"{record['step']}.f32")
        print(f"done {record['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Trace replay: feed given token ids through a model step by step and write logits.

Nothing is sampled and nothing is scheduled: each input line names, for every request of the
step, its next tokens and the places whose logits are wanted.  The replay drives the same
model, step function, cache manager and kernels that generation uses; it owns no forward
pass, cache or loader.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

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

PAGE_SIZE = 16
MAX_LIVE = 8


class ReplaySession:
    """Requests by id over one runner; `step` runs one input line."""

    def __init__(self, model_dir, dtype_name: str, max_tokens: int, device="cuda:0",
                 page_size: int = PAGE_SIZE):
        import torch

        from ..cache.manager import CacheManager
        from ..config.engine_config import _DTYPE_BY_NAME
        from ..weights.loader import load_model_folder
        from .runner import ModelRunner

        if dtype_name not in _DTYPE_BY_NAME:
            raise SystemExit(f"--dtype must be bfloat16 or float32, got {dtype_name!r}")
        dtype = _DTYPE_BY_NAME[dtype_name]
        self.torch = torch
        self.model = load_model_folder(model_dir, dtype, device)
        pages = max(1, -(-int(max_tokens) // page_size))
        has_state = any(layer.mixer.state_spec() is not None for layer in self.model.layers)
        self.manager = CacheManager(self.model.cache_slots, pages, page_size, MAX_LIVE, has_state)
        limit = min(self.model.max_positions or pages * page_size, pages * page_size)
        self.runner = ModelRunner(self.model, self.manager, dtype, device, limit)
        self.progress: dict = {}

    def step(self, entries: list, end: list):
        """Returns float32 logits [wanted, V] on the host, or None when nothing is wanted."""
        from .batch import SeqChunk

        chunks = []
        for entry in entries:
            key, tokens = entry["id"], list(entry["tokens"])
            want = list(entry.get("want", []))
            if not tokens:
                continue
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
    parser.add_argument("--device", default="cuda:0")
    args = parser.parse_args(argv)

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    session = ReplaySession(args.model, args.dtype, args.max_tokens, args.device)
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

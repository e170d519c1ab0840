"""Shared by the tests: the two tiny configurations, model folders, replay drivers."""

from __future__ import annotations

import json
import subprocess
import sys
import tempfile
from pathlib import Path

import numpy as np
import torch

from tests.plain import qwen2_plain as plain

ROOT = Path(__file__).resolve().parent.parent

# Tiny Qwen2 configurations that differ in every size and option: heads and groups (GQA 4/2,
# MQA 8/1, a group of 3), head size (16, 32, 48), layers, vocabulary, eps, theta, tied vs
# untied head; C has a width, an intermediate size and a vocabulary that are no power of two
# nor a multiple of 64.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 64, "intermediate_size": 176, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "vocab_size": 512, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 2048,
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 256, "intermediate_size": 704, "num_hidden_layers": 3,
    "num_attention_heads": 8, "num_key_value_heads": 1, "head_dim": 32,
    "vocab_size": 1000, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 1024,
}
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "hidden_size": 168, "intermediate_size": 410, "num_hidden_layers": 1,
    "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48,
    "vocab_size": 1003, "rope_theta": 50000.0, "rms_norm_eps": 3e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 768,
}
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}

_FOLDERS: dict = {}


def model_folder(name: str, std: float = 0.05, seed: int = 7) -> Path:
    """A temporary model folder with bfloat16-representable random weights, written once per
    test process by the engine's random-weights mode."""
    from mercury_amd.weights import write_random_model

    key = (name, std, seed)
    if key not in _FOLDERS:
        folder = Path(tempfile.mkdtemp(prefix=f"mercury_tiny_{name}_"))
        write_random_model(folder, TINY[name], seed=seed, std=std, dtype=torch.bfloat16)
        _FOLDERS[key] = folder
    return _FOLDERS[key]


def plain_model(folder):
    return plain.read_weights(folder), plain.read_config(folder)


def random_tokens(vocab: int, count: int, seed: int) -> list:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()


def context_from_spans(spans: list, device, token_ids=None):
    """A step context without a cache manager: `spans` lists (token count, start position)
    per sequence.  Block tables are left to the caller."""
    from mercury_amd.engine.batch import StepContext

    step = StepContext()
    counts = [c for c, _ in spans]
    starts = [s for _, s in spans]
    cu = np.zeros(len(spans) + 1, dtype=np.int64)
    np.cumsum(counts, out=cu[1:])
    token_seq = np.repeat(np.arange(len(spans)), counts)
    positions = np.arange(int(cu[-1])) - cu[token_seq] + np.asarray(starts)[token_seq]
    as_dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=device)
    step.num_tokens, step.num_seqs = int(cu[-1]), len(spans)
    step.token_ids = as_dev(token_ids if token_ids is not None else np.zeros(int(cu[-1])))
    step.positions, step.token_seq, step.cu_q = as_dev(positions), as_dev(token_seq), as_dev(cu)
    step.kv_len = as_dev(np.asarray(starts) + np.asarray(counts))
    step.state_slots = as_dev(np.arange(len(spans)))
    step.spans = [(int(cu[s]), counts[s], starts[s]) for s in range(len(spans))]
    step.max_q_len, step.max_kv_len = max(counts), max(s + c for c, s in spans)
    step.all_decode = step.max_q_len == 1
    return step


class TraceRun:
    """Drives ``bin/trace_run`` as a child process, one step at a time."""

    def __init__(self, folder, dtype: str, max_tokens: int, block_size=None, max_live=None):
        self.out = Path(tempfile.mkdtemp(prefix="mercury_trace_"))
        options = []
        if block_size is not None:
            options += ["--block-size", str(block_size)]
        if max_live is not None:
            options += ["--max-live", str(max_live)]
        self.proc = subprocess.Popen(
            [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype",
             dtype, "--out", str(self.out), "--max-tokens", str(max_tokens), *options],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.step_no = 0
        self.vocab = json.loads((Path(folder) / "config.json").read_text())["vocab_size"]

    def step(self, entries, end=()):
        record = {"step": self.step_no, "entries": entries, "end": list(end)}
        self.proc.stdin.write(json.dumps(record) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {self.step_no}", f"trace_run said {line!r}"
        path = self.out / f"{self.step_no}.f32"
        self.step_no += 1
        wanted = sum(len(e.get("want", [])) for e in entries)
        if not wanted:
            assert not path.exists()
            return None
        data = np.fromfile(path, dtype="<f4")
        return torch.from_numpy(data.reshape(wanted, self.vocab).copy())

    def close(self) -> int:
        self.proc.stdin.close()
        return self.proc.wait(timeout=60)

"""Engine options: the reference's names and meanings where it has them
(reference: mercury/config.py:84-157), plus what chunked prefill and the cache groups need."""

from __future__ import annotations

from dataclasses import asdict, dataclass, field

import torch

POLICIES = ("fcfs", "lpm", "lpm_aging")

_DTYPE_BY_NAME = {
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
}


@dataclass
class EngineConfig:
    """
    model            folder with ``config.json`` and safetensors weights
    dtype            ``bfloat16`` (serving kernels) or ``float32`` (everything in true 32-bit)
    block_size       tokens per cache page (a power of two)
    num_blocks       pages in each cache group's pool; -1 sizes the pool to free memory
    max_running      most requests admitted at a time
    prefill_budget   most prompt tokens one step computes; longer prompts are cut into
                     portions (the reference admits whole prompts under this budget,
                     mercury/scheduler.py:146-152)
    max_model_len    most tokens (prompt + generated) a request may reach
    policy           admission order: ``fcfs``, ``lpm`` (longest cached prefix first) or
                     ``lpm_aging`` (the same with waiting time traded in and a deadline)
    aging_tokens_per_s, max_wait_s, scan_limit   parameters of the policies
    cryptographic_hashes   SHA-256 page hashes instead of the fast 64-bit ones
    seed             seed of the per-request sampling streams
    random_weights   draw the weights instead of reading them: `model` then names a folder
                     with a ``config.json`` (or that file), or the engine is given the
                     configuration as a dict; weight_seed and weight_std (the normal
                     deviates' spread; norm weights are 1 + deviate) say which weights,
                     weight_dtype the storage type they are rounded to, as a checkpoint's
                     would be, before the engine converts them to its own dtype
    """

    model: str = ""
    device: str = "cuda:0"
    dtype: str = "bfloat16"

    block_size: int = 16
    num_blocks: int = 4096
    gpu_memory_fraction: float = 0.85

    max_running: int = 64
    prefill_budget: int = 8192
    max_model_len: int = 8192

    policy: str = "fcfs"
    aging_tokens_per_s: float = 2000.0
    max_wait_s: float = 5.0
    scan_limit: int = 128

    cryptographic_hashes: bool = False
    seed: int = 0

    random_weights: bool = False
    weight_seed: int = 0
    weight_std: float = 0.02
    weight_dtype: str = "bfloat16"

    idle_sleep_s: float = 5e-4
    max_step_records: int = 500_000
    debug_invariants: bool = False
    use_graphs: bool = True
    # Captured decode graphs: one per (number of sequences, length bound), sharing one index
    # buffer and one workspace; at most max_graphs are kept (the least recently used goes),
    # and steps of more than max_graph_batch sequences are launched without a graph.
    max_graph_batch: int = 256
    max_graphs: int = 96
    # Start a decode step before the previous one's tokens have been read, when the scheduler
    # expects the same requests to go on (needs use_graphs).
    lookahead: bool = True

    extra: dict = field(default_factory=dict)

    def __post_init__(self) -> None:
        if self.policy not in POLICIES:
            raise ValueError(f"policy must be one of {POLICIES}, got {self.policy!r}")
        if self.dtype not in _DTYPE_BY_NAME:
            raise ValueError(
                f"unsupported dtype {self.dtype!r}; this engine runs {sorted(set(_DTYPE_BY_NAME))}"
            )
        if self.weight_dtype not in _DTYPE_BY_NAME:
            raise ValueError(f"unsupported weight_dtype {self.weight_dtype!r}")
        if self.block_size <= 0 or self.block_size & (self.block_size - 1):
            raise ValueError("block_size must be a positive power of two")
        if self.max_running <= 0:
            raise ValueError("max_running must be positive")
        if self.prefill_budget <= 0:
            raise ValueError("prefill_budget must be positive")

    @property
    def torch_dtype(self) -> torch.dtype:
        return _DTYPE_BY_NAME[self.dtype]

    @property
    def kv_capacity_tokens(self) -> int:
        return self.num_blocks * self.block_size

    def validate_against(self, max_position_embeddings: int) -> None:
        """(reference: mercury/config.py:133-145)"""
        if self.max_model_len > max_position_embeddings:
            raise ValueError(
                f"max_model_len {self.max_model_len} exceeds the model's "
                f"{max_position_embeddings} position embeddings"
            )
        if self.num_blocks > 0 and self.kv_capacity_tokens < self.max_model_len:
            raise ValueError(
                f"the cache pool holds {self.kv_capacity_tokens} tokens but a single request may "
                f"reach {self.max_model_len}; such a request would preempt itself forever. "
                f"Raise num_blocks above {self.max_model_len // self.block_size} or lower "
                f"max_model_len."
            )

    def to_dict(self) -> dict:
        return asdict(self)


def blocks_for_capacity(num_tokens: int, block_size: int = 16) -> int:
    """Pages that hold `num_tokens` (reference: mercury/config.py:160-161)."""
    return max(1, -(-int(num_tokens) // block_size))

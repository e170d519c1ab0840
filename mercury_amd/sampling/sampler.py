"""Turning logits into tokens: greedy, temperature and nucleus sampling
(reference: mercury/sampling.py:17-35), with one reproducible random stream per request.

The reference draws every row of a step from one engine-wide generator, so a request's tokens
depend on what else is in the batch.  Here the uniform number for output token `index` of a
request is a function of (seed, request id, index) alone: a request samples the same tokens
alone, batched, cut into portions or after a preemption.
"""

from __future__ import annotations

import hashlib
import struct

import torch

from ..kernels import ops


def uniform_for(seed: int, rid: str, index: int) -> float:
    """A number in [0, 1) with 24 random bits, from a keyed hash of the three arguments."""
    digest = hashlib.blake2b(f"{rid}:{index}".encode(), digest_size=8,
                             key=struct.pack("<q", int(seed) & (2**63 - 1))).digest()
    return (int.from_bytes(digest, "little") >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, seed: int = 0):
        self.seed = int(seed)
        self._staging: list = []     # pinned [3, n] float32 buffers, used in turn
        self._next = 0

    def _to_device(self, rows: list, device) -> torch.Tensor:
        """[len(rows), n] float32 on the device without making the host wait for the GPU: a
        copy out of pageable memory would, and a step may be running ahead.  A staging buffer
        comes round again after four uses, long after its copy has run (at most two steps'
        sampling is ever in flight)."""
        n = len(rows[0])
        if device.type != "cuda":
            return torch.tensor(rows, dtype=torch.float32, device=device)
        if not self._staging or self._staging[0].numel() < len(rows) * n:
            size = len(rows) * max(256, 2 * n)
            self._staging = [torch.empty(size, dtype=torch.float32, pin_memory=True)
                             for _ in range(4)]
        host = self._staging[self._next][: len(rows) * n].view(len(rows), n)
        self._next = (self._next + 1) % len(self._staging)
        host.copy_(torch.tensor(rows, dtype=torch.float32))
        return host.to(device, non_blocking=True)

    def sample(self, logits: torch.Tensor, requests: list) -> list:
        """One token per row of float32 logits [n, V]; row i belongs to requests[i], whose
        next output index is request.num_out."""
        if not requests:
            if logits.shape[0]:
                raise ValueError(f"{logits.shape[0]} rows of logits for no requests")
            return []
        return self.launch(logits, requests).cpu().tolist()

    def launch(self, logits: torch.Tensor, requests: list, ahead: int = 0) -> torch.Tensor:
        """The same as int32 tokens [n] left on the device, without waiting for them.  `ahead`
        is how many tokens each request will have got before this one that it has not got
        yet (for a step started before the previous one's tokens were read)."""
        if logits.shape[0] != len(requests):
            raise ValueError(f"{logits.shape[0]} rows of logits for {len(requests)} requests")
        if all(r.params.greedy for r in requests):
            return ops.argmax(logits)
        temps = [float(r.params.temperature) for r in requests]
        top_ps = [float(r.params.top_p) for r in requests]
        us = [uniform_for(self.seed if r.params.seed is None else r.params.seed, r.rid,
                          r.num_out + ahead) for r in requests]
        packed = self._to_device([temps, top_ps, us], logits.device)
        nucleus = packed[1] if any(p < 1.0 for p in top_ps) else None
        return ops.sample(logits, packed[0], nucleus, packed[2])

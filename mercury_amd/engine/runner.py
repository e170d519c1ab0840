"""The step function: run a batch of next tokens through the model, from the cache, and
return the logits at the wanted places.

`ModelRunner` owns the device memory that outlives a step: the paged key/value tensors of
every cache slot and the per-request state tensors.  It runs only the tokens it is given;
everything earlier comes from the cache that earlier steps left
(reference: mercury/runner.py:106-178 runs prompts and decoding as separate forwards and
returns sampled tokens; here one forward takes any mix and returns logits).
"""

from __future__ import annotations

import torch

from ..parts.base import LayerCache
from .batch import SeqChunk, StepContext, build_step


def require_gpu(device: torch.device) -> None:
    if device.type != "cuda":
        raise RuntimeError(
            f"the step function runs hand-written GPU kernels only; device {device} is not a GPU")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible to this process; there is no CPU path")


class ModelRunner:
    def __init__(self, model, manager, dtype: torch.dtype, device, max_model_len: int):
        device = torch.device(device)
        require_gpu(device)
        self.model, self.manager = model, manager
        self.dtype, self.device = dtype, device
        self.max_model_len = int(max_model_len)
        self.page_size = manager.page_size
        model.prepare(self.max_model_len, device)

        # Paged keys [pages, kv_heads, page, head_dim] and values [pages, kv_heads, head_dim,
        # page] per cache slot.
        self.kv = {}
        for slot, spec in model.cache_slots.items():
            group = manager.group_of_slot[slot]
            pages = manager.groups[group].pool.num_pages
            self.kv[slot] = (
                torch.zeros((pages, spec.kv_heads, self.page_size, spec.head_dim), dtype=dtype, device=device),
                torch.zeros((pages, spec.kv_heads, spec.head_dim, self.page_size), dtype=dtype, device=device))
        self.caches = {}
        for n, call in enumerate(model.calls):
            if call.cache is None:
                continue
            k, v = self.kv[call.cache]
            self.caches[n] = LayerCache(k, v, manager.group_of_slot[call.cache], self.page_size,
                                        call.writes)
        # Per-request state of fixed size, one tensor per layer that declares it.
        self.states = {}
        for i, layer in enumerate(model.layers):
            spec = layer.mixer.state_spec()
            if spec is not None:
                self.states[i] = torch.zeros((manager.state_slots.num_slots, *spec.shape),
                                             dtype=spec.dtype, device=device)

    @property
    def kv_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for kv in self.kv.values() for t in kv)

    def kv_bytes_per_token(self) -> int:
        return sum(2 * k.shape[1] * k.shape[3] * k.element_size() for k, _ in self.kv.values())

    def build(self, chunks: list) -> StepContext:
        return build_step(chunks, self.manager, self.model.vocab_size, self.max_model_len,
                          self.device)

    @torch.inference_mode()
    def step(self, chunks: list) -> torch.Tensor:
        """Run the chunks' tokens as one batch.  Returns float32 logits [wanted, V] in the
        order of the chunks and of each chunk's `want`."""
        ctx = self.build(chunks)
        return self.run(ctx)

    @torch.inference_mode()
    def run(self, ctx: StepContext) -> torch.Tensor:
        if self.states and ctx.fresh_slots:
            index = torch.tensor(ctx.fresh_slots, device=self.device)
            for state in self.states.values():
                state.index_fill_(0, index, 0)
        return self.model.forward(ctx, self.caches, self.states)


__all__ = ["ModelRunner", "SeqChunk", "StepContext"]

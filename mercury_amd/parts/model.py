"""A decoder as data: embedding, a list of layers, the order they run in, final norm, head."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops
from .base import Norm, Part, TensorSpec
from .block import PreNormBlock


@dataclass(frozen=True)
class LayerCall:
    """One entry of the execution list.

    layer
        index into the model's layers (their weights); a layer may be named more than once.
    cache
        the cache slot this call works on, or None when the mixer keeps no paged cache.
        Calls that name the same slot share keys and values.
    writes
        whether this call writes its tokens' keys and values into the slot; a call that only
        reads attends over what the writing call stored earlier in the same step.
    """

    layer: int
    cache: int | None
    writes: bool = True


class DecoderModel(Part):
    """Token embedding -> layers in execution-list order -> final norm -> output head.

    The head multiplies by ``head_name`` or, when `tied`, by the embedding matrix
    (reference: mercury/model/qwen2.py:100-114, :128-130, :145-150).  Logits are float32.
    """

    def __init__(self, vocab_size: int, hidden_size: int, layers: list, final_norm: Norm,
                 tied_head: bool, calls: list | None = None, layer_prefix: str = "model.layers.{}.",
                 embed_name: str = "model.embed_tokens.weight",
                 norm_prefix: str = "model.norm.", head_name: str = "lm_head.weight",
                 max_positions: int = 0, eos_token_ids: tuple = (), config=None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.layers = list(layers)
        self.final_norm = final_norm
        self.tied_head = bool(tied_head)
        self.calls = list(calls) if calls is not None else [
            LayerCall(i, i if layer.mixer.cache_spec() is not None else None)
            for i, layer in enumerate(self.layers)
        ]
        self.layer_prefix, self.embed_name = layer_prefix, embed_name
        self.norm_prefix, self.head_name = norm_prefix, head_name
        self.max_positions = int(max_positions)
        self.eos_token_ids = tuple(eos_token_ids)
        self.config = config
        self.embedding = self.head = None
        self.dtype = None
        self._check_calls()

    def _check_calls(self) -> None:
        writers = {}
        for n, call in enumerate(self.calls):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"execution list entry {n} names layer {call.layer}")
            spec = self.layers[call.layer].mixer.cache_spec()
            if (spec is None) != (call.cache is None):
                raise ValueError(f"execution list entry {n}: cache slot does not match the mixer")
            if call.cache is None:
                continue
            if call.writes:
                if call.cache in writers:
                    raise ValueError(f"cache slot {call.cache} is written by two entries")
                writers[call.cache] = spec
            elif call.cache not in writers:
                raise ValueError(f"entry {n} reads cache slot {call.cache} before it is written")
            elif writers[call.cache].as_tuple()[:4] != spec.as_tuple()[:4]:
                raise ValueError(f"entry {n} reads cache slot {call.cache} of another shape")
        self.cache_slots = writers  # slot -> CacheSpec

    # ---- tensors

    def ignored_names(self) -> set:
        """Checkpoint tensors that may be present without a home: a stored head beside a
        tied embedding (reference: mercury/model/loader.py:88-89)."""
        return {self.head_name} if self.tied_head else set()

    def param_specs(self) -> dict:
        specs = {self.embed_name: TensorSpec((self.vocab_size, self.hidden_size))}
        for i, layer in enumerate(self.layers):
            prefix = self.layer_prefix.format(i)
            for name, spec in layer.param_specs().items():
                specs[prefix + name] = spec
        for name, spec in self.final_norm.param_specs().items():
            specs[self.norm_prefix + name] = spec
        if not self.tied_head:
            specs[self.head_name] = TensorSpec((self.vocab_size, self.hidden_size))
        return specs

    def bind(self, params, dtype, device) -> None:
        self.dtype = dtype
        self.embedding = params[self.embed_name]
        self.head = self.embedding if self.tied_head else params[self.head_name]
        for i, layer in enumerate(self.layers):
            prefix = self.layer_prefix.format(i)
            layer.bind({n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)},
                       dtype, device)
        prefix = self.norm_prefix
        self.final_norm.bind({n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)},
                             dtype, device)

    def prepare(self, max_positions: int, device) -> None:
        for layer in self.layers:
            layer.prepare(max_positions, device)

    def kv_bytes_per_token(self, dtype: torch.dtype) -> int:
        """Bytes of keys and values one token adds to the cache, over all cache slots
        (reference: mercury/config.py:73-81)."""
        total = 0
        for spec in self.cache_slots.values():
            elem = torch.empty((), dtype=spec.dtype or dtype).element_size()
            total += spec.kv_heads * (spec.head_dim + spec.v_dim) * elem
        return total

    def decode_weight_bytes(self) -> int:
        """Bytes of weights a step reads once: every layer the execution list runs, the final
        norm and the head (the embedding is gathered, not streamed)."""
        total = sum(self.layers[c.layer].weight_bytes() for c in self.calls)
        total += self.final_norm.weight_bytes()
        total += self.head.numel() * self.head.element_size()
        return total

    # ---- as a program of the host core

    def compile(self, caches: dict, states: dict):
        """The step as a program: embedding, every execution-list entry whose layer hands its
        work over (the others stay with the caller, as one `host` operation each), final norm
        and head."""
        from ..hostcore import core

        if not getattr(self.final_norm, "lowerable", False):
            return None
        program = core.Program(ops.dtype_code(self.dtype), self.hidden_size, self.vocab_size)
        program.embed(self.embedding.data_ptr(), ops.dtype_code(self.embedding.dtype), self.vocab_size)
        for n, call in enumerate(self.calls):
            layer = self.layers[call.layer]
            can = getattr(layer, "lowerable_with", None)
            if can is not None and can(states.get(call.layer)):
                layer.lower(program, caches.get(n))
            else:
                program.host(n)
        norm = self.final_norm
        program.head(norm.weight.data_ptr(), ops.dtype_code(norm.weight.dtype), norm.eps,
                     self.head.data_ptr())
        return program

    # ---- one step

    def forward(self, step, caches: dict, states: dict) -> torch.Tensor:
        """Run the step's tokens; return float32 logits [len(step.logit_rows), V].

        caches: execution-list index -> LayerCache; states: layer index -> state tensor.
        """
        with ops.on_current_stream():
            h = ops.embed(step.token_ids, self.embedding)
            pending = None
            for n, call in enumerate(self.calls):
                pending = self.layers[call.layer].forward(
                    h, step, caches.get(n), states.get(call.layer), self.dtype, pending)
            if step.num_logit_rows == 0:
                return torch.empty((0, self.vocab_size), dtype=torch.float32, device=h.device)
            x = self.final_norm.forward(h, self.dtype, rows=step.logit_rows, partials=pending)
            return ops.linear(x, self.head, out_dtype=torch.float32)

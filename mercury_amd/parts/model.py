"""A decoder as data: embedding, a list of layers, the order they run in, final norm, head."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops
from .base import Norm, Part
from .embedding import OutputHead, TokenEmbedding


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


@dataclass
class Registers:
    """What a step of the program works on, as tensors, for a step the caller runs itself:
    the float32 residual stream `h`, the previous operation's output `x` and partial sums
    `pending` (either may be None), the step context, and `logits` once they exist.  A
    caller-run step changes h in place and leaves its own `x`, `pending` or `logits` here."""

    h: torch.Tensor
    x: torch.Tensor | None
    pending: torch.Tensor | None
    step: object
    logits: torch.Tensor | None = None


@dataclass
class CallerStep:
    """An entry of the program that stays with Python: `run(registers)`."""

    run: object
    gives_x: bool = False
    what: str = ""


class DecoderModel(Part):
    """Embedding -> layers in execution-list order -> final norm -> output head, each a part.

    `embedding` and `head` default to a plain lookup and a bias-free product with
    ``head_name`` or, when `tied_head`, with the embedding matrix
    (reference: mercury/model/qwen2.py:100-114, :128-130, :145-150); a model with a scaled
    embedding, a head bias or capped logits passes parts that say so.  Logits are float32.
    """

    def __init__(self, vocab_size: int, hidden_size: int, layers: list, final_norm: Norm,
                 tied_head: bool, calls: list | None = None, layer_prefix: str = "model.layers.{}.",
                 embed_name: str = "model.embed_tokens.weight",
                 norm_prefix: str = "model.norm.", head_name: str = "lm_head.weight",
                 max_positions: int = 0, eos_token_ids: tuple = (), config=None,
                 embedding: Part | None = None, head: Part | None = None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.layers = list(layers)
        self.final_norm = final_norm
        self.tied_head = bool(tied_head)
        self.calls = list(calls) if calls is not None else [
            LayerCall(i, i if layer.mixer.cache_spec() is not None else None)
            for i, layer in enumerate(self.layers)
        ]
        if not embed_name.endswith("weight") or not head_name.endswith("weight"):
            raise ValueError("embed_name and head_name name the parts' `weight` tensors")
        self.layer_prefix, self.embed_name = layer_prefix, embed_name
        self.norm_prefix, self.head_name = norm_prefix, head_name
        self.embed_prefix = embed_name[:-len("weight")]
        self.head_prefix = head_name[:-len("weight")]
        self.embedding_part = embedding or TokenEmbedding(self.vocab_size, self.hidden_size)
        self.head_part = head or OutputHead(self.vocab_size, self.hidden_size, tied=self.tied_head)
        self.max_positions = int(max_positions)
        self.eos_token_ids = tuple(eos_token_ids)
        self.config = config
        self.embedding = self.head = None
        self.dtype = None
        self.caller_steps: list = []
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
        specs = {self.embed_prefix + name: spec
                 for name, spec in self.embedding_part.param_specs().items()}
        for i, layer in enumerate(self.layers):
            prefix = self.layer_prefix.format(i)
            for name, spec in layer.param_specs().items():
                specs[prefix + name] = spec
        for name, spec in self.final_norm.param_specs().items():
            specs[self.norm_prefix + name] = spec
        for name, spec in self.head_part.param_specs().items():
            specs[self.head_prefix + name] = spec
        return specs

    def bind(self, params, dtype, device) -> None:
        self.dtype = dtype
        under = lambda prefix: {n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)}
        self.embedding_part.bind(under(self.embed_prefix), dtype, device)
        self.embedding = params[self.embed_name]
        head_params = under(self.head_prefix)
        if self.tied_head:
            head_params["weight"] = self.embedding
        self.head_part.bind(head_params, dtype, device)
        self.head = head_params["weight"]
        for i, layer in enumerate(self.layers):
            layer.bind(under(self.layer_prefix.format(i)), dtype, device)
        self.final_norm.bind(under(self.norm_prefix), dtype, device)

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
        total += self.head_part.weight_bytes()
        return total

    # ---- as a program of the host core

    def compile(self, caches: dict, states: dict):
        """The step as a program: the embedding, every execution-list entry, the final norm
        over the wanted rows, the head.  A part that hands its work over appends its
        operations; any other becomes a step the caller runs (`caller_steps`, by index), on
        the same registers, between two stretches of the program."""
        from ..hostcore import core

        program = core.Program(ops.dtype_code(self.dtype), self.hidden_size, self.vocab_size)
        self.caller_steps = []

        def stays(run, what, gives_x=False):
            self.caller_steps.append(CallerStep(run, gives_x, what))
            program.host(len(self.caller_steps) - 1, gives_x)

        if self.embedding_part.can_lower():
            self.embedding_part.lower(program)
        else:
            stays(lambda r: self.embedding_part.forward(r.step, out=r.h), "embedding")
        for n, call in enumerate(self.calls):
            layer = self.layers[call.layer]
            cache, state = caches.get(n), states.get(call.layer)
            can = getattr(layer, "lowerable_with", None)
            if can is not None and can(state):
                if state is None:
                    layer.lower(program, cache)
                else:
                    layer.lower(program, cache, state)
                continue

            def run_layer(r, layer=layer, cache=cache, state=state):
                r.pending = layer.forward(r.h, r.step, cache, state, self.dtype, r.pending)
                r.x = None

            stays(run_layer, f"layer {call.layer}")
        if self.final_norm.can_lower():
            self.final_norm.lower(program, select_rows=True)
        else:
            def run_norm(r):
                r.x = self.final_norm.forward(r.h, self.dtype, rows=r.step.logit_rows,
                                              partials=r.pending)
                r.pending = None

            stays(run_norm, "final norm", gives_x=True)
        if self.head_part.can_lower():
            self.head_part.lower(program)
        else:
            def run_head(r):
                r.logits = self.head_part.forward(r.x)
                r.x = None

            stays(run_head, "head")
        # a dry walk over a small step: operations that do not fit together fail here, at
        # build time, with the operation's index in the message
        program.workspace_bytes_for([2, 1], 2, 3, 1 + max((c.group for c in caches.values()), default=0))
        return program

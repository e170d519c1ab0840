"""Causal grouped-query softmax attention over a paged cache."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import CacheSpec, Mixer, PositionEncoding, TensorSpec
from .lowering import OneOp

# Leaf names of the stored tensors, under the prefix the builder gives; an architecture whose
# checkpoints call them otherwise passes its own map.
DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj"}


class Attention(Mixer):
    """q/k/v projections (optionally biased), position encoding on q and k, keys and values
    written to the paged cache, softmax(q k^T * scale) v over the sequence's cached keys,
    output projection (optionally biased) added into the accumulator.

    Query head h reads key/value head h // (n_q / n_kv).  A query at absolute position p sees
    keys j <= p, and with a window only j > p - window
    (reference: mercury/model/qwen2.py:45-69, mercury/model/attention.py:9-32, :87-101).
    `names` maps q, k, v, o to the stored tensors' leaf names (default ``q_proj`` ...).
    `score_cap` bounds the scaled score to cap * tanh(score / cap); a position encoding may
    bring a penalty on the distance in the score (`PositionDescriptor.distance_slopes`).  The
    reference has neither; with either the float32-arithmetic attention kernel runs.
    """

    graph_safe = True   # forward launches kernels only: a decode step may be captured in a graph

    def __init__(self, hidden: int, n_q: int, n_kv: int, head_dim: int,
                 position: PositionEncoding, qkv_bias: bool = True, o_bias: bool = False,
                 scale: float | None = None, window: int | None = None,
                 names: dict | None = None, score_cap: float | None = None):
        if n_q % n_kv:
            raise ValueError(f"{n_q} query heads are not a multiple of {n_kv} key/value heads")
        self.hidden, self.n_q, self.n_kv, self.head_dim = int(hidden), int(n_q), int(n_kv), int(head_dim)
        self.position = position
        self.qkv_bias, self.o_bias = bool(qkv_bias), bool(o_bias)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window = int(window) if window else None
        self.score_cap = float(score_cap) if score_cap else 0.0
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None
        self._alone: dict = {}

    # ---- declarations

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.n_kv, self.head_dim, self.window)

    def param_specs(self) -> dict:
        q, kv, h = self.n_q * self.head_dim, self.n_kv * self.head_dim, self.hidden
        n = self.names
        specs = {
            f"{n['q']}.weight": TensorSpec((q, h)),
            f"{n['k']}.weight": TensorSpec((kv, h)),
            f"{n['v']}.weight": TensorSpec((kv, h)),
            f"{n['o']}.weight": TensorSpec((h, q)),
        }
        if self.qkv_bias:
            specs[f"{n['q']}.bias"] = TensorSpec((q,), role="vector")
            specs[f"{n['k']}.bias"] = TensorSpec((kv,), role="vector")
            specs[f"{n['v']}.bias"] = TensorSpec((kv,), role="vector")
        if self.o_bias:
            specs[f"{n['o']}.bias"] = TensorSpec((h,), role="vector")
        return specs

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # One projection for q, k and v: rows [q heads | k heads | v heads].
        self.w_qkv = torch.cat(
            [params[f"{n['q']}.weight"], params[f"{n['k']}.weight"], params[f"{n['v']}.weight"]],
            dim=0).contiguous()
        if self.qkv_bias:
            biases = [params[f"{n['q']}.bias"], params[f"{n['k']}.bias"], params[f"{n['v']}.bias"]]
            common = torch.float32 if any(b.dtype == torch.float32 for b in biases) else dtype
            self.b_qkv = torch.cat([b.to(common) for b in biases]).contiguous()
        self.w_o = params[f"{n['o']}.weight"]
        self.b_o = params.get(f"{n['o']}.bias")
        self._alone.clear()

    def prepare(self, max_positions: int, device) -> None:
        self.position.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        total = 0
        for t in (self.w_qkv, self.b_qkv, self.w_o, self.b_o):
            if t is not None:
                total += t.numel() * t.element_size()
        return total

    # ---- one step

    @property
    def lowerable(self) -> bool:
        """The host core runs this attention itself when the kernels can apply its position
        encoding."""
        return self.position.describe() is not None

    def lower(self, program, cache, state=None) -> None:
        pos = self.position.describe()
        if pos is None:
            raise ValueError("an attention whose position encoding applies itself is not lowered")
        spec = self.cache_spec()
        if spec.v_dim != self.head_dim:
            raise ValueError("the attention kernels keep values as wide as keys")
        if cache.k.dtype != self.w_qkv.dtype:
            raise ValueError("the kernels keep keys and values in the compute dtype")
        bias_code = lambda t: ops.dtype_code(t.dtype) if t is not None else ops.F32
        ptr = lambda t: 0 if t is None else t.data_ptr()
        w, b = self.w_qkv, self.b_qkv
        if not cache.writes:
            # Reads a cache another entry fills: only the queries are projected.
            rows = self.n_q * self.head_dim
            w, b = w[:rows], None if b is None else b[:rows]
        program.append("attention", core.attention_params(
            w_qkv=w.data_ptr(), b_qkv=ptr(b), b_qkv_dtype=bias_code(b),
            w_o=self.w_o.data_ptr(), b_o=ptr(self.b_o), b_o_dtype=bias_code(self.b_o),
            n_q=self.n_q, n_kv=self.n_kv, head_dim=self.head_dim, rotary_dim=pos.rotary_dim,
            cos=ptr(pos.cos), sin=ptr(pos.sin),
            table_positions=0 if pos.cos is None else pos.cos.shape[0],
            interleaved=pos.interleaved, k_cache=cache.k.data_ptr(), v_cache=cache.v.data_ptr(),
            group=cache.group, page_size=cache.page_size, scale=self.scale,
            window=self.window or 0, writes=cache.writes, score_cap=self.score_cap,
            distance_slopes=ptr(pos.distance_slopes)))

    def forward(self, x, step, cache, state, accum):
        if self.position.describe() is not None:
            # the operations `lower` appends, as a program of their own
            key = (cache.k.data_ptr(), cache.group, cache.writes)
            alone = self._alone.get(key)
            if alone is None:
                alone = self._alone[key] = OneOp(x.dtype, self.hidden, 0,
                                                 lambda program: self.lower(program, cache))
            _logits, _x, pending = alone.run(step, accum, x=x)
            return pending
        # The encoding applies itself: project, let it transform q and k where they lie, then
        # write keys and values to the cache as they are.
        n_q, n_kv, d = self.n_q, self.n_kv, self.head_dim
        table = step.block_tables[cache.group]
        w, b = self.w_qkv, self.b_qkv
        if not cache.writes:
            w, b = w[:n_q * d], None if b is None else b[:n_q * d]
        k_cache, v_cache = (cache.k, cache.v) if cache.writes else (None, None)
        q = ops.linear(x, w, b)
        heads_kv = n_kv if cache.writes else 0
        q_part = q[:, :n_q * d].view(-1, n_q, d)
        k_part = q[:, n_q * d:(n_q + heads_kv) * d].view(-1, heads_kv, d) if heads_kv else None
        self.position.apply(q_part, k_part, step.positions)
        ops.rope_kv_write(q, None, None, step.positions, step.token_seq, table, k_cache,
                          v_cache, n_q, heads_kv, d, 0, cache.writes)
        attended = ops.attention(q, q.shape[1], cache.k, cache.v, step, table, n_q, n_kv, d,
                                 self.scale, self.window, score_cap=self.score_cap)
        return ops.project_into_stream(attended, self.w_o, self.b_o, accum)

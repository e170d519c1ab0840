"""What every part of a layer declares and does.

A model is put together from parts: a *mixer* (what lets tokens see each other: attention
here), a *feed-forward*, *norms*, a *position encoding* inside the mixer, and a *block* that
arranges them around the residual stream.  A part is constructed from its own sizes and
constants only; it never learns which model, layer index or checkpoint it belongs to.  The
names under which its tensors are stored are given to it from outside (by the architecture's
builder), as a prefix.

Interfaces
----------
``Part.param_specs()``
    local tensor name -> :class:`TensorSpec`.  The loader checks the checkpoint against the
    union of all parts' specs and fills ``Part.bind``.
``Part.bind(params, dtype, device)``
    receives the loaded tensors (already on the device, in the dtype the spec's role
    implies) and may repack them (concatenate q/k/v, gate/up) for its kernels.
``Norm.forward(h, out_dtype, rows=None, partials=None) -> x``
    h is the float32 residual stream [T, H].
``Mixer.forward(x, step, cache, state, accum)`` / ``FeedForward.forward(x, step, accum)``
    x is the normed input [T, H] in the compute dtype; the part **adds** its output into
    ``accum`` (float32 [T, H]), which the block chooses (the residual stream in a pre-norm
    block).  ``step`` is the :class:`~mercury_amd.engine.batch.StepContext` of this step
    (per-token ids, positions and sequence index; per-sequence spans, lengths, block tables
    and state slots).  ``cache`` is the :class:`LayerCache` the execution list assigns to this
    call (possibly another layer's, read-only), ``state`` the per-request state tensor
    [slots, ...] when the mixer declared a :class:`StateSpec`.
``Mixer.cache_spec()`` / ``Mixer.state_spec()``
    what the cache manager must provide: pages of keys and values (all of them or a window),
    and/or a fixed-size state per request.
``PositionEncoding.describe()`` / ``PositionEncoding.apply(q, k, positions)``
    how the encoding transforms queries and keys: as a :class:`PositionDescriptor` the
    kernels apply themselves (fused into the projection where they can), or, when `describe`
    returns None, by the part's own `apply` on the projected q and k.
``Part.lower(program, ...)``
    optional: append the part's operations to a step program of the host core, which then
    launches them without coming back to Python (``csrc/host/program.*``).  An operation is
    a registered kind (``hostcore.core.register_op``) and a block of parameter bytes; the
    package's own kinds live in ``csrc/ops``.  A part without `lower` is run through its
    `forward`; a model may mix both kinds, layer by layer.  A subclass that overrides
    `forward` without defining `lower` again is run through its `forward` (`can_lower`).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class TensorSpec:
    """A stored tensor a part needs.

    role
        ``"matrix"``: an operand of a projection, kept in the compute dtype.
        ``"vector"``: a bias or norm weight; kept in float32 when the checkpoint stores it in
        32 bits, otherwise in the compute dtype.
        ``"table"``: integers, kept as int32.
    init
        how the random-weights mode fills it: ``"normal"`` (mean 0), ``"one_plus_normal"``
        (mean 1), ``"zeros"``.
    """

    shape: tuple
    role: str = "matrix"
    init: str = "normal"
    optional: bool = False


@dataclass(frozen=True)
class CacheSpec:
    """Per-token cache need of a mixer: keys of `kv_heads` heads of `head_dim` and values of as
    many heads of `value_dim` (default: the keys' width), stored as `dtype` (default: the
    model's compute dtype); all earlier tokens (`window` None) or the last `window` of them."""

    kv_heads: int
    head_dim: int
    window: int | None = None
    value_dim: int | None = None
    dtype: torch.dtype | None = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    def as_tuple(self) -> tuple:
        """(kv_heads, key width, value width, dtype code or -1, window or 0): what the cache
        manager groups slots by."""
        code = -1 if self.dtype is None else {torch.float32: 0, torch.bfloat16: 1}[self.dtype]
        return (self.kv_heads, self.head_dim, self.v_dim, code, self.window or 0)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer: one tensor of `shape` and `dtype` per request
    slot, zeroed when a request takes the slot."""

    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """The paged keys and values one execution-list entry works on.

    k: [pages, kv_heads, page_size, head_dim]; v: [pages, kv_heads, head_dim, page_size]
    (values lie transposed within a page, which is how the matrix-core attention kernels
    read them).  `group` indexes the step's block tables.
    `writes` is false when the entry only reads a cache another entry fills.
    """

    k: torch.Tensor
    v: torch.Tensor
    group: int
    page_size: int
    writes: bool = True


@dataclass(frozen=True)
class PositionDescriptor:
    """A position encoding as the kernels understand it: the first `rotary_dim` dims of every
    query and key head are turned by the angle tables `cos` / `sin` ([positions, rotary_dim/2],
    float32), pair j being dims (j, j + rotary_dim/2) of the head, or (2j, 2j + 1) when
    `interleaved`.  rotary_dim 0: queries and keys stay as projected.  `distance_slopes`
    (float32 [query heads]): an encoding that lives in the score, slope[head] * (query position
    - key position) being subtracted from it (the float32-arithmetic attention kernel computes
    that; the matrix-core kernels do not)."""

    rotary_dim: int = 0
    cos: torch.Tensor | None = None
    sin: torch.Tensor | None = None
    interleaved: bool = False
    distance_slopes: torch.Tensor | None = None


class Part:
    """Base of all parts: declares tensors, receives them."""

    # True when forward() only launches kernels on the current stream (no host reads of device
    # data, no host-side branching on them), so a decode step through the part can be captured
    # in a HIP graph and replayed.  A layer is captured only if all of its parts say so.
    graph_safe = False

    def param_specs(self) -> dict:
        return {}

    def bind(self, params: dict, dtype: torch.dtype, device) -> None:
        pass

    def weight_bytes(self) -> int:
        """Bytes of weights one step reads from this part (for roofline accounting)."""
        return 0

    # A part that can hand its work to the host core defines
    #     lower(self, program, ...) -> None
    # appending its operations to `program`; `lowerable` says whether this instance does (a
    # part may decide by its parameters, e.g. an attention whose position encoding applies
    # itself cannot).
    lowerable = False

    def can_lower(self) -> bool:
        """Whether the host core may run this part in place of its `forward`: the instance
        says so, its class (or a base) defines `lower`, and no class below that one overrides
        `forward`: an override the lowered operations know nothing of would silently never
        run."""
        if not self.lowerable:
            return False
        lower_in = forward_in = None
        for cls in type(self).__mro__:
            if lower_in is None and "lower" in cls.__dict__:
                lower_in = cls
            if forward_in is None and "forward" in cls.__dict__:
                forward_in = cls
        if lower_in is None:
            return False
        return forward_in is None or issubclass(lower_in, forward_in)


class Norm(Part):
    def forward(self, h, out_dtype, rows=None, partials=None):
        raise NotImplementedError


class PositionEncoding(Part):
    """Turns absolute positions into a transform of q and k.  `prepare` builds whatever tables
    the transform needs for positions [0, max_positions).  The mixer asks `describe()`; an
    encoding the kernels cannot express returns None there and transforms q and k itself in
    `apply`."""

    def prepare(self, max_positions: int, device) -> None:
        pass

    def describe(self) -> PositionDescriptor | None:
        return PositionDescriptor()

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """Transform, in place, the projected queries q [T, n_q, d] and keys k [T, n_kv, d]
        (views into one buffer; k is None when the layer reads another layer's keys) of the
        tokens at `positions` (int32 [T], absolute)."""
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> CacheSpec | None:
        return None

    def state_spec(self) -> StateSpec | None:
        return None

    def prepare(self, max_positions: int, device) -> None:
        pass

    def forward(self, x, step, cache, state, accum) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x, step, accum) -> None:
        raise NotImplementedError

"""Python faces of the HIP kernels: tensors in, tensors out, shapes checked before the launch.

Every function here runs a hand-written kernel on the current HIP stream of the tensors'
device.  Nothing falls back to the CPU or to a library routine: a tensor that is not on the
GPU, or a missing kernel library, raises.
"""

from __future__ import annotations

import torch

from . import lib as _lib

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelArgumentError(f"kernels take float32 or bfloat16 tensors, not {dtype}") from None


_pinned_stream: int | None = None


def _stream() -> int:
    if _pinned_stream is not None:
        return _pinned_stream
    return torch.cuda.current_stream().cuda_stream


class on_current_stream:
    """Within this context every kernel here goes to the stream that was current at its entry,
    looked up once instead of at every launch (the lookup costs as much as a launch).  Not to
    be held across a change of the current stream, such as entering a graph capture."""

    def __enter__(self):
        global _pinned_stream
        self.before = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self.before
        return False


def _dev(*tensors) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelArgumentError(
                "kernel arguments must live on the GPU; there is no CPU path in this engine"
            )
        if not t.is_contiguous():
            raise KernelArgumentError(f"kernel argument of shape {tuple(t.shape)} is not contiguous")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32:
        raise KernelArgumentError(f"{name} must be int32, got {t.dtype}")


# --------------------------------------------------------------------------------- plumbing
#
# Which kernel runs a projection, a q/k/v projection or an attention of given sizes, and with
# which arguments, is written down once, in the host core (csrc/ops/launch.cc, with the
# decisions and the measurements behind them in csrc/ops/dispatch.cc).  The functions below
# check shapes, allocate results and call those launch sequences by device address; a step's
# program calls the same ones.


def _core():
    from ..hostcore import core

    return core


def _ensure(x: torch.Tensor):
    """The libraries an operand of this dtype may need, loaded (into this process and into the
    host core, which makes the choices below)."""
    _lib.load("core")
    if x.dtype == torch.bfloat16:
        _lib.load("mfma")
    return _core()


class Scratch:
    """Memory for what a launch sequence allocates by itself (results and temporaries): one
    byte tensor, asked for once the sequence knows how much it needs; results are views of
    it, which keep it alive."""

    def __init__(self, device):
        self.device, self.tensor = device, None

    def __call__(self, nbytes: int) -> int:
        self.tensor = torch.empty(int(nbytes), dtype=torch.uint8, device=self.device)
        return self.tensor.data_ptr()

    def view(self, address: int, shape: tuple, dtype: torch.dtype) -> torch.Tensor:
        count = 1
        for n in shape:
            count *= n
        if count == 0 or self.tensor is None:
            return torch.empty(shape, dtype=dtype, device=self.device)
        offset = address - self.tensor.data_ptr()
        size = count * torch.empty((), dtype=dtype).element_size()
        if offset < 0 or offset + size > self.tensor.numel():
            raise RuntimeError("a launch sequence's result lies outside its scratch memory")
        return self.tensor[offset:offset + size].view(dtype).view(*shape)


# ------------------------------------------------------------------------------ row-wise ops


def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None,
          scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as float32 [T, H]."""
    _dev(ids, table, out)
    _i32(ids, "ids")
    tokens, (vocab, hidden) = ids.shape[0], table.shape
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    if out.shape != (tokens, hidden) or out.dtype != torch.float32:
        raise KernelArgumentError("embed: out must be float32 [T, H]")
    _ensure(table).launch_embed(_ptr(ids), _ptr(table), dtype_code(table.dtype), _ptr(out), tokens,
                                hidden, vocab, float(scale), _stream())
    return out


def rmsnorm(h: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: torch.Tensor | None = None, partials: torch.Tensor | None = None,
            out: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm of the float32 residual stream h [T, H] into `out_dtype`.

    `partials` [P, T, H] float32 are first summed into h (and h is updated); `rows` selects
    and orders the rows to normalise.
    """
    _dev(h, weight, rows, partials, out)
    if h.dtype != torch.float32 or h.dim() != 2:
        raise KernelArgumentError("rmsnorm: h must be float32 [T, H]")
    tokens, hidden = h.shape
    if weight.shape != (hidden,):
        raise KernelArgumentError(f"rmsnorm: weight {tuple(weight.shape)} does not match H={hidden}")
    n_partials = 0
    if partials is not None:
        if partials.dtype != torch.float32 or partials.shape[1:] != h.shape:
            raise KernelArgumentError("rmsnorm: partials must be float32 [P, T, H]")
        n_partials = partials.shape[0]
    out_rows = tokens
    if rows is not None:
        _i32(rows, "rows")
        out_rows = rows.shape[0]
    if out is None:
        out = torch.empty((out_rows, hidden), dtype=out_dtype, device=h.device)
    if out.shape != (out_rows, hidden) or out.dtype != out_dtype:
        raise KernelArgumentError("rmsnorm: out has the wrong shape or dtype")
    _ensure(h).launch_rmsnorm(_ptr(h), tokens, hidden, _ptr(partials), n_partials, _ptr(weight),
                              dtype_code(weight.dtype), float(eps), _ptr(rows), out_rows,
                              _ptr(out), dtype_code(out_dtype), _stream())
    return out


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i] for gate_up [T, 2I]."""
    _dev(gate_up, out)
    tokens, two_i = gate_up.shape
    if two_i % 2:
        raise KernelArgumentError("silu_mul: the last dimension must be even")
    inter = two_i // 2
    if out is None:
        out = torch.empty((tokens, inter), dtype=gate_up.dtype, device=gate_up.device)
    if out.shape != (tokens, inter) or out.dtype != gate_up.dtype:
        raise KernelArgumentError("silu_mul: out has the wrong shape or dtype")
    _ensure(gate_up).launch_silu_mul(_ptr(gate_up), _ptr(out), dtype_code(gate_up.dtype), tokens,
                                     inter, _stream())
    return out


def logit_cap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _dev(logits)
    if logits.dtype != torch.float32 or cap <= 0:
        raise KernelArgumentError("logit_cap: float32 logits and a positive cap are required")
    _ensure(logits).launch_logit_cap(_ptr(logits), logits.numel(), float(cap), _stream())
    return logits


# --------------------------------------------------------------------------------- projection

SKINNY_MAX_ROWS = 64           # most rows the fused skinny q/k/v kernel takes


def wants_partials(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether x W^T is best computed as K-split float32 partial sums (`linear_partials`):
    bfloat16 x of few enough rows, and a matrix large enough for bandwidth to matter, that
    whole-K workgroups would leave compute units idle or unevenly loaded."""
    core = _ensure(x)
    return core.wants_partials(dtype_code(x.dtype), dtype_code(w.dtype), x.shape[0], w.shape[0],
                               w.shape[1])


def _mfma_eligible(x, w: torch.Tensor) -> bool:
    return _core().mfma_eligible(dtype_code(x.dtype), dtype_code(w.dtype), x.shape[0], x.shape[1])


def linear_partials(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Float32 partial sums [P, M, N] of x W^T over P slices of K; the consumer (rmsnorm,
    rope_kv_write: their `partials` forms) adds them up in slice order.  At most 16 rows of
    a matrix of modest size: the weights stream straight into the matrix cores; otherwise
    tiles through LDS."""
    _dev(x, w)
    if not _mfma_eligible(x, w) or x.shape[1] != w.shape[1]:
        raise KernelArgumentError(f"linear_partials: x {tuple(x.shape)} / W {tuple(w.shape)} not eligible")
    m, k = x.shape
    n = w.shape[0]
    scratch = Scratch(x.device)
    address, slices = _ensure(x).launch_linear_partials(_ptr(x), m, _ptr(w), n, k,
                                                        dtype_code(x.dtype), scratch, _stream())
    return scratch.view(address, (slices, m, n), torch.float32)


def fuses_gating(x: torch.Tensor, w_gate_up: torch.Tensor) -> bool:
    """Whether `gated_projection` takes these operands (bfloat16, K a multiple of 8)."""
    if x.dtype not in _DTYPE_CODE or w_gate_up.dtype not in _DTYPE_CODE:
        return False
    return _core().fuses_gating(dtype_code(x.dtype), dtype_code(w_gate_up.dtype), x.shape[0],
                                x.shape[1], w_gate_up.shape[0])


def gated_projection(x: torch.Tensor, w_gate_up: torch.Tensor,
                     tile_config: int | None = None) -> torch.Tensor:
    """act = silu(x Wg^T) * (x Wu^T) for W = [Wg | Wu] stacked [2 I, K]: for bfloat16 one
    kernel on the matrix cores, the gating in the projection's epilogue (the skinny kernel for
    few rows, the tiled one for many; `tile_config` forces the tiled one with that tile
    configuration, -1 for its own choice); otherwise the projection and the gating kernel."""
    _dev(x, w_gate_up)
    if x.shape[1] != w_gate_up.shape[1] or w_gate_up.shape[0] % 2:
        raise KernelArgumentError("gated_projection: operands do not match")
    if tile_config is not None and not fuses_gating(x, w_gate_up):
        raise KernelArgumentError("gated_projection: operands not eligible")
    m, k = x.shape
    inter = w_gate_up.shape[0] // 2
    scratch = Scratch(x.device)
    address = _ensure(x).launch_gated(_ptr(x), m, k, _ptr(w_gate_up), inter, dtype_code(x.dtype),
                                      -2 if tile_config is None else int(tile_config), scratch,
                                      _stream())
    return scratch.view(address, (m, inter), x.dtype)


def linear(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None = None,
           out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
           accumulate: bool = False, kernel: str = "auto", tile_config: int = -1) -> torch.Tensor:
    """y = x W^T (+ bias) for x [M, K], W [N, K].

    With `accumulate` the product is added into the float32 tensor `out` (the residual
    stream) instead of being stored.  The result's dtype is `out_dtype` (default: x's).
    kernel: "auto" takes the matrix-core kernels for bfloat16 with K % 8 == 0 and the float32
    multiply-add kernel otherwise; "generic" and "mfma" force one.  tile_config picks the tile
    shape of the matrix-core kernel for many rows (-1: by the problem's size).
    """
    _dev(x, w, bias, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelArgumentError(f"linear: x {tuple(x.shape)} and W {tuple(w.shape)} do not match")
    if x.dtype != w.dtype:
        raise KernelArgumentError(f"linear: x is {x.dtype} but W is {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    if bias is not None and bias.shape != (n,):
        raise KernelArgumentError(f"linear: bias {tuple(bias.shape)} does not match N={n}")
    if accumulate:
        if out is None or out.dtype != torch.float32:
            raise KernelArgumentError("linear: accumulation needs a float32 `out`")
        out_dtype = torch.float32
    if out is None:
        out_dtype = out_dtype or x.dtype
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    else:
        out_dtype = out.dtype
    if out.shape != (m, n):
        raise KernelArgumentError(f"linear: out {tuple(out.shape)} is not [{m}, {n}]")
    if m == 0:
        return out
    if kernel == "mfma" and (x.dtype != torch.bfloat16 or k % 8):
        raise KernelArgumentError("linear: the matrix-core kernels take bfloat16 with K % 8 == 0")
    _ensure(x).launch_linear(_ptr(x), m, _ptr(w), n, k, dtype_code(x.dtype), _ptr(bias),
                             dtype_code(bias.dtype) if bias is not None else F32, _ptr(out),
                             dtype_code(out_dtype), bool(accumulate),
                             {"auto": 0, "generic": 1, "mfma": 2}[kernel], int(tile_config),
                             _stream())
    return out


def project_into_stream(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None,
                        h: torch.Tensor) -> torch.Tensor | None:
    """h += x W^T (+ bias), the way a step's program does it: where partial sums over slices of
    K stream the weights faster they are returned ([P, T, H] float32) for the next norm to add,
    and h is left as it is; otherwise None."""
    _dev(x, w, bias, h)
    if h.dtype != torch.float32 or h.shape != (x.shape[0], w.shape[0]) or x.shape[1] != w.shape[1]:
        raise KernelArgumentError("project_into_stream: shapes do not match the float32 stream")
    m, k = x.shape
    n = w.shape[0]
    scratch = Scratch(x.device)
    address, count = _ensure(x).launch_project(_ptr(x), m, _ptr(w), n, k, dtype_code(x.dtype),
                                               _ptr(bias),
                                               dtype_code(bias.dtype) if bias is not None else F32,
                                               _ptr(h), scratch, _stream())
    return scratch.view(address, (count, m, n), torch.float32) if count else None


# ---------------------------------------------------------------------- positions and the cache


def _check_caches(what, k_cache, v_cache, n_kv, head_dim, dtype) -> int:
    """Keys [pages, n_kv, page, d]; values transposed in the page [pages, n_kv, d, page]."""
    if k_cache is None or v_cache is None or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelArgumentError(f"{what}: 4-dimensional key and value caches are required")
    pages, heads, page_size, d = k_cache.shape
    if heads != n_kv or d != head_dim or tuple(v_cache.shape) != (pages, n_kv, head_dim, page_size):
        raise KernelArgumentError(
            f"{what}: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} are not "
            f"[pages, {n_kv}, page, {head_dim}] / [pages, {n_kv}, {head_dim}, page]")
    if k_cache.dtype != dtype or v_cache.dtype != dtype:
        raise KernelArgumentError(f"{what}: cache dtype differs from the activations'")
    return page_size


def _check_tables(what, cos, sin, rotary_dim) -> int:
    if not rotary_dim:
        return 0
    if cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
            or cos.shape != sin.shape or cos.shape[1] != rotary_dim // 2:
        raise KernelArgumentError(f"{what}: float32 cos and sin tables of the rotary width are required")
    return cos.shape[0]


def _qkv_args(what, w, bias, cos, sin, k_cache, v_cache, n_q, n_kv, head_dim, rotary_dim,
              write_kv, interleaved, dtype) -> dict:
    """The q/k/v side of an attention by name, as the launch sequences take it; checks the
    tables and the caches against the sizes."""
    page_size = _check_caches(what, k_cache, v_cache, n_kv, head_dim, dtype) if write_kv else 1
    return dict(
        w_qkv=_ptr(w), b_qkv=_ptr(bias), b_qkv_dtype=dtype_code(bias.dtype) if bias is not None else F32,
        n_q=n_q, n_kv=n_kv, head_dim=head_dim, rotary_dim=rotary_dim, cos=_ptr(cos), sin=_ptr(sin),
        table_positions=_check_tables(what, cos, sin, rotary_dim), interleaved=bool(interleaved),
        k_cache=_ptr(k_cache) if write_kv else 0, v_cache=_ptr(v_cache) if write_kv else 0,
        page_size=page_size, writes=bool(write_kv))


def _arrays(what, tokens, positions, token_seq, block_table, cu_q=None, kv_len=None) -> dict:
    _i32(positions, "positions")
    _i32(token_seq, "token_seq")
    _i32(block_table, "block_table")
    if positions.shape[0] != tokens or token_seq.shape[0] != tokens:
        raise KernelArgumentError(f"{what}: positions/token_seq must have one entry per token")
    if block_table.dim() != 2:
        raise KernelArgumentError(f"{what}: the block table is [sequences, pages]")
    return dict(positions=_ptr(positions), token_seq=_ptr(token_seq), cu_q=_ptr(cu_q),
                kv_len=_ptr(kv_len), table=_ptr(block_table), table_stride=block_table.shape[1])


def rope_kv_write(qkv: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  positions: torch.Tensor, token_seq: torch.Tensor, block_table: torch.Tensor,
                  k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, n_q: int,
                  n_kv: int, head_dim: int, rotary_dim: int, write_kv: bool = True,
                  bias: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
                  interleaved: bool = False):
    """Rotate q and k by their absolute positions; write k into the paged key cache
    [pages, n_kv, page_size, head_dim] and v into the value cache
    [pages, n_kv, head_dim, page_size] at the slots the block table gives.

    The first `rotary_dim` dims of a head turn; pair j is dims (j, j + rotary_dim/2), or
    (2j, 2j + 1) when `interleaved`.
    qkv [T, (n_q + 2 n_kv) d] in the compute dtype is rotated in place (q part) and returned.
    qkv as float32 partial sums [P, T, width] is summed (plus `bias`) first, and the rotated q
    comes back as a new [T, n_q d] tensor of `out_dtype`."""
    _dev(qkv, cos, sin, positions, token_seq, block_table, k_cache, v_cache, bias)
    heads_kv = n_kv if write_kv else 0
    width = (n_q + 2 * heads_kv) * head_dim
    if qkv.dim() == 3:
        slices, tokens, got = qkv.shape
        if qkv.dtype != torch.float32 or out_dtype is None:
            raise KernelArgumentError("rope: partial sums are float32 and need an out_dtype")
        if got != width:
            raise KernelArgumentError(f"rope: partial sums of width {got} do not match the heads")
        if bias is not None and bias.shape != (width,):
            raise KernelArgumentError("rope: bias does not match the projection width")
        args = _qkv_args("rope", None, bias, cos, sin, k_cache, v_cache, n_q, max(n_kv, 1),
                         head_dim, rotary_dim, write_kv, interleaved, out_dtype)
        scratch = Scratch(qkv.device)
        address = _ensure(qkv).launch_qkv_finish(
            _ptr(qkv), slices, tokens, dtype_code(out_dtype), args,
            _arrays("rope", tokens, positions, token_seq, block_table), scratch, _stream())
        return scratch.view(address, (tokens, n_q * head_dim), out_dtype)
    if bias is not None:
        raise KernelArgumentError("rope: a bias is only added to partial sums")
    tokens, row = qkv.shape
    args = _qkv_args("rope", None, None, cos, sin, k_cache, v_cache, n_q, max(n_kv, 1), head_dim,
                     rotary_dim, write_kv, interleaved, qkv.dtype)
    _ensure(qkv).launch_rope_kv_write(_ptr(qkv), row, tokens, dtype_code(qkv.dtype), args,
                                      _arrays("rope", tokens, positions, token_seq, block_table),
                                      _stream())
    return qkv


def fuses_qkv(x, w: torch.Tensor, head_dim: int, rotary_dim: int, page_size: int) -> bool:
    """Whether `qkv_project` runs as one kernel by itself: bfloat16 rows, K a multiple of 8,
    heads a multiple of 32 wide and rotated over their whole width or not at all, pages a
    power of two; and not up to a few hundred rows over a matrix so large that partial sums
    over slices of K, followed by the rotation, stream it faster (7168 x 5120 at 64 rows: 43 us
    in one kernel, 20 + 7 in two)."""
    return _qkv_kernel(x, w, head_dim, rotary_dim, page_size) in ("skinny", "tiled")


_QKV_KINDS = ("skinny", "tiled", "partials", "plain")


def _qkv_kernel(x, w, head_dim, rotary_dim, page_size, half_layout: bool = True):
    """ "skinny" (up to 64 rows: weights straight into the matrix cores, one workgroup per 32
    rows of W with all of K), "tiled" (any number of rows, through LDS, where whole-K tiles
    are the faster projection anyway), "partials" (K-split partial sums, then the finishing
    kernel) or "plain" (the projection, then the rotation and cache-write kernel)."""
    kind = _ensure(x).choose_qkv(dtype_code(x.dtype), dtype_code(w.dtype), x.shape[0], w.shape[0],
                                 x.shape[1], head_dim, rotary_dim, page_size, half_layout)
    return _QKV_KINDS[kind]


def qkv_project(x, w: torch.Tensor, bias: torch.Tensor | None, cos: torch.Tensor | None,
                sin: torch.Tensor | None, positions: torch.Tensor, token_seq: torch.Tensor,
                block_table: torch.Tensor, k_cache: torch.Tensor | None,
                v_cache: torch.Tensor | None, n_q: int, n_kv: int, head_dim: int,
                rotary_dim: int, write_kv: bool = True, fused: bool | None = None,
                tile_config: int = -1, interleaved: bool = False) -> torch.Tensor:
    """q, k, v = x W^T + bias for W = [q heads | k heads | v heads]; q and k rotated by their
    positions; k and v written to the paged cache (`write_kv`; otherwise W holds the query
    heads only).  Returns the rotated q, one row per token (the rows may be wider than
    n_q d: when the projection and the rotation are two kernels, q stays in the projected
    buffer).

    Where `fuses_qkv` says so, one kernel does all of it (projection, bias, rotation and cache
    write in its epilogue: the skinny kernel for few rows, the tiled one for many); otherwise
    the projection (whole or as partial sums) is followed by the rotation and cache write.
    `fused` forces one or the other, `tile_config` a tile configuration of the tiled kernel."""
    _dev(x, w, bias, cos, sin, positions, token_seq, block_table, k_cache, v_cache)
    heads_kv = n_kv if write_kv else 0
    width = (n_q + 2 * heads_kv) * head_dim
    if w.shape[0] != width or w.shape[1] != x.shape[1]:
        raise KernelArgumentError(f"qkv_project: W {tuple(w.shape)} is not [{width}, {x.shape[1]}]")
    if bias is not None and bias.shape != (width,):
        raise KernelArgumentError("qkv_project: bias does not match the projection width")
    page_size = k_cache.shape[2] if write_kv and k_cache is not None else 1
    half = not (interleaved and rotary_dim)
    core = _ensure(x)
    if fused is None:
        kind = -1
    elif not fused:
        kind = 2 if half and wants_partials(x, w) else 3
    elif not core.qkv_fusable(dtype_code(x.dtype), dtype_code(w.dtype), x.shape[0], x.shape[1],
                              head_dim, rotary_dim, page_size, half):
        raise KernelArgumentError("qkv_project: these operands cannot take the fused kernel")
    else:
        kind = 0 if x.shape[0] <= SKINNY_MAX_ROWS and tile_config < 0 else 1
    tokens, k = x.shape
    args = _qkv_args("qkv_project", w, bias, cos, sin, k_cache, v_cache, n_q, n_kv, head_dim,
                     rotary_dim, write_kv, interleaved, x.dtype)
    scratch = Scratch(x.device)
    address, stride = core.launch_qkv_project(
        _ptr(x), tokens, k, dtype_code(x.dtype), args,
        _arrays("qkv_project", tokens, positions, token_seq, block_table), kind, int(tile_config),
        scratch, _stream())
    return scratch.view(address, (tokens, stride), x.dtype)


def attention(q: torch.Tensor, q_stride: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
              step, block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int, scale: float,
              window: int | None = None, out: torch.Tensor | None = None,
              kernel: str = "auto", tile_rows: int | None = None,
              split_override: tuple | None = None, staged: bool | None = None,
              score_cap: float | None = None,
              distance_slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Causal grouped-query attention of every token of the step over its sequence's cached
    keys; q is read from rows of `q` with stride `q_stride` (the fused qkv buffer).
    `step` describes the batch (positions, token_seq, cu_q, kv_len, spans, tiles());
    `block_table` is the step's table of the cache group.  Returns [T, n_q * head_dim].

    kernel: "auto" takes the matrix-core kernel for bfloat16 where it covers the head and page
    size and the float32-arithmetic kernel otherwise; "generic" and "mfma" force one.
    tile_rows (16, 32 or 64) overrides how many rows a wavefront of the matrix-core kernel
    takes, split_override = (splits, key blocks per split) how the keys are split, staged
    (False, or 1, 2 or 4 groups of wavefronts that split a workgroup's keys among them)
    whether workgroups of four wavefronts share the keys and values of one sequence's rows
    through LDS; by default the step's size decides all three.
    score_cap bounds the scaled score to cap * tanh(score / cap); distance_slopes (float32
    [n_q]) subtracts slope[head] * (query position - key position) from it.  With either the
    float32-arithmetic kernel runs, whatever the dtype.
    """
    _dev(q, k_cache, v_cache, step.positions, step.token_seq, block_table, out, distance_slopes)
    if distance_slopes is not None and (distance_slopes.dtype != torch.float32
                                        or distance_slopes.shape != (n_q,)):
        raise KernelArgumentError(f"attention: distance_slopes must be float32 [{n_q}]")
    tokens = step.num_tokens
    if q.numel() < (tokens - 1) * q_stride + n_q * head_dim and tokens:
        raise KernelArgumentError("attention: q buffer too small")
    if block_table.dim() != 2 or block_table.shape[0] != step.num_seqs:
        raise KernelArgumentError("attention: the block table needs one row per sequence")
    page_size = _check_caches("attention", k_cache, v_cache, n_kv, head_dim, q.dtype)
    if out is not None and (out.shape != (tokens, n_q * head_dim) or out.dtype != q.dtype):
        raise KernelArgumentError("attention: out has the wrong shape or dtype")
    counts = [count for _first, count, _start in step.spans]
    force = dict(kernel={"auto": 0, "generic": 1, "mfma": 2}[kernel],
                 tile_rows=-1 if tile_rows is None else int(tile_rows),
                 staged=-1 if staged is None else int(staged),
                 splits=split_override[0] if split_override is not None else 0,
                 split_blocks=split_override[1] if split_override is not None else 0)
    args = dict(n_q=n_q, n_kv=n_kv, head_dim=head_dim, page_size=page_size,
                window=int(window or 0), scale=float(scale), k_cache=_ptr(k_cache),
                v_cache=_ptr(v_cache), score_cap=float(score_cap or 0.0),
                distance_slopes=_ptr(distance_slopes))

    def tiles(group, rows):
        seq, row0, count = step.tiles(group, rows)
        return _ptr(seq), _ptr(row0), count

    scratch = Scratch(q.device)
    address = _ensure(q).launch_attention(
        _ptr(q), int(q_stride), dtype_code(q.dtype), args,
        _arrays("attention", tokens, step.positions, step.token_seq, block_table, step.cu_q,
                step.kv_len),
        counts, step.max_q_len, step.max_kv_len, force, tiles, _ptr(out), scratch, _stream())
    if out is not None:
        return out
    return scratch.view(address, (tokens, n_q * head_dim), q.dtype)


def attention_project(q: torch.Tensor, q_stride: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      step, block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int,
                      scale: float, window: int | None, w_o: torch.Tensor,
                      b_o: torch.Tensor | None, h: torch.Tensor, fold: bool | None = None):
    """`attention` followed by the output projection into the float32 stream h [T, H], the way
    a step's program runs the two: h += attended W_o^T (+ b_o), or float32 partial sums
    [P, T, H] returned for the next norm to add.  Decoding with split keys merges the splits
    inside the projection's kernel where that pays (`fold`: None by the sizes, False never,
    True wherever the sizes allow)."""
    _dev(q, k_cache, v_cache, step.positions, step.token_seq, block_table, w_o, b_o, h)
    tokens, hidden = step.num_tokens, w_o.shape[0]
    if h.dtype != torch.float32 or h.shape != (tokens, hidden) or w_o.shape[1] != n_q * head_dim:
        raise KernelArgumentError("attention_project: shapes do not match the float32 stream")
    page_size = _check_caches("attention", k_cache, v_cache, n_kv, head_dim, q.dtype)
    counts = [count for _first, count, _start in step.spans]
    args = dict(n_q=n_q, n_kv=n_kv, head_dim=head_dim, page_size=page_size,
                window=int(window or 0), scale=float(scale), k_cache=_ptr(k_cache),
                v_cache=_ptr(v_cache))

    def tiles(group, rows):
        seq, row0, count = step.tiles(group, rows)
        return _ptr(seq), _ptr(row0), count

    scratch = Scratch(q.device)
    address, count = _ensure(q).launch_attention_project(
        _ptr(q), int(q_stride), dtype_code(q.dtype), args,
        _arrays("attention", tokens, step.positions, step.token_seq, block_table, step.cu_q,
                step.kv_len),
        counts, step.max_q_len, step.max_kv_len, tiles, _ptr(w_o), _ptr(b_o),
        dtype_code(b_o.dtype) if b_o is not None else F32, hidden, _ptr(h),
        -1 if fold is None else int(bool(fold)), scratch, _stream())
    return scratch.view(address, (count, tokens, hidden), torch.float32) if count else None


# ----------------------------------------------------------------------------------- sampling


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index of the largest value of each row of float32 logits [n, V] -> int32 [n]."""
    _dev(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelArgumentError("argmax: logits must be float32 [n, V]")
    rows, vocab = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    parts = torch.empty((rows, 64, 2), dtype=torch.int32, device=logits.device)
    lib = _lib.load("core")
    _lib.check(lib, lib.mk_argmax(_ptr(logits), rows, vocab, vocab, _ptr(out), _ptr(parts),
                                  _stream()), "argmax")
    return out


def sample(logits: torch.Tensor, temperatures: torch.Tensor, top_ps: torch.Tensor | None,
           uniforms: torch.Tensor) -> torch.Tensor:
    """One token per row: argmax where temperature <= 0, else an inverse-CDF draw from the
    temperature softmax restricted to the nucleus, using the row's uniform number.
    `top_ps` None says that no row restricts its nucleus, which takes a faster path (the
    vocabulary shared out over many workgroups, no threshold search)."""
    _dev(logits, temperatures, top_ps, uniforms)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelArgumentError("sample: logits must be float32 [n, V]")
    rows, vocab = logits.shape
    for name, t in (("temperatures", temperatures), ("top_ps", top_ps), ("uniforms", uniforms)):
        if t is not None and (t.dtype != torch.float32 or t.shape != (rows,)):
            raise KernelArgumentError(f"sample: {name} must be float32 [{rows}]")
    lib = _lib.load("core")
    scratch = torch.empty((lib.mk_sample_scratch_bytes(rows, int(top_ps is not None)),),
                          dtype=torch.uint8, device=logits.device)
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    _lib.check(lib, lib.mk_sample(_ptr(logits), rows, vocab, vocab, _ptr(temperatures),
                                  _ptr(top_ps), _ptr(uniforms), _ptr(scratch), _ptr(out),
                                  _stream()), "sample")
    return out

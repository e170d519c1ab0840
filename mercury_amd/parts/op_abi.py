"""The C interface of a program's operations (``csrc/host/op_abi.h``) as ctypes structures, and
a way to register an operation kind whose run function is written in Python.

An operation kind is a C function; the host core calls it once per step with the operation's
parameter block and the step's context.  A kind written in C or C++ is registered with
``hostcore.core.register_op(name, address_of_run, address_of_tiles, flags)``.  For parts
defined in Python, `register_python_op` wraps a Python function into such a C function: it
runs on the host when the step's kernels are launched (under a graph capture: once, at
capture) and launches kernels itself, through the kernel libraries' C entry points or any
other way that puts work on `ctx.stream`.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char, c_float, c_int, c_size_t, c_void_p

from ..hostcore import core


class TileList(ctypes.Structure):
    _fields_ = [("group", c_int), ("tile_rows", c_int), ("count", c_int),
                ("seq", c_void_p), ("row0", c_void_p)]


class StepView(ctypes.Structure):
    _fields_ = [("num_tokens", c_int), ("num_seqs", c_int), ("num_rows", c_int),
                ("max_q_len", c_int), ("max_kv_len", c_int),
                ("token_ids", c_void_p), ("positions", c_void_p), ("token_seq", c_void_p),
                ("cu_q", c_void_p), ("kv_len", c_void_p), ("state_slots", c_void_p),
                ("logit_rows", c_void_p),
                ("num_groups", c_int), ("tables", POINTER(c_void_p)), ("widths", POINTER(c_int)),
                ("counts", POINTER(c_int)),
                ("num_tile_lists", c_int), ("tile_lists", POINTER(TileList))]


ALLOC = ctypes.CFUNCTYPE(c_void_p, c_void_p, c_size_t)


class OpContext(ctypes.Structure):
    _fields_ = [("step", POINTER(StepView)), ("stream", c_void_p), ("dry", c_int),
                ("dtype", c_int), ("hidden", c_int), ("vocab", c_int),
                ("h", c_void_p), ("x", c_void_p), ("x_rows", c_int), ("x_live", c_int),
                ("pending", c_void_p), ("pending_count", c_int), ("logits", c_void_p),
                ("out_x", c_void_p), ("out_x_rows", c_int), ("out_x_live", c_int),
                ("out_pending", c_void_p), ("out_pending_count", c_int),
                ("out_logits_ready", c_int),
                ("arena", c_void_p), ("alloc", ALLOC), ("error", c_char * 512),
                # a step of few tokens with its residual stream in fixed point (h is then
                # null), which only kinds flagged FIXED_STREAM ever see
                ("stream_fixed", c_int), ("h_fixed", c_void_p),
                ("norm_weight", c_void_p), ("norm_weight_dtype", c_int), ("norm_eps", c_float),
                ("out_norm_weight", c_void_p), ("out_norm_weight_dtype", c_int),
                ("out_norm_eps", c_float)]

    def allocate(self, nbytes: int) -> int:
        """Device memory from the operation's arena (0 in a dry walk)."""
        return self.alloc(self.arena, nbytes) or 0


RUN = ctypes.CFUNCTYPE(c_int, c_void_p, POINTER(OpContext))

READS_X = core.OP_READS_X
FOLDS_PENDING = core.OP_FOLDS_PENDING
FIXED_STREAM = core.OP_FIXED_STREAM

_kept: dict = {}      # name -> the C function object; the registry holds its bare address


def register_python_op(name: str, run, flags: int = 0) -> None:
    """Register the operation kind `name` whose work `run(params_address, ctx)` does:
    `params_address` is where the operation's parameter block lies (read it with a ctypes
    structure's ``from_address``), `ctx` an :class:`OpContext`.  An exception becomes the
    step's error."""

    def entry(params, ctx_pointer):
        ctx = ctx_pointer.contents
        try:
            run(params, ctx)
            return 0
        except Exception as error:      # the C side turns the message into its own error
            ctx.error = f"{type(error).__name__}: {error}".encode()[:500]
            return 1

    function = RUN(entry)
    _kept[name] = function
    core.register_op(name, ctypes.cast(function, c_void_p).value, 0, flags)


__all__ = ["ALLOC", "FIXED_STREAM", "FOLDS_PENDING", "OpContext", "READS_X", "RUN", "StepView", "TileList",
           "c_float", "register_python_op"]

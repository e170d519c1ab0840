"""Running a part's own operations on tensors.

A part that hands its work to the host core says what it does once, in `lower`: the
operations it appends to a step program.  When such a part has to run by itself (inside a
layer that stays with Python, or alone in a test) it runs those same operations, as a
program of its own over the tensors it is given, instead of a second copy of the launch
sequence written in Python.
"""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops


class _BareStep:
    """A step of one sequence of `tokens` tokens with no index arrays behind it: enough for
    operations that work row by row and read none (a feed-forward, a norm)."""

    def __init__(self, tokens: int):
        self.spans = [(0, tokens, 0)]
        self.num_logit_rows = 0
        self.max_q_len = self.max_kv_len = tokens
        self.block_tables: list = []

    def as_view(self, program=None) -> dict:
        tokens = self.spans[0][1]
        return {"counts": [tokens], "num_rows": 0, "max_q_len": tokens, "max_kv_len": tokens,
                "tables": [], "tiles": []}


class OneOp:
    """The operations `lower_into(program)` appends, as a program of their own."""

    def __init__(self, dtype: torch.dtype, hidden: int, vocab: int, lower_into):
        self.dtype = dtype
        self.hidden, self.vocab = int(hidden), int(vocab)
        self.program = core.Program(ops.dtype_code(dtype), self.hidden, self.vocab)
        lower_into(self.program)
        if "host" in self.program.kinds:
            raise ValueError("a part's own program cannot hold steps the caller runs")

    def run(self, step, h: torch.Tensor, x: torch.Tensor | None = None,
            pending: torch.Tensor | None = None, want_logits: bool = False):
        """Run on the residual stream `h` (float32 [T, H], updated in place), with `x` as the
        previous operation's output and `pending` as its partial sums.  Returns
        (logits or None, x or None, pending or None); the tensors are views of scratch memory
        that lives as long as they do."""
        if h.dtype != torch.float32 or h.dim() != 2 or h.shape[1] != self.hidden or not h.is_cuda:
            raise ops.KernelArgumentError("a part runs on a float32 residual stream [T, H] on the GPU")
        ops._ensure(torch.empty((), dtype=self.dtype))
        program = self.program
        if step is None:
            step = _BareStep(h.shape[0])
        counts = [count for _first, count, _start in step.spans]
        rows = step.num_logit_rows
        x_rows = 0 if x is None else x.shape[0]
        need = program.workspace_bytes_for(counts, rows, step.max_kv_len,
                                           max(1, len(step.block_tables)), x_rows, own_stream=True)
        scratch = torch.empty(max(need, 256), dtype=torch.uint8, device=h.device)
        logits = None
        if want_logits:
            logits = torch.empty((rows, self.vocab), dtype=torch.float32, device=h.device)
        stream = torch.cuda.current_stream(h.device).cuda_stream
        logits_at, x_at, x_out_rows, pending_at, pending_count = program.run_on(
            step.as_view(program), scratch.data_ptr(), scratch.numel(), stream, h.data_ptr(),
            0 if logits is None else logits.data_ptr(), 0 if x is None else x.data_ptr(), x_rows,
            0 if pending is None else pending.data_ptr(),
            0 if pending is None else pending.shape[0])

        def view(address, shape, dtype):
            count = 1
            for n in shape:
                count *= n
            offset = address - scratch.data_ptr()
            size = count * torch.empty((), dtype=dtype).element_size()
            if offset < 0 or offset + size > scratch.numel():
                raise RuntimeError("an operation's result lies outside its workspace")
            return scratch[offset:offset + size].view(dtype).view(*shape)

        x_out = view(x_at, (x_out_rows, self.hidden), self.dtype) if x_at else None
        pending_out = (view(pending_at, (pending_count, h.shape[0], self.hidden), torch.float32)
                       if pending_count else None)
        return (logits if logits_at else None), x_out, pending_out

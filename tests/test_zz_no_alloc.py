"""The argmax entry point that allocates nothing (its partial results live in a device array
of the library's own) against the one that takes the caller's buffer, through ctypes: two
calls in a row, the second with a smaller input."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_argmax_without_allocation_equals_argmax_with_a_buffer():
    from mercury_amd.kernels import build

    lib = ctypes.CDLL(str(build.build_library("core", force=False)))
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
    lib.mk_argmax.argtypes = [P, I, I, L, P, P, P]
    lib.mk_argmax_static.argtypes = [P, I, I, L, P, P]
    lib.mk_last_error.restype = ctypes.c_char_p
    limit = lib.mk_argmax_static_max_rows()
    assert limit >= 64

    device = torch.device("cuda:0")
    stream = torch.cuda.current_stream(device).cuda_stream
    # the address of the library's array, resolved before any call that might be captured
    assert lib.mk_argmax_static_init() == 0, lib.mk_last_error()
    # the first case fills the array to its stated limit (the last row's parts lie in its last
    # slots); the following, smaller ones run over what it left there
    for rows, vocab, seed in ((limit, 16_384, 4), (64, 151_936, 1), (5, 20_011, 2), (3, 1_003, 3)):
        g = torch.Generator().manual_seed(seed)
        logits = torch.randn(rows, vocab, generator=g).to(device)
        logits[0, vocab - 1] = 50.0                     # the very last place
        logits[rows - 1, :2] = 60.0                     # a tie: the lowest index wins
        want = torch.empty(rows, dtype=torch.int32, device=device)
        got = torch.full((rows,), -1, dtype=torch.int32, device=device)
        parts = torch.empty(rows * 64 * 8, dtype=torch.uint8, device=device)
        code = lib.mk_argmax(logits.data_ptr(), rows, vocab, vocab, want.data_ptr(),
                             parts.data_ptr(), stream)
        assert code == 0, lib.mk_last_error()
        code = lib.mk_argmax_static(logits.data_ptr(), rows, vocab, vocab, got.data_ptr(), stream)
        assert code == 0, lib.mk_last_error()
        torch.cuda.synchronize(device)
        assert torch.equal(got, want), (rows, vocab)
        assert torch.equal(got.cpu().long(), logits.argmax(-1).cpu())
        assert int(got[0]) == vocab - 1 and int(got[rows - 1]) == 0

    # beyond the stated maximum: refused, with a message, and nothing launched
    logits = torch.zeros(limit + 1, 16_384, device=device)
    out = torch.empty(limit + 1, dtype=torch.int32, device=device)
    code = lib.mk_argmax_static(logits.data_ptr(), limit + 1, 16_384, 16_384, out.data_ptr(), stream)
    assert code != 0 and b"at most" in lib.mk_last_error()

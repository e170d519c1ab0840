"""The host core's step programs without a GPU: operation kinds registered from outside, dry
walks that size a workspace and refuse operations that do not fit together, the parameter
blocks of the built-in kinds."""

from __future__ import annotations

import ctypes

import pytest

from mercury_amd.hostcore import core
from mercury_amd.parts import op_abi

F32 = 0


class Sizes(ctypes.Structure):
    _fields_ = [("bytes_out", ctypes.c_int), ("gives_x", ctypes.c_int), ("gives_pending", ctypes.c_int)]


def allocating(params, ctx):
    """A kind that allocates what its parameters say and hands on what they say."""
    p = Sizes.from_address(params)
    at = ctx.allocate(p.bytes_out)
    assert ctx.dry and at == 0          # these tests only walk dry
    if p.gives_x:
        ctx.out_x, ctx.out_x_rows, ctx.out_x_live = at, ctx.step.contents.num_tokens, 1
    if p.gives_pending:
        ctx.out_pending, ctx.out_pending_count = at, p.gives_pending


op_abi.register_python_op("test_producer", allocating)
op_abi.register_python_op("test_reader", allocating, op_abi.READS_X)
op_abi.register_python_op("test_folder", allocating, op_abi.FOLDS_PENDING)


def op(bytes_out=0, gives_x=0, gives_pending=0) -> bytes:
    return bytes(Sizes(bytes_out, gives_x, gives_pending))


def test_ctypes_mirror_matches_the_header():
    layout = core.op_abi_layout()
    assert ctypes.sizeof(op_abi.OpContext) == layout["context_size"]
    assert ctypes.sizeof(op_abi.StepView) == layout["step_size"]
    assert ctypes.sizeof(op_abi.TileList) == layout["tile_list_size"]
    assert op_abi.OpContext.error.offset == layout["context_error_offset"]
    assert op_abi.OpContext.alloc.offset == layout["context_alloc_offset"]
    assert op_abi.OpContext.out_x.offset == layout["context_out_x_offset"]
    assert op_abi.StepView.tables.offset == layout["step_tables_offset"]


def test_kinds_from_outside_are_listed_and_unknown_ones_refused():
    assert {"embed", "norm", "attention", "gated_mlp", "head", "test_producer"} <= set(core.op_kinds())
    program = core.Program(F32, 64, 100)
    with pytest.raises(RuntimeError, match="no operation kind 'nonesuch'.*known:.*norm"):
        program.append("nonesuch", b"")
    with pytest.raises(RuntimeError, match="name of its own"):
        core.register_op("host", 1)


def test_dry_walk_sizes_two_alternating_arenas():
    program = core.Program(F32, 64, 100)
    program.append("test_producer", op(1000, gives_x=1))      # arena 0: 1024 (256-byte units)
    program.append("test_reader", op(5000, gives_x=1))        # arena 1: 5120
    program.append("test_reader", op(300))                    # arena 0 again: 512
    assert program.kinds == ["test_producer", "test_reader", "test_reader"]
    tokens, rows = 7, 2
    persistent = (tokens * 64 * 4 + 255) // 256 * 256 + (rows * 100 * 4 + 255) // 256 * 256
    assert program.workspace_bytes_for([4, 3], rows, 50) == persistent + 2 * 5120


def test_an_operation_that_reads_x_needs_it_from_the_one_before():
    program = core.Program(F32, 64, 100)
    program.append("test_producer", op(256, gives_x=1))
    program.append("test_reader", op(256))
    program.append("test_reader", op(256))        # the first reader left no x
    with pytest.raises(RuntimeError, match=r"operation 2 \('test_reader'\) reads x"):
        program.workspace_bytes_for([3], 1, 3)
    lonely = core.Program(F32, 64, 100)
    lonely.append("test_reader", op(256))
    with pytest.raises(RuntimeError, match=r"operation 0 .* reads x"):
        lonely.workspace_bytes_for([3], 1, 3)
    # an x of the caller's for the first operation is another matter
    assert lonely.workspace_bytes_for([3], 1, 3, x_rows=3) > 0


def test_partial_sums_must_be_added_up_by_the_next_operation():
    program = core.Program(F32, 64, 100)
    program.append("test_producer", op(256, gives_pending=3))
    program.append("test_producer", op(256))
    with pytest.raises(RuntimeError, match=r"operation 1 .* does not add them up"):
        program.workspace_bytes_for([3], 1, 3)
    fine = core.Program(F32, 64, 100)
    fine.append("test_producer", op(256, gives_pending=3))
    fine.append("test_folder", op(256, gives_x=1))
    fine.append("test_reader", op(256))
    assert fine.workspace_bytes_for([3], 1, 3) > 0


def test_caller_steps_cut_the_walk_and_say_what_they_leave():
    program = core.Program(F32, 64, 100)
    program.append("test_producer", op(256))
    program.host(0, gives_x=True)
    program.append("test_reader", op(256))
    program.host(1)
    program.append("test_reader", op(256))            # nothing gives this one its x
    assert program.kinds == ["test_producer", "host", "test_reader", "host", "test_reader"]
    assert [program.host_index(i) for i in (1, 3)] == [0, 1]
    with pytest.raises(RuntimeError, match=r"operation 4 .* reads x"):
        program.workspace_bytes_for([3], 1, 3)


def test_built_in_operations_in_the_wrong_order_fail_at_build_time():
    """The built-in kinds under the same rules: an attention without a norm before it, a
    feed-forward behind an attention without a norm in between."""
    attention = core.attention_params(
        w_qkv=1, w_o=1, n_q=4, n_kv=2, head_dim=16, rotary_dim=0, k_cache=1, v_cache=1, group=0,
        page_size=16, scale=0.25, window=0, writes=True)
    norm = core.norm_params(1, F32, 1e-6)
    mlp = core.gated_mlp_params(1, 1, 176)
    embed = core.embed_params(1, F32, 512)
    good = core.Program(F32, 64, 512)
    for kind, params in (("embed", embed), ("norm", norm), ("attention", attention), ("norm", norm),
                         ("gated_mlp", mlp), ("norm", core.norm_params(1, F32, 1e-6, True)),
                         ("head", core.head_params(1))):
        good.append(kind, params)
    assert good.workspace_bytes_for([5, 1], 2, 40) > 0
    headless = core.Program(F32, 64, 512)
    for kind, params in (("embed", embed), ("attention", attention)):
        headless.append(kind, params)
    with pytest.raises(RuntimeError, match=r"operation 1 \('attention'\) reads x"):
        headless.workspace_bytes_for([5, 1], 2, 40)
    stale = core.Program(F32, 64, 512)
    for kind, params in (("embed", embed), ("norm", norm), ("attention", attention), ("gated_mlp", mlp)):
        stale.append(kind, params)
    with pytest.raises(RuntimeError, match=r"operation 3 \('gated_mlp'\)"):
        stale.workspace_bytes_for([5, 1], 2, 40)
    with pytest.raises(RuntimeError, match="head counts"):
        core.attention_params(w_qkv=1, w_o=1, n_q=5, n_kv=2, head_dim=16)


def test_an_error_inside_an_operation_names_it():
    def failing(params, ctx):
        raise ValueError("made to fail")

    op_abi.register_python_op("test_failing", failing)
    program = core.Program(F32, 64, 100)
    program.append("test_producer", op(256))
    program.append("test_failing", b"")
    with pytest.raises(RuntimeError, match=r"operation 1 \('test_failing'\): ValueError: made to fail"):
        program.workspace_bytes_for([3], 1, 3)


# ---- steps of few tokens with the residual stream in fixed point

SEEN: list = []


def watching(params, ctx):
    """A kind that records what the walk tells it about the stream, and may leave a norm to
    the operation behind it."""
    p = Sizes.from_address(params)
    SEEN.append((ctx.stream_fixed, bool(ctx.x_live), ctx.norm_weight or 0, round(ctx.norm_eps, 6)))
    at = ctx.allocate(p.bytes_out)
    if p.gives_x:
        ctx.out_x_rows, ctx.out_x_live = ctx.step.contents.num_tokens, 1
        if ctx.stream_fixed or p.gives_x == 2:   # a norm left undone: no x, but its weight and eps
            ctx.out_norm_weight, ctx.out_norm_weight_dtype, ctx.out_norm_eps = 4096, 1, 0.125
        else:
            ctx.out_x = at


op_abi.register_python_op("test_fixed_any", watching, op_abi.FIXED_STREAM)
op_abi.register_python_op("test_fixed_reader", watching, op_abi.READS_X | op_abi.FIXED_STREAM)


@pytest.fixture
def fixed_up_to_four():
    before = core.set_fixed_stream_limit(4)
    yield
    core.set_fixed_stream_limit(before)


def test_few_tokens_walk_in_fixed_point_when_every_operation_can(fixed_up_to_four):
    program = core.Program(F32, 64, 100)
    program.append("test_fixed_any", op(256, gives_x=1))
    program.append("test_fixed_reader", op(256))
    assert program.fixed_stream(4) and not program.fixed_stream(5) and not program.fixed_stream(0)
    rows = 1
    logits = (rows * 100 * 4 + 255) // 256 * 256
    # 8 bytes a value of the stream instead of 4
    assert program.workspace_bytes_for([3], rows, 9) == 3 * 64 * 8 + logits + 2 * 256
    assert program.workspace_bytes_for([5], rows, 9) == 5 * 64 * 4 + logits + 2 * 256
    # a run on a stream of the caller's own is never in fixed point
    assert program.workspace_bytes_for([3], rows, 9, own_stream=True) == 2 * 256
    SEEN.clear()
    program.workspace_bytes_for([3], rows, 9)
    assert SEEN == [(1, False, 0, 0.0), (1, True, 4096, 0.125)]     # the norm reaches the reader
    mixed = core.Program(F32, 64, 100)
    mixed.append("test_fixed_any", op(256))
    mixed.append("test_producer", op(256))
    assert not mixed.fixed_stream(2)              # one operation that cannot: the float stream
    SEEN.clear()
    mixed.workspace_bytes_for([2], rows, 9)
    assert SEEN == [(0, False, 0, 0.0)]


def test_a_norm_left_undone_outside_fixed_point_is_refused(fixed_up_to_four):
    program = core.Program(F32, 64, 100)
    program.append("test_fixed_any", op(256, gives_x=2))      # leaves it whatever the stream is
    program.append("test_fixed_reader", op(256))
    assert program.workspace_bytes_for([3], 1, 9) > 0
    with pytest.raises(RuntimeError, match="left a norm undone outside a step in fixed point"):
        program.workspace_bytes_for([7], 1, 9)


def test_the_limit_switches_fixed_point_off():
    before = core.set_fixed_stream_limit(0)
    try:
        program = core.Program(1, 64, 100)
        program.append("test_fixed_any", op(256))
        assert not program.fixed_stream(1)
    finally:
        core.set_fixed_stream_limit(before)
    # the kernels' own rule again: float32 models never
    program = core.Program(F32, 64, 100)
    program.append("test_fixed_any", op(256))
    assert not program.fixed_stream(1)

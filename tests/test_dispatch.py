"""Which attention kernel the host core picks for a step's shape (csrc/host/dispatch.cc): the
choices behind the benchmark's numbers, each with the measurement that set its threshold.
The planner runs on the host; it only asks the kernel library what it has."""

import pytest

BF16 = 1


@pytest.fixture(scope="module")
def core():
    try:
        from mercury_amd import hostcore
        from mercury_amd.kernels import lib

        lib.load("core")
        lib.load("mfma")
    except Exception as error:   # no compiler and no built library here
        pytest.skip(f"the kernel libraries are not available: {error}")
    return hostcore.core


def plan(core, heads, kv_heads, size, counts, context, window=0, page=16):
    return core.plan_attention(BF16, size, page, heads, kv_heads, window, counts, max(counts), context)


def test_decoding_splits_the_keys_in_fours(core):
    """Few tiles: every tile's keys in as many parts as fill the chip with wavefronts, in
    fours, which one workgroup's wavefronts add up before writing (8 sequences at 4,096, 14
    heads of 64: 9.0 us with 64 parts against 11.5 with 63)."""
    p = plan(core, 14, 2, 64, [1] * 8, 4096)
    assert (p["staged"], p["rows"], p["splits"]) == (0, 16, 64)
    p = plan(core, 14, 2, 64, [1], 4096)
    assert p["splits"] == 64 and p["num_tiles"] == 1      # no more parts than pairs of key blocks
    p = plan(core, 28, 4, 128, [1] * 8, 4096)
    assert p["splits"] == 32
    p = plan(core, 14, 2, 64, [1] * 64, 4096)
    assert p["splits"] == 8
    # many sequences fill the chip by themselves
    assert plan(core, 40, 8, 128, [1] * 128, 4096)["splits"] == 1
    # a short context has few blocks to hand out
    assert plan(core, 14, 2, 64, [1] * 8, 100)["splits"] <= 2


def test_prompts_go_through_lds(core):
    """A 2,048-token prompt of 14 heads of 64 is 224 workgroups of 128 rows, fewer than compute
    units: the 16-row kernel with the keys in four chains (30 us against 40 in the 32-row
    kernel, a tie with its three chains)."""
    p = plan(core, 14, 2, 64, [2048], 2048)
    assert (p["staged"], p["rows"], p["tile_rows"], p["num_tiles"]) == (4, 16, 64, 224)   # x 2 kv heads
    # 28 heads of 64: 448 workgroups, chains too short to cut: the 32-row kernel (44 us against 47)
    assert plan(core, 28, 4, 64, [2048], 2048)["staged"] == 8
    # 128-wide heads from 256 workgroups (28 heads, 2,048 tokens: 79 us against 96)
    p = plan(core, 28, 4, 128, [2048], 2048)
    assert (p["staged"], p["rows"], p["tile_rows"]) == (8, 32, 128)


def test_long_prompts_take_32_row_wavefronts(core):
    """8,192 tokens: 0.55-0.80 PFLOP/s in the 32-row kernel against 0.42-0.54 in the 16-row
    one, at every head shape."""
    for heads, kv_heads, size in ((14, 2, 64), (28, 4, 64), (28, 4, 128), (40, 8, 128)):
        p = plan(core, heads, kv_heads, size, [8192], 8192)
        assert (p["staged"], p["rows"]) == (8, 32)
    assert plan(core, 14, 2, 64, [2048] * 4, 2048)["staged"] == 8      # 73 us against 90


def test_chunks_over_long_prefixes_cut_the_keys_into_chains(core):
    """Fewer workgroups than fill the chip, each with a long chain of key blocks: 64-wide heads
    in three chains (2,048 tokens over 30,720: 347 us against 500 in the 16-row kernel; 4,096
    tokens: 63 against 92), 128-wide in two (1,024 over 3,072, 28 heads: 92 against 133)."""
    assert plan(core, 14, 2, 64, [2048], 2048 + 30720)["staged"] == 24
    assert plan(core, 14, 2, 64, [4096], 4096)["staged"] == 24
    assert plan(core, 28, 4, 128, [1024], 4096)["staged"] == 16
    # too few workgroups for either: the 16-row kernel, more of them (512 over 7,680: 71 against 93)
    assert plan(core, 14, 2, 64, [512], 8192)["staged"] in (1, 2, 4)


def test_head_sizes_the_32_row_kernel_does_not_take(core):
    p = plan(core, 8, 2, 96, [8192], 8192)
    assert p["mfma"] and p["staged"] == 0 and p["rows"] in (16, 32)
    p = plan(core, 8, 2, 256, [8192], 8192)
    assert p["mfma"] and p["staged"] == 0 and p["rows"] == 16
    assert not plan(core, 8, 2, 48, [64], 64)["mfma"]        # no matrix-core kernel of that size


def test_mixed_steps_use_the_prompt_kernel_when_a_portion_is_long(core):
    """A portion of 512 tokens beside 63 decoded ones: the prompt kernel for all of them."""
    p = plan(core, 14, 2, 64, [512] + [1] * 63, 4096)
    assert p["staged"] in (1, 2, 4) and p["splits"] == 1


def test_the_qkv_projection_is_one_kernel_where_that_is_faster(core):
    """Projection, bias, rotation and cache write in one kernel: the skinny one for few rows of
    a small matrix (1152 x 896 at 8 rows: 6.0 us against 10.6 as partial sums and a finishing
    kernel), the tiled one for many rows.  A matrix of 24 MB or more at up to 256 rows goes as
    K-split partial sums and a finishing kernel (4608 x 3584 at 8..64 rows: 14.0..16.5 us
    against 15.2..30.7 in the one skinny kernel)."""
    skinny, tiled, partials, unfused = 0, 1, 2, 3
    for rows, want in ((1, skinny), (8, skinny), (16, skinny), (64, tiled), (2048, tiled)):
        assert core.choose_qkv(BF16, BF16, rows, 1152, 896, 64, 64, 16, True) == want
    for rows, want in ((1, partials), (8, partials), (64, partials), (256, partials), (2048, tiled)):
        assert core.choose_qkv(BF16, BF16, rows, 4608, 3584, 128, 128, 16, True) == want
        assert core.choose_qkv(BF16, BF16, rows, 7168, 5120, 128, 128, 16, True) == want
    # what the fused kernels do not take: heads that are no multiple of 32 wide, a rotation
    # over part of the head, interleaved pairs
    assert core.choose_qkv(BF16, BF16, 8, 18 * 48, 168, 48, 48, 16, True) in (partials, unfused)
    assert core.choose_qkv(BF16, BF16, 8, 1152, 896, 64, 32, 16, True) == unfused
    assert core.choose_qkv(BF16, BF16, 8, 1152, 896, 64, 64, 16, False) == unfused


def test_projections_into_the_residual_stream(core):
    """Few rows: K in slices with partial sums where the matrix is large enough for bandwidth
    to matter (the 0.5B down projection, 8.7 MB, at 8 rows: 5.2 us in 8 slices against 9.5
    whole), all of K in one workgroup where latency is the cost (the 0.5B o projection, 1.6 MB);
    the skinny kernel up to 16 rows of a matrix under 20 MB, tiles beyond."""
    by_skinny, slices = core.plan_partials(8, 896, 4864)
    assert by_skinny and slices == 8
    by_skinny, slices = core.plan_partials(8, 3584, 18944)
    assert not by_skinny and slices >= 2          # 136 MB: tiles stream it faster
    by_skinny, slices = core.plan_partials(64, 3584, 18944)
    assert not by_skinny and slices >= 2
    generic, skinny, skinny_acc, tiled = 0, 1, 2, 3
    F32 = 0
    assert core.choose_linear(BF16, 8, 896, 896, False, True, F32, 0) == skinny_acc
    assert core.choose_linear(BF16, 2048, 896, 896, False, True, F32, 0) == tiled
    assert core.choose_linear(BF16, 1, 151936, 896, False, False, F32, 0) == skinny      # the head
    assert core.choose_linear(BF16, 8, 151936, 896, False, False, F32, 0) == tiled
    assert core.choose_linear(BF16, 8, 896, 900, False, True, F32, 0) == generic         # K % 8
    assert core.choose_linear(F32, 8, 896, 896, False, True, F32, 0) == generic

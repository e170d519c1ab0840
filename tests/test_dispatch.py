"""Which kernel the host core picks for a step's shape (csrc/ops/dispatch.cc).

Most of this file does not pin the planner's present choices (those move whenever a
threshold is measured again) but what must hold of every choice: the matrix-core attention
accepts every plan the planner can emit (checked with the kernel entry point's own argument
checks, without a launch), the tile lists have the length the plan says, key splits never
leave a part without blocks, and a fused q/k/v kernel is only ever chosen for operands it
takes.  A handful of choices behind the benchmark's numbers stay pinned at the end.
The planner runs on the host; it only asks the kernel library what it has."""

import random

import pytest

F32, BF16 = 0, 1
HEAD_SIZES = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256)


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


def random_step(rng):
    """(head size, page, heads, kv heads, window, tokens per sequence, longest length)."""
    size = rng.choice(HEAD_SIZES)
    page = rng.choice((8, 16, 32, 64, 128))
    kv_heads = rng.choice((1, 2, 3, 4, 8))
    heads = kv_heads * rng.choice((1, 2, 3, 4, 7, 8, 16))
    window = rng.choice((0, 0, 0, 24, 1000, 5000))
    kind = rng.random()
    if kind < 0.35:          # decoding
        counts = [1] * rng.choice((1, 2, 7, 8, 33, 64, 200, 256))
    elif kind < 0.6:         # one prompt, short to very long
        counts = [rng.choice((2, 17, 64, 100, 200, 300, 512, 2048, 4700, 8192, 30000))]
    else:                    # portions beside decoded tokens
        counts = [rng.choice((1, 1, 1, 2, 16, 100, 512, 2048)) for _ in range(rng.randint(1, 40))]
    longest = max(counts) + rng.choice((0, 0, 5, 300, 4000, 30000))
    return size, page, heads, kv_heads, window, counts, longest


def test_every_plan_is_one_the_kernel_accepts(core):
    rng = random.Random(11)
    seen = {"generic": 0, "split": 0, "staged": 0, "wide": 0, "plain": 0}
    for _ in range(3000):
        size, page, heads, kv_heads, window, counts, longest = random_step(rng)
        p = core.plan_attention(BF16, size, page, heads, kv_heads, window, counts, max(counts), longest)
        case = (size, page, heads, kv_heads, window, counts[:4], len(counts), longest, p)
        if not p["mfma"]:
            seen["generic"] += 1
            continue
        # the entry point's own checks, without the launch
        assert core.validate_attention_plan(p, size, page, heads, kv_heads) == "", case
        group = heads // kv_heads
        # the tile list the packer lays out is the one the plan counted
        assert core.count_tiles(counts, group, p["tile_rows"]) == p["num_tiles"], case
        seq, row0 = core.build_tiles(counts, group, p["tile_rows"])
        assert len(seq) == len(row0) == p["num_tiles"], case
        assert all(0 <= s < len(counts) for s in seq), case
        assert all(r % p["tile_rows"] == 0 and r < counts[s] * group for s, r in zip(seq, row0)), case
        half = p["staged"] >= 8 and p["staged"] % 8 == 4      # the 32-row kernel on tiles of 64 rows
        assert p["tile_rows"] == p["rows"] * (2 if half else 4 if p["staged"] else 1), case
        # key splits: only without staging, never more parts than pairs of 32-key blocks of
        # the longest span, in fours from four on
        span = min(longest, window + max(counts)) if window else longest
        blocks = max(1, -(-span // 32))
        assert 1 <= p["splits"] <= max(1, blocks // 2) or p["splits"] == 1, case
        if p["splits"] > 1:
            assert p["staged"] == 0 and (p["splits"] < 4 or p["splits"] % 4 == 0), case
        # without a tile list: only where every sequence brings one token whose heads are one
        # tile of 16 rows, unwindowed, the keys' parts every n-th block
        if p["direct"]:
            assert set(counts) == {1} and group <= 16 and not window and not p["staged"], case
            assert p["rows"] == 16 and p["split_blocks"] == 0 and p["num_tiles"] == len(counts), case
        elif set(counts) == {1} and group <= 16 and not window:
            assert False, case      # a decode step that misses the direct kernel
        # the kernel of 32-row wavefronts: only where a sequence has at least 128 rows
        if p["staged"] >= 8:
            assert max(counts) * group >= (64 if half else 128) and p["rows"] == 32, case
        seen["wide" if p["staged"] >= 8 else "staged" if p["staged"] else
             "split" if p["splits"] > 1 else "plain"] += 1
    # the generator reaches every kind of plan
    assert all(n >= 30 for n in seen.values()), seen


def test_float32_and_unsupported_sizes_take_the_float32_kernel(core):
    for size in HEAD_SIZES:
        assert not core.plan_attention(F32, size, 16, 8, 2, 0, [64], 64, 64)["mfma"]
    assert not plan(core, 8, 2, 48, [64], 64)["mfma"]
    assert not plan(core, 8, 2, 64, [64], 64, page=8)["mfma"]
    with pytest.raises(RuntimeError, match="bfloat16 only"):
        core.plan_attention(F32, 64, 16, 8, 2, 0, [64], 64, 64, force=2)


def test_qkv_choices_are_ones_the_kernels_take(core):
    rng = random.Random(5)
    skinny, tiled, partials, unfused = 0, 1, 2, 3
    counts = {skinny: 0, tiled: 0, partials: 0, unfused: 0}
    for _ in range(3000):
        size = rng.choice(HEAD_SIZES)
        kv = rng.choice((1, 2, 4, 8))
        heads = kv * rng.choice((1, 2, 4, 7))
        width = (heads + 2 * kv) * size
        k = rng.choice((64, 168, 896, 900, 1024, 3584, 5120))
        rows = rng.choice((1, 2, 8, 16, 17, 64, 65, 256, 257, 2048))
        rotary = rng.choice((0, size, size // 2))
        half = rng.random() < 0.8
        page = rng.choice((8, 16, 64))
        dtype = BF16 if rng.random() < 0.85 else F32
        kind = core.choose_qkv(dtype, dtype, rows, width, k, size, rotary, page, half)
        counts[kind] += 1
        fusable = core.qkv_fusable(dtype, dtype, rows, k, size, rotary, page, half)
        case = (dtype, rows, width, k, size, rotary, page, half, kind)
        if kind in (skinny, tiled):
            assert fusable and dtype == BF16 and k % 8 == 0 and size % 32 == 0, case
            assert rotary in (0, size) and (half or rotary == 0), case
        if kind == skinny:
            assert rows <= 64, case
        if kind == partials:
            # the finishing kernel rotates in the half-split layout only, and partial sums
            # come from the matrix-core kernels
            assert (half or rotary == 0) and core.wants_partials(dtype, dtype, rows, width, k), case
        if dtype == F32 or k % 8:
            assert kind == unfused, case
    assert all(n >= 30 for n in counts.values()), counts


def test_projection_choices_are_ones_the_kernels_take(core):
    rng = random.Random(7)
    generic, skinny, skinny_acc, tiled = 0, 1, 2, 3
    for _ in range(2000):
        m = rng.choice((1, 7, 8, 16, 17, 64, 65, 512))
        n = rng.choice((896, 1000, 4864, 151936))
        k = rng.choice((64, 896, 900, 4864))
        bias, accumulate = rng.random() < 0.3, rng.random() < 0.5
        dtype = BF16 if rng.random() < 0.8 else F32
        out = F32 if accumulate or rng.random() < 0.5 else dtype
        kind = core.choose_linear(dtype, m, n, k, bias, accumulate, out, 0)
        case = (dtype, m, n, k, bias, accumulate, out, kind)
        if dtype == F32 or k % 8:
            assert kind == generic, case
            assert not core.wants_partials(dtype, dtype, m, n, k), case
            continue
        assert kind != generic, case
        if kind == skinny:          # float32 out, no bias, not accumulating: what it computes
            assert out == F32 and not bias and not accumulate and m < 8, case
        if kind == skinny_acc:
            assert accumulate and m <= 64, case
        if core.wants_partials(dtype, dtype, m, n, k):
            by_skinny, slices = core.plan_partials(m, n, k)
            assert slices >= 1 and (not by_skinny or m <= 16), case   # one slice: a whole product left as float32 for the next norm


# ---- pinned: the choices behind the benchmark's numbers, each with its measurement


def test_pinned_choices_of_the_benchmark_shapes(core):
    # 0.5B decoding, 8 sequences at 4,096: the keys in 64 parts, in fours that one workgroup's
    # wavefronts add up before writing (9.0 us against 11.5 with 63)
    p = plan(core, 14, 2, 64, [1] * 8, 4096)
    assert (p["staged"], p["rows"], p["splits"]) == (0, 16, 64)
    # many sequences fill the chip by themselves
    assert plan(core, 40, 8, 128, [1] * 128, 4096)["splits"] == 1
    # 8,192-token prompts: the kernel of 32-row wavefronts at every head shape (0.55-0.80
    # PFLOP/s against 0.42-0.54)
    for heads, kv_heads, size in ((14, 2, 64), (28, 4, 128), (40, 8, 128)):
        p = plan(core, heads, kv_heads, size, [8192], 8192)
        assert (p["staged"], p["rows"]) == (8, 32)
    # shorter prompts: the same kernel with the keys in several chains, or on tiles of 64 rows
    # where 128-row workgroups would be too few (0.5B, 2,048 tokens: four chains on 64-row
    # tiles, 28.0 us against 29.5 in the 16-row kernel; 512 tokens over 3,584: 36.4 against
    # 40.7; 1,024 tokens of 28 heads in 4 groups: two chains, 19.0 against 23.8; 3,072 tokens
    # of 14 heads: three chains on 128-row tiles, 39.7 against 55.9), and two chains for
    # 128-wide heads (7B, 2,048 tokens: 58.3 against 67.9 in one)
    assert plan(core, 14, 2, 64, [2048], 2048)["staged"] == 36
    p = plan(core, 14, 2, 64, [512], 4096)
    assert (p["staged"], p["rows"], p["tile_rows"]) == (36, 32, 64)
    assert plan(core, 28, 4, 64, [1024], 1024)["staged"] == 20
    assert plan(core, 14, 2, 64, [3072], 3072)["staged"] == 24
    assert plan(core, 28, 4, 128, [2048], 2048)["staged"] == 16
    assert plan(core, 28, 4, 128, [512], 512)["staged"] < 8
    # the q/k/v projection: one skinny kernel for few rows of a small matrix (1152 x 896 at 8
    # rows: 6.0 us against 10.6 as partial sums and a finishing kernel), partial sums for a
    # matrix of 24 MB or more (4608 x 3584 at 8..64 rows: 14.0..16.5 us against 15.2..30.7)
    assert core.choose_qkv(BF16, BF16, 8, 1152, 896, 64, 64, 16, True) == 0
    assert core.choose_qkv(BF16, BF16, 8, 4608, 3584, 128, 128, 16, True) == 2
    # the head: the skinny kernel below 8 rows, tiles from there (152064 x 3584: 188 / 204 us
    # skinny at 1 / 8 rows, 187 / 191 tiled)
    assert core.choose_linear(BF16, 1, 151936, 896, False, False, F32, 0) == 1
    assert core.choose_linear(BF16, 8, 151936, 896, False, False, F32, 0) == 3

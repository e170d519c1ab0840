"""Each HIP kernel alone against a plain float32 reference of the same op, at sizes other than
the engine's own (odd row counts, widths that are no power of two, several head sizes)."""

from __future__ import annotations

import math

import pytest
import torch

from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops():
    from mercury_amd.kernels import ops as o

    return o


def tol(dtype):
    # float32: a few ulps of accumulated error; bfloat16: one rounding of the output (2^-8).
    return dict(atol=2e-6, rtol=1e-5) if dtype == torch.float32 else dict(atol=1e-2, rtol=1.6e-2)


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def as_dtype(x, dtype):
    """The values the kernel will see, as float32 on the host, and the device tensor."""
    d = x.to(dtype)
    return d.float(), d.to(DEV)


# ------------------------------------------------------------------------------- embedding


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [168, 165, 3584, 8])
def test_embed_gathers_rows_as_float32(dtype, hidden):
    table_h, table_d = as_dtype(rnd(1003, hidden), dtype)
    ids = torch.tensor([0, 1002, 5, 5, 77], dtype=torch.int32)
    out = ops().embed(ids.to(DEV), table_d)
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table_h[ids.long()])


# --------------------------------------------------------------------------------- RMSNorm


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1, 896), (7, 1000), (129, 168), (3, 4100), (300, 5120),
                                       (2, 20000), (260, 8200), (3, 40004), (2, 1003)])
def test_rmsnorm_matches_plain(dtype, rows, cols):
    h = rnd(rows, cols, seed=1, scale=3.0)
    w_h, w_d = as_dtype(1 + rnd(cols, seed=2, scale=0.1), dtype)
    want, _ = plain.rms_norm(h, w_h, 1e-5)
    got = ops().rmsnorm(h.to(DEV), w_d, 1e-5, dtype)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype))


def test_rmsnorm_against_the_library_routine():
    h = rnd(5, 264, seed=3)
    w = 1 + rnd(264, seed=4, scale=0.1)
    want = torch.nn.functional.rms_norm(h, (264,), w, 1e-6)
    got = ops().rmsnorm(h.to(DEV), w.to(DEV), 1e-6, torch.float32)
    torch.testing.assert_close(got.cpu(), want, atol=2e-6, rtol=1e-5)


def test_rmsnorm_constant_and_zero_rows():
    eps = 1e-6
    h = torch.zeros(2, 300)
    h[1] = 2.5
    got = ops().rmsnorm(h.to(DEV), torch.ones(300, device=DEV), eps, torch.float32).cpu()
    assert torch.equal(got[0], torch.zeros(300))            # no NaN from an all-zero row
    assert torch.allclose(got[1], torch.full((300,), 2.5 / math.sqrt(2.5**2 + eps)), atol=1e-6)


@pytest.mark.parametrize("rows,cols,slices", [(9, 200, 3), (300, 5120, 3), (2, 1003, 5), (70, 8200, 2)])
def test_rmsnorm_adds_partial_sums_into_the_stream_first(rows, cols, slices):
    """The residual sum is part of the norm: h <- h + sum(partials), then normalise
    (reference: the sum is the norm's second result, mercury/model/qwen2.py:27-31)."""
    h = rnd(rows, cols, seed=5)
    parts = rnd(slices, rows, cols, seed=6)
    w = 1 + rnd(cols, seed=7, scale=0.1)
    want, total = plain.rms_norm(parts.sum(0), w, 1e-6, residual=h)
    h_d = h.clone().to(DEV)
    got = ops().rmsnorm(h_d, w.to(DEV), 1e-6, torch.float32, partials=parts.to(DEV))
    torch.testing.assert_close(h_d.cpu(), total, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(got.cpu(), want, atol=3e-6, rtol=1e-5)


def test_rmsnorm_selected_rows_in_caller_order():
    h = rnd(20, 128, seed=8)
    w = torch.ones(128)
    rows = torch.tensor([19, 0, 7], dtype=torch.int32)
    want, _ = plain.rms_norm(h[rows.long()], w, 1e-6)
    got = ops().rmsnorm(h.to(DEV), w.to(DEV), 1e-6, torch.float32, rows=rows.to(DEV))
    torch.testing.assert_close(got.cpu(), want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("weight_dtype", DTYPES)
def test_rmsnorm_bfloat16_output_with_either_weight_precision(weight_dtype):
    h = rnd(4, 896, seed=9)
    w_h, w_d = as_dtype(1 + rnd(896, seed=10, scale=0.1), weight_dtype)
    want, _ = plain.rms_norm(h, w_h, 1e-6)
    got = ops().rmsnorm(h.to(DEV), w_d, 1e-6, torch.bfloat16)
    torch.testing.assert_close(got.float().cpu(), want, **tol(torch.bfloat16))


# ------------------------------------------------------------------------------ projections


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 1003, 168), (70, 130, 50), (129, 64, 257), (5, 1, 7)])
def test_linear_matches_the_library_product(dtype, m, n, k):
    x_h, x_d = as_dtype(rnd(m, k, seed=11), dtype)
    w_h, w_d = as_dtype(rnd(n, k, seed=12, scale=0.1), dtype)
    b_h, b_d = as_dtype(rnd(n, seed=13), dtype)
    want = torch.nn.functional.linear(x_h.double(), w_h.double(), b_h.double()).float()
    got = ops().linear(x_d, w_d, b_d)
    assert got.dtype == dtype
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype))
    # float32 result from bfloat16 operands (the logits path)
    got32 = ops().linear(x_d, w_d, None, out_dtype=torch.float32)
    want32 = torch.nn.functional.linear(x_h.double(), w_h.double()).float()
    torch.testing.assert_close(got32.cpu(), want32, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_accumulates_into_the_float32_stream(dtype):
    x_h, x_d = as_dtype(rnd(33, 100, seed=14), dtype)
    w_h, w_d = as_dtype(rnd(72, 100, seed=15, scale=0.1), dtype)
    acc = rnd(33, 72, seed=16)
    acc_d = acc.clone().to(DEV)
    ops().linear(x_d, w_d, out=acc_d, accumulate=True)
    want = acc + (x_h.double() @ w_h.double().T).float()
    torch.testing.assert_close(acc_d.cpu(), want, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("m,n,k", [(1, 1003, 168), (8, 896, 4864), (17, 1152, 896), (64, 130, 264),
                                   (33, 9728, 896), (5, 7, 8)])
def test_skinny_projection_partial_sums(m, n, k):
    """Few rows on the matrix cores: float32 slices over K whose sum is the product."""
    x_h, x_d = as_dtype(rnd(m, k, seed=21), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(n, k, seed=22, scale=0.1), torch.bfloat16)
    parts = ops().linear_partials(x_d, w_d)
    assert parts.dtype == torch.float32 and parts.shape[1:] == (m, n)
    want = (x_h.double() @ w_h.double().T).float()
    torch.testing.assert_close(parts.sum(0).cpu(), want, atol=2e-4, rtol=1e-4)
    whole = ops().linear(x_d, w_d, out_dtype=torch.float32, kernel="mfma")   # one slice: the logits path
    torch.testing.assert_close(whole.cpu(), want, atol=2e-4, rtol=1e-4)
    assert not ops().wants_partials(x_d.float(), w_d.float())


@pytest.mark.parametrize("m,n,k", [(17, 130, 264), (64, 3584, 1024), (300, 72, 2048), (129, 1152, 896),
                                   (512, 896, 4864), (40, 1003, 4104)])
def test_tiled_projection_partial_sums(m, n, k):
    """More than 16 rows over a long K: tiles through LDS over slices of K, every slice with a
    float32 result of its own; their sum is the product, for the planner's own number of
    slices and for any other that the stages of K divide into."""
    lib = ops()._lib.load("mfma")
    x_h, x_d = as_dtype(rnd(m, k, seed=51), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(n, k, seed=52, scale=0.1), torch.bfloat16)
    want = (x_h.double() @ w_h.double().T).float()
    parts = ops().linear_partials(x_d, w_d)
    assert parts.shape == (lib.mk_linear_tiled_slices(m, n, k), m, n)
    torch.testing.assert_close(parts.sum(0).cpu(), want, atol=5e-4, rtol=1e-4)
    stages = -(-k // 64)
    for slices in (1, 2, 3, 5):
        per = -(-stages // slices)
        if -(-stages // per) != slices:
            continue
        out = torch.full((slices, m, n), 7.0, device=DEV)
        ops()._lib.check(lib, lib.mk_linear_tiled_partials(
            x_d.data_ptr(), w_d.data_ptr(), out.data_ptr(), m, n, k, slices,
            torch.cuda.current_stream().cuda_stream), "partials")
        torch.testing.assert_close(out.sum(0).cpu(), want, atol=5e-4, rtol=1e-4)


@pytest.mark.parametrize("m,n,k", [(70, 130, 56), (129, 1152, 896), (300, 64, 264), (2048, 896, 4864),
                                   (65, 1003, 168)])
def test_tiled_projection(m, n, k):
    """Many rows on the matrix cores through LDS: bfloat16 with bias, float32, accumulate."""
    x_h, x_d = as_dtype(rnd(m, k, seed=23), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(n, k, seed=24, scale=0.1), torch.bfloat16)
    b_h, b_d = as_dtype(rnd(n, seed=25), torch.bfloat16)
    want = (x_h.double() @ w_h.double().T).float()
    got = ops().linear(x_d, w_d, b_d, kernel="mfma")
    torch.testing.assert_close(got.float().cpu(), want + b_h, **tol(torch.bfloat16))
    got = ops().linear(x_d, w_d, b_d.float(), kernel="mfma")            # a float32 bias
    torch.testing.assert_close(got.float().cpu(), want + b_h, **tol(torch.bfloat16))
    got32 = ops().linear(x_d, w_d, out_dtype=torch.float32, kernel="mfma")
    torch.testing.assert_close(got32.cpu(), want, atol=5e-4, rtol=1e-4)
    acc = rnd(m, n, seed=26)
    acc_d = acc.clone().to(DEV)
    ops().linear(x_d, w_d, out=acc_d, accumulate=True, kernel="mfma")
    torch.testing.assert_close(acc_d.cpu(), acc + want, atol=5e-4, rtol=1e-4)


@pytest.mark.parametrize("m,inter,k", [(1, 4864, 896), (8, 410, 168), (33, 704, 256), (64, 176, 64),
                                       (65, 410, 168), (300, 4864, 896), (2048, 176, 64), (129, 704, 264)])
def test_gated_projection(m, inter, k):
    """silu(x Wg^T) * (x Wu^T) with the gating in the projection's epilogue equals the gating
    kernel applied to the stored projection."""
    x_h, x_d = as_dtype(rnd(m, k, seed=31), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(2 * inter, k, seed=32, scale=0.1), torch.bfloat16)
    got = ops().gated_projection(x_d, w_d)
    stored = (x_h.double() @ w_h.double().T).float().to(torch.bfloat16)
    want = ops().silu_mul(stored.to(DEV))
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), atol=2e-3, rtol=1.6e-2)
    plain_want = plain.gated_mlp(x_h, w_h[:inter], w_h[inter:], torch.eye(inter))
    torch.testing.assert_close(got.float().cpu(), plain_want, **tol(torch.bfloat16))


@pytest.mark.parametrize("m,n,k", [(300, 520, 200), (257, 130, 64), (70, 1004, 1096), (513, 264, 8),
                                   (40, 776, 136)])
def test_every_tile_configuration(m, n, k):
    """Each tile shape of the tiled projection, forced, at sizes that leave partial tiles in
    both directions and a partial last stage of K: every epilogue, and the gated form with
    gate and up rows interleaved per wavefront."""
    lib = ops()._lib.load("mfma")
    x_h, x_d = as_dtype(rnd(m, k, seed=27), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(n, k, seed=28, scale=0.1), torch.bfloat16)
    b_h, b_d = as_dtype(rnd(n, seed=29), torch.bfloat16)
    want = (x_h.double() @ w_h.double().T).float()
    inter = n // 2
    stored = want.to(torch.bfloat16)
    gated_want = ops().silu_mul(stored.to(DEV)).float().cpu()
    acc = rnd(m, n, seed=30)
    for config in range(lib.mk_linear_tiled_configs()):
        got = ops().linear(x_d, w_d, b_d, kernel="mfma", tile_config=config)
        torch.testing.assert_close(got.float().cpu(), want + b_h, **tol(torch.bfloat16))
        got32 = ops().linear(x_d, w_d, out_dtype=torch.float32, kernel="mfma", tile_config=config)
        torch.testing.assert_close(got32.cpu(), want, atol=5e-4, rtol=1e-4)
        acc_d = acc.clone().to(DEV)
        ops().linear(x_d, w_d, out=acc_d, accumulate=True, kernel="mfma", tile_config=config)
        torch.testing.assert_close(acc_d.cpu(), acc + want, atol=5e-4, rtol=1e-4)
        gated = ops().gated_projection(x_d, w_d, tile_config=config)
        assert gated.shape == (m, inter)
        torch.testing.assert_close(gated.float().cpu(), gated_want, atol=2e-3, rtol=1.6e-2)


def test_the_tile_configuration_follows_the_problem():
    """Large tiles where they fill the chip, small ones where large ones would leave compute
    units idle, and at most 64 tile rows for at most 64 rows of x."""
    lib = ops()._lib.load("mfma")
    assert lib.mk_linear_tiled_config(8192, 8192, 8192, 2) == 0        # 256 x 256
    assert lib.mk_linear_tiled_config(2048, 896, 4864, 8) == 4         # 64 x 64: 448 tiles
    assert lib.mk_linear_tiled_config(2048, 3584, 18944, 8) == 1       # 128 x 256: 224 tiles
    assert lib.mk_linear_tiled_config(40, 151936, 896, 4) in (4, 5)
    # gate and up rows in one tile: few rows stream the weights, a large matrix fastest
    # through the 128 x 256 tile's three stages (a small one in tiles that spread over the
    # compute units); some hundred rows want 128 x 256 too, thousands 256 x 256
    # (128 x 192 where those tiles spread better over the compute units than 128 x 256)
    assert lib.mk_gated_tiled_config(32, 18944, 3584) == 7 and lib.mk_gated_tiled_config(32, 27648, 5120) == 1
    assert lib.mk_gated_tiled_config(32, 4864, 896) == 4
    assert lib.mk_gated_tiled_config(512, 27648, 5120) == 0
    # 256 x 192 where 256 columns leave the last round of tiles half empty: 4608 columns at
    # 2,048 rows of x (72 us against 90 in 128 x 256)
    assert lib.mk_linear_tiled_config(2048, 4608, 3584, 2) == 6
    # 256 x 320, the most products per byte a stage brings, where its tiles fill the chip:
    # 18944 pairs of rows at 512 rows of x (126 us against 179 in 128 x 256, 183 in 256 x 192),
    # at 2,048 (448 against 488 in 256 x 256); 4864 pairs at 2,048 (45 against 54 in 256 x 192)
    assert lib.mk_gated_tiled_config(512, 18944, 3584) == 9
    assert lib.mk_gated_tiled_config(2048, 18944, 3584) == 9
    assert lib.mk_gated_tiled_config(2048, 4864, 896) == 9


def test_which_skinny_projections_are_split():
    """K is split into partial sums wherever the matrix is large enough for bandwidth to
    matter; how often follows how evenly the workgroups then spread over the compute units."""
    lib = ops()._lib.load("mfma")

    def wants(m, n, k):
        return ops().wants_partials(torch.zeros(m, k, dtype=torch.bfloat16, device=DEV),
                                    torch.zeros(n, k, dtype=torch.bfloat16, device=DEV))
    assert wants(8, 896, 4864)             # 8.7 MB behind 28 tiles of rows
    assert not wants(8, 896, 896)          # small: latency is the cost, not bandwidth
    assert wants(8, 3584, 4096) and wants(64, 3584, 4096)
    assert not wants(8, 896, 4868)         # K % 8 != 0: not for the matrix cores at all
    assert lib.mk_linear_skinny_slices(8, 896, 4864) == 8      # 224 workgroups: one a unit
    assert lib.mk_linear_skinny_slices(8, 3584, 18944) == 2    # 224 again
    assert lib.mk_linear_skinny_slices(8, 5120, 27648) == 3    # 480: two a unit, few idle
    assert lib.mk_linear_skinny_slices(8, 8192, 8192) == 1     # 256 as it is


@pytest.mark.parametrize("m,n,k", [(1, 896, 896), (8, 1003, 168), (17, 130, 264), (64, 3584, 1024),
                                   (33, 20000, 64), (5, 7, 8)])
@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16, torch.float32])
def test_skinny_projection_into_the_stream(m, n, k, bias_dtype):
    """Few rows, all of K in a workgroup, the product (and a bias) added to the float32
    stream in the epilogue."""
    x_h, x_d = as_dtype(rnd(m, k, seed=41), torch.bfloat16)
    w_h, w_d = as_dtype(rnd(n, k, seed=42, scale=0.1), torch.bfloat16)
    acc = rnd(m, n, seed=43)
    acc_d = acc.clone().to(DEV)
    want = acc + (x_h.double() @ w_h.double().T).float()
    bias_d = None
    if bias_dtype is not None:
        b_h, bias_d = as_dtype(rnd(n, seed=44), bias_dtype)
        want = want + b_h
    ops().linear(x_d, w_d, bias_d, out=acc_d, accumulate=True, kernel="mfma")
    torch.testing.assert_close(acc_d.cpu(), want, atol=2e-4, rtol=1e-4)


QKV_CASES = [  # n_q, n_kv, d, page, K, rows
    (14, 2, 64, 16, 896, 8), (6, 1, 32, 8, 168, 1), (4, 4, 128, 32, 264, 17), (3, 1, 96, 16, 72, 64),
    (2, 2, 64, 16, 64, 16), (14, 2, 64, 32, 896, 200), (4, 4, 128, 32, 264, 130)]


@pytest.mark.parametrize("n_q,n_kv,d,page,k,m", QKV_CASES)
@pytest.mark.parametrize("mode", ["plain", "unrotated", "queries_only"])
def test_qkv_projection_with_rotation_and_cache_write_in_one_kernel(n_q, n_kv, d, page, k, m, mode):
    """The fused q/k/v kernels (the skinny one for few rows, the tiled one in every tile
    configuration for any number) equal projection, then rotary + cache write, and the plain
    implementation; tokens sit on page edges, in several sequences, one of them on a page
    that was given back."""
    o = ops()
    write_kv = mode != "queries_only"
    rot = 0 if mode == "unrotated" else d
    heads_kv = n_kv if write_kv else 0
    width = (n_q + 2 * heads_kv) * d
    theta, max_pos = 10000.0, 8 * page
    cos, sin = rotary_tables(d, theta, max_pos)
    w_h, w_d = as_dtype(rnd(width, k, seed=51, scale=0.05), torch.bfloat16)
    b_h, b_d = as_dtype(rnd(width, seed=52), torch.bfloat16)
    # positions around page edges, spread over three sequences
    edge = [page - 1, page, 2 * page - 1, 0, 3 * page, 1]
    positions = [edge[i % len(edge)] + (i // len(edge)) for i in range(m)]
    token_seq = [i % 3 for i in range(m)]
    seen = set()
    for i in range(m):                       # one slot per (sequence, position)
        while (token_seq[i], positions[i]) in seen:
            positions[i] += 1
        seen.add((token_seq[i], positions[i]))
    table = torch.arange(1, 1 + 3 * 8, dtype=torch.int32).view(3, 8).contiguous()
    dropped = None
    if write_kv and m >= 3:
        dropped = 2
        table[token_seq[dropped], positions[dropped] // page] = -1
    pos_d = torch.tensor(positions, dtype=torch.int32, device=DEV)
    seq_d = torch.tensor(token_seq, dtype=torch.int32, device=DEV)
    caches = [[torch.zeros(32, n_kv, page, d, dtype=torch.bfloat16, device=DEV),
               torch.zeros(32, n_kv, d, page, dtype=torch.bfloat16, device=DEV)] for _ in range(2)]
    x_h, x_d = as_dtype(rnd(m, k, seed=55), torch.bfloat16)
    x_in = x_d
    assert o.fuses_qkv(x_in, w_d, d, rot, page)
    cos_d, sin_d = (cos.to(DEV), sin.to(DEV)) if rot else (None, None)
    q_got = o.qkv_project(x_in, w_d, b_d, cos_d, sin_d, pos_d, seq_d, table.to(DEV),
                          caches[0][0] if write_kv else None, caches[0][1] if write_kv else None,
                          n_q, n_kv, d, rot, write_kv, fused=True)
    assert q_got.shape == (m, n_q * d) and q_got.dtype == torch.bfloat16
    stored = o.linear(x_d, w_d, b_d, kernel="mfma" if m > 64 else "auto")
    q_ref = o.rope_kv_write(stored, cos_d, sin_d, pos_d, seq_d, table.to(DEV),
                            caches[1][0] if write_kv else None, caches[1][1] if write_kv else None,
                            n_q, heads_kv, d, rot, write_kv)[:, : n_q * d]
    # q, k and v are rounded to bfloat16 before the rotation mixes two of them: an error of one
    # rounding of the largest projected value can land on a small rotated one
    bf = dict(atol=float(stored.float().abs().max()) * 2.0 ** -7, rtol=1.6e-2)
    torch.testing.assert_close(q_got.float().cpu(), q_ref.float().cpu(), **bf)
    if write_kv:
        torch.testing.assert_close(caches[0][0].float().cpu(), caches[1][0].float().cpu(), **bf)
        torch.testing.assert_close(caches[0][1].float().cpu(), caches[1][1].float().cpu(), **bf)
        assert (caches[0][0] != 0).eq(caches[1][0] != 0).all()      # the same slots, no others
        assert (caches[0][1] != 0).eq(caches[1][1] != 0).all()
        assert caches[0][0].abs().sum() > 0
    for config in range(o._lib.load("mfma").mk_linear_tiled_configs()):
        tiled = [torch.zeros_like(caches[0][0]), torch.zeros_like(caches[0][1])]
        q_tiled = o.qkv_project(x_in, w_d, b_d, cos_d, sin_d, pos_d, seq_d, table.to(DEV),
                                tiled[0] if write_kv else None, tiled[1] if write_kv else None,
                                n_q, n_kv, d, rot, write_kv, fused=True, tile_config=config)
        torch.testing.assert_close(q_tiled.float().cpu(), q_ref.float().cpu(), **bf)
        if write_kv:
            torch.testing.assert_close(tiled[0].float().cpu(), caches[1][0].float().cpu(), **bf)
            torch.testing.assert_close(tiled[1].float().cpu(), caches[1][1].float().cpu(), **bf)
            assert (tiled[0] != 0).eq(caches[1][0] != 0).all() and (tiled[1] != 0).eq(caches[1][1] != 0).all()
    # and the plain implementation, from the formulas
    y = ((x_h.double() @ w_h.double().T).float() + b_h).to(torch.bfloat16).float()
    q = y[:, : n_q * d].view(m, n_q, d)
    if rot:
        full_cos, full_sin = plain.rotary_table(d, positions, theta)
        kk = y[:, n_q * d: (n_q + n_kv) * d].view(m, n_kv, d) if write_kv else q[:, :1]
        q, k_want = plain.apply_rotary(q, kk, full_cos, full_sin)
    elif write_kv:
        k_want = y[:, n_q * d: (n_q + n_kv) * d].view(m, n_kv, d)
    torch.testing.assert_close(q_got.float().cpu().view(m, n_q, d), q, **bf)
    if write_kv:
        v_want = y[:, (n_q + n_kv) * d:].view(m, n_kv, d)
        for t in range(m):
            pg, off = int(table[token_seq[t], positions[t] // page]), positions[t] % page
            if pg < 0:          # the page that was given back, and whoever else sits on it
                continue
            assert t != dropped
            torch.testing.assert_close(caches[0][0][pg, :, off].float().cpu(), k_want[t], **bf)
            torch.testing.assert_close(caches[0][1][pg, :, :, off].float().cpu(), v_want[t], **bf)


def test_qkv_projection_falls_back_where_the_fused_kernel_does_not_apply():
    o = ops()
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=DEV)
    many = torch.zeros(40, 64, dtype=torch.bfloat16, device=DEV)
    assert o.fuses_qkv(x, torch.zeros(512, 64, dtype=torch.bfloat16, device=DEV), 64, 64, 16)
    assert o.fuses_qkv(many, torch.zeros(512, 64, dtype=torch.bfloat16, device=DEV), 64, 64, 16)
    big = torch.zeros(7168, 5120, dtype=torch.bfloat16, device=DEV)
    assert not o.fuses_qkv(torch.zeros(64, 5120, dtype=torch.bfloat16, device=DEV), big, 128, 128, 16)
    assert o.fuses_qkv(many, torch.zeros(4608, 64, dtype=torch.bfloat16, device=DEV), 128, 128, 16)
    # a large matrix goes as partial sums and a finishing kernel at any small number of rows
    assert not o.fuses_qkv(torch.zeros(8, 5120, dtype=torch.bfloat16, device=DEV), big, 128, 128, 16)
    mid = torch.zeros(4608, 3584, dtype=torch.bfloat16, device=DEV)
    assert not o.fuses_qkv(torch.zeros(64, 3584, dtype=torch.bfloat16, device=DEV), mid, 128, 128, 16)
    assert o.fuses_qkv(torch.zeros(2048, 3584, dtype=torch.bfloat16, device=DEV), mid, 128, 128, 16)
    assert not o.fuses_qkv(x, x, 48, 48, 16)          # heads not a multiple of 32 wide
    assert not o.fuses_qkv(x, x, 64, 32, 16)          # rotation over part of the head
    assert not o.fuses_qkv(x.float(), x.float(), 64, 64, 16)
    assert o.fuses_qkv(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), x, 64, 64, 16)  # tiles
    assert not o.fuses_qkv(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), x, 48, 48, 16)


def test_matrix_core_projection_refuses_what_it_cannot_do():
    from mercury_amd.kernels.ops import KernelArgumentError

    x = torch.zeros(4, 50, dtype=torch.bfloat16, device=DEV)      # K % 8 != 0
    w = torch.zeros(6, 50, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelArgumentError):
        ops().linear(x, w, kernel="mfma")
    assert ops().linear(x, w).shape == (4, 6)                       # "auto" takes the other kernel


def test_consumers_of_partial_sums():
    """Rotary + cache write over K-split slices equals the stored-projection form applied to
    the rounded sum."""
    n_q, n_kv, d, page = 6, 2, 32, 16
    width = (n_q + 2 * n_kv) * d
    parts = rnd(4, 5, width, seed=28)
    bias = rnd(width, seed=29).to(torch.bfloat16)
    cos, sin = rotary_tables(d, 10000.0, 64)
    positions = torch.tensor([3, 4, 40, 41, 0], dtype=torch.int32, device=DEV)
    token_seq = torch.tensor([0, 0, 1, 1, 2], dtype=torch.int32, device=DEV)
    table = torch.tensor([[1, -1, -1], [2, 3, 4], [5, -1, -1]], dtype=torch.int32, device=DEV)
    caches = [[torch.zeros(8, n_kv, page, d, dtype=torch.bfloat16, device=DEV),
               torch.zeros(8, n_kv, d, page, dtype=torch.bfloat16, device=DEV)] for _ in range(2)]
    stored = (parts.sum(0) + bias.float()).to(torch.bfloat16).to(DEV)
    q_want = ops().rope_kv_write(stored, cos.to(DEV), sin.to(DEV), positions, token_seq, table,
                                 caches[0][0], caches[0][1], n_q, n_kv, d, d)[:, : n_q * d]
    q_got = ops().rope_kv_write(parts.to(DEV), cos.to(DEV), sin.to(DEV), positions, token_seq, table,
                                caches[1][0], caches[1][1], n_q, n_kv, d, d, bias=bias.to(DEV),
                                out_dtype=torch.bfloat16)
    assert torch.equal(q_got.cpu(), q_want.cpu())
    assert torch.equal(caches[0][0].cpu(), caches[1][0].cpu())
    assert torch.equal(caches[0][1].cpu(), caches[1][1].cpu())
    assert caches[0][0].abs().sum() > 0


def test_linear_rows_do_not_depend_on_the_batch():
    """A row's result is bitwise the same alone and among 100 others."""
    x = rnd(101, 300, seed=17).to(DEV)
    w = rnd(77, 300, seed=18).to(DEV)
    together = ops().linear(x, w)
    alone = ops().linear(x[50:51].contiguous(), w)
    assert torch.equal(together[50:51], alone)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_matches_plain(dtype):
    gu_h, gu_d = as_dtype(rnd(13, 2 * 410, seed=19, scale=2.0), dtype)
    want = plain.silu(gu_h[:, :410]) * gu_h[:, 410:]
    got = ops().silu_mul(gu_d)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype))
    assert torch.equal(ops().silu_mul(torch.zeros(2, 8, device=DEV)).cpu(), torch.zeros(2, 4))
    torch.testing.assert_close(plain.silu(gu_h), torch.nn.functional.silu(gu_h))


# ------------------------------------------------------------------- rotary + cache write


def rotary_tables(d, theta, positions):
    cos, sin = plain.rotary_table(d, range(positions), theta)
    return cos[:, : d // 2].contiguous(), sin[:, : d // 2].contiguous()


def paged(kv, pages, page_size, num_pages, dtype, transposed=False):
    """Host helper: lay [S, n_kv, d] out in a key cache [num_pages, n_kv, page, d] or, with
    `transposed`, a value cache [num_pages, n_kv, d, page]."""
    s, n_kv, d = kv.shape
    cache = torch.zeros(num_pages, n_kv, page_size, d, dtype=dtype)
    for p in range(s):
        cache[pages[p // page_size], :, p % page_size, :] = kv[p].to(dtype)
    return cache.transpose(2, 3).contiguous() if transposed else cache


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,d,page", [(4, 2, 16, 16), (6, 1, 48, 8), (3, 3, 80, 32)])
def test_rope_and_cache_write(dtype, n_q, n_kv, d, page):
    theta, max_pos = 10000.0, 128
    cos, sin = rotary_tables(d, theta, max_pos)
    # two sequences: tokens at positions 30..39 of sequence 0, position 70 of sequence 1
    positions = list(range(30, 40)) + [70]
    token_seq = [0] * 10 + [1]
    table = torch.full((2, max_pos // page), -1, dtype=torch.int32)
    table[0, : 40 // page + 1] = torch.arange(3, 3 + 40 // page + 1, dtype=torch.int32)
    table[1, : 70 // page + 1] = torch.arange(20, 20 + 70 // page + 1, dtype=torch.int32)
    tokens = len(positions)
    qkv_h, qkv_d = as_dtype(rnd(tokens, (n_q + 2 * n_kv) * d, seed=20), dtype)
    k_cache = torch.zeros(40, n_kv, page, d, dtype=dtype, device=DEV)
    v_cache = torch.zeros(40, n_kv, d, page, dtype=dtype, device=DEV)
    ops().rope_kv_write(qkv_d, cos.to(DEV), sin.to(DEV),
                        torch.tensor(positions, dtype=torch.int32, device=DEV),
                        torch.tensor(token_seq, dtype=torch.int32, device=DEV), table.to(DEV),
                        k_cache, v_cache, n_q, n_kv, d, d)
    q = qkv_h[:, : n_q * d].view(tokens, n_q, d)
    k = qkv_h[:, n_q * d: (n_q + n_kv) * d].view(tokens, n_kv, d)
    v = qkv_h[:, (n_q + n_kv) * d:].view(tokens, n_kv, d)
    full_cos, full_sin = plain.rotary_table(d, positions, theta)
    q_want, k_want = plain.apply_rotary(q, k, full_cos, full_sin)
    torch.testing.assert_close(qkv_d[:, : n_q * d].float().cpu().view(tokens, n_q, d), q_want, **tol(dtype))
    touched = torch.zeros(40, page, dtype=torch.bool)
    for t, (p, s) in enumerate(zip(positions, token_seq)):
        pg, off = int(table[s, p // page]), p % page
        assert plain.slot_mapping(table[s].tolist(), p, p + 1, page) == [pg * page + off]
        torch.testing.assert_close(k_cache[pg, :, off].float().cpu(), k_want[t], **tol(dtype))
        assert torch.equal(v_cache[pg, :, :, off].float().cpu(), v[t])
        touched[pg, off] = True
    untouched = ~touched[:, None, :, None].expand(40, n_kv, page, d)
    assert torch.count_nonzero(k_cache.cpu()[untouched]) == 0
    assert torch.count_nonzero(v_cache.cpu().transpose(2, 3)[untouched]) == 0


def test_rotary_pairing_sign_and_identity_at_zero():
    """rotate_half([1,2,3,4]) = [-3,-4,1,2] (reference: tests/test_attention.py:177-179):
    with cos = 0 and sin = 1 the kernel must return exactly that; position 0 is the identity."""
    assert torch.equal(plain.rotate_half(torch.tensor([[1.0, 2.0, 3.0, 4.0]])),
                       torch.tensor([[-3.0, -4.0, 1.0, 2.0]]))
    cos = torch.tensor([[1.0, 1.0], [0.0, 0.0]], device=DEV)
    sin = torch.tensor([[0.0, 0.0], [1.0, 1.0]], device=DEV)
    qkv = torch.tensor([[1.0, 2.0, 3.0, 4.0], [1.0, 2.0, 3.0, 4.0]], device=DEV)
    ops().rope_kv_write(qkv, cos, sin, torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                        torch.zeros(2, dtype=torch.int32, device=DEV),
                        torch.zeros(1, 1, dtype=torch.int32, device=DEV), None, None, 1, 0, 4, 4,
                        write_kv=False)
    assert torch.equal(qkv.cpu(), torch.tensor([[1.0, 2.0, 3.0, 4.0], [-3.0, -4.0, 1.0, 2.0]]))


def test_rotary_scores_depend_on_distance_only():
    """<rot(q, m), rot(k, n)> is the same for (3, 3) and (9, 9), and for (5, 2) and (105, 102)
    (reference: tests/test_attention.py:182-197)."""
    d = 32
    cos, sin = rotary_tables(d, 10000.0, 128)
    base_h = rnd(1, 2 * d, seed=21)

    def rotated(pos_q, pos_k):
        out = []
        for pos in (pos_q, pos_k):
            buf = base_h.clone().to(DEV)  # two heads: q and "k" both as q heads
            ops().rope_kv_write(buf, cos.to(DEV), sin.to(DEV),
                                torch.tensor([pos], dtype=torch.int32, device=DEV),
                                torch.zeros(1, dtype=torch.int32, device=DEV),
                                torch.zeros(1, 1, dtype=torch.int32, device=DEV), None, None, 2, 0,
                                d, d, write_kv=False)
            out.append(buf.cpu())
        return float((out[0][0, :d] * out[1][0, d:]).sum())

    assert abs(rotated(3, 3) - rotated(9, 9)) < 1e-5
    assert abs(rotated(5, 2) - rotated(105, 102)) < 1e-4
    assert abs(rotated(5, 2) - rotated(2, 5)) > 1e-3   # the sign of the distance matters


# --------------------------------------------------------------------------------- attention


def run_attention(q_h, k_h, v_h, dtype, pages_per_seq, page, num_pages, seq_lens, q_lens, scale,
                  window=None, poison=None, kernel="auto", hide_before=None, tile_rows=None,
                  split_override=None, staged=None):
    """q_h: list per sequence of [q_len, n_q, d] (the last q_len positions of the sequence);
    k_h/v_h: list per sequence of [seq_len, n_kv, d].  `hide_before`: per sequence, the number
    of leading pages to drop from the table (-1) and to poison, as after a window passed."""
    from tests.helpers import context_from_spans

    n_q, d = q_h[0].shape[1:]
    n_kv = k_h[0].shape[1]
    k_cache = torch.zeros(num_pages, n_kv, page, d, dtype=dtype)
    v_cache = torch.zeros_like(k_cache)
    if poison is not None:
        k_cache[:] = poison
        v_cache[:] = poison
    width = max(len(p) for p in pages_per_seq)
    table = torch.full((len(q_h), width), -1, dtype=torch.int32)
    for s, pages in enumerate(pages_per_seq):
        table[s, : len(pages)] = torch.tensor(pages, dtype=torch.int32)
        for p in range(seq_lens[s]):
            k_cache[pages[p // page], :, p % page] = k_h[s][p].to(dtype)
            v_cache[pages[p // page], :, p % page] = v_h[s][p].to(dtype)
        for g in range(hide_before[s] if hide_before else 0):
            k_cache[pages[g]] = 1e4
            v_cache[pages[g]] = 1e4
            table[s, g] = -1
    step = context_from_spans([(ql, sl - ql) for ql, sl in zip(q_lens, seq_lens)], DEV)
    q_flat = torch.cat([q.reshape(q.shape[0], n_q * d) for q in q_h]).to(dtype).to(DEV)
    v_cache = v_cache.transpose(2, 3).contiguous()      # values lie transposed within a page
    out = ops().attention(q_flat, n_q * d, k_cache.to(DEV), v_cache.to(DEV), step, table.to(DEV),
                          n_q, n_kv, d, scale, window, kernel=kernel, tile_rows=tile_rows,
                          split_override=split_override, staged=staged)
    return out.float().cpu().view(-1, n_q, d)


# (dtype, kernel) pairs: the float32-arithmetic kernel in both dtypes, the matrix-core kernel
# in bfloat16 where the head size allows it.
def kernels_for(d, page):
    pairs = [(torch.float32, "generic"), (torch.bfloat16, "generic")]
    if d % 32 == 0 and page >= 16:
        pairs.append((torch.bfloat16, "mfma"))
    return pairs


def rounded(x, dtype):
    return x.to(dtype).float()


ATTENTION_SHAPES = [(4, 2, 8, 16), (6, 1, 48, 8), (2, 2, 128, 16), (14, 2, 64, 16), (3, 1, 80, 4),
                    (5, 5, 32, 32), (12, 4, 96, 16), (8, 1, 256, 64), (28, 4, 128, 16)]
ATTENTION_CASES = [(n_q, n_kv, d, page, dtype, kernel) for n_q, n_kv, d, page in ATTENTION_SHAPES
                   for dtype, kernel in kernels_for(d, page)]


@pytest.mark.parametrize("n_q,n_kv,d,page,dtype,kernel", ATTENTION_CASES)
def test_attention_whole_prompt_matches_plain(n_q, n_kv, d, page, dtype, kernel):
    """(reference: tests/test_attention.py:67-81; scattered pages as in :135-153)"""
    s = 40 if d < 100 else 70
    q, k, v = (rounded(rnd(s, h, d, seed=30 + i), dtype) for i, h in enumerate((n_q, n_kv, n_kv)))
    pages = [11, 3, 7, 30, 2, 19, 25, 1, 9, 14, 22, 5, 28, 8, 17, 6, 4, 12][: -(-s // page)]
    got = run_attention([q], [k], [v], dtype, [pages], page, 32, [s], [s], d ** -0.5, poison=1e4,
                        kernel=kernel)
    want = plain.causal_attention(q, k, v, d ** -0.5)
    torch.testing.assert_close(got, want, **tol(dtype))
    if dtype == torch.float32:
        lib = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(0, 1)[None], k.repeat_interleave(n_q // n_kv, 1).transpose(0, 1)[None],
            v.repeat_interleave(n_q // n_kv, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
        torch.testing.assert_close(got, lib, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("d,dtype,kernel", [(8, torch.float32, "generic"), (8, torch.bfloat16, "generic"),
                                            (64, torch.bfloat16, "mfma"), (32, torch.bfloat16, "mfma")])
def test_attention_suffix_over_a_cached_prefix_and_decode_rows(d, dtype, kernel):
    """A 16-token portion at positions 32..47, beside two single decoded tokens of sequences
    of 33 and 17 tokens, in one batch (reference: tests/test_attention.py:84-132 tests the two
    cases separately)."""
    n_q, n_kv, page = 4, 2, 16
    lens, q_lens = [48, 33, 17], [16, 1, 1]
    qs, ks, vs = [], [], []
    for i, (s, ql) in enumerate(zip(lens, q_lens)):
        ks.append(rounded(rnd(s, n_kv, d, seed=40 + i), dtype))
        vs.append(rounded(rnd(s, n_kv, d, seed=50 + i), dtype))
        qs.append(rounded(rnd(s, n_q, d, seed=60 + i), dtype))
    got = run_attention([q[-ql:] for q, ql in zip(qs, q_lens)], ks, vs, dtype,
                        [[2, 5, 9], [12, 1, 30], [7, 20]], page, 32, lens, q_lens, d ** -0.5,
                        poison=1e4, kernel=kernel)
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5)[-ql:]
                      for q, k, v, ql in zip(qs, ks, vs, q_lens)])
    torch.testing.assert_close(got, want, **tol(dtype))


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "generic"), (torch.bfloat16, "generic"),
                                          (torch.bfloat16, "mfma")])
@pytest.mark.parametrize("target", [0, 15, 16, 31, 32, 255, 256, 499, 500])
def test_attention_finds_one_far_key(dtype, kernel, target):
    """One key among 501 is made to win the softmax outright (its score stands 40 above the
    rest); the output must be that key's value row.  Random weights alone would average over
    hundreds of keys and hide a key that is skipped or read from the wrong slot: the first
    key, the last, and both sides of page edges are each tried."""
    n_q, n_kv, d, page, s = 2, 1, 32, 16, 501
    k = rounded(rnd(s, n_kv, d, seed=70, scale=0.1), dtype)
    v = rounded(rnd(s, n_kv, d, seed=71), dtype)
    q = rounded(rnd(1, n_q, d, seed=72, scale=0.1), dtype)
    direction = torch.zeros(d)
    direction[3] = 16.0
    k[target, 0] = direction
    q[0, :] = direction * (40.0 * math.sqrt(d) / 256.0)
    q = rounded(q, dtype)
    pages = list(range(40, 40 + -(-s // page)))
    got = run_attention([q], [k], [v], dtype, [pages], page, 80, [s], [1], d ** -0.5, poison=1e4,
                        kernel=kernel)
    torch.testing.assert_close(got[0, 0], v[target, 0], atol=1e-3, rtol=1e-3)
    torch.testing.assert_close(got, plain.causal_attention(q, k, v, d ** -0.5, s - 1), **tol(dtype))


@pytest.mark.parametrize("d,page,dtype,kernel", [(16, 8, torch.float32, "generic"),
                                                 (16, 8, torch.bfloat16, "generic"),
                                                 (32, 16, torch.bfloat16, "mfma")])
def test_attention_special_cases_reduce_to_means(d, page, dtype, kernel):
    """One visible key -> its value; equal scores -> the mean of the visible values."""
    n_q, n_kv = 2, 1
    v = rounded(rnd(20, n_kv, d, seed=73), dtype)
    k = torch.zeros(20, n_kv, d)
    q = rounded(rnd(20, n_q, d, seed=74), dtype)
    got = run_attention([q], [k], [v], dtype, [[4, 2, 6]], page, 8, [20], [20], d ** -0.5,
                        kernel=kernel)
    for p in (0, 1, 7, 8, 19):
        want = v[: p + 1, 0].mean(0)
        torch.testing.assert_close(got[p, 0], want, **tol(dtype))


@pytest.mark.parametrize("d,page,dtype,kernel", [(16, 8, torch.float32, "generic"),
                                                 (16, 8, torch.bfloat16, "generic"),
                                                 (64, 16, torch.bfloat16, "mfma")])
@pytest.mark.parametrize("window", [1, 5, 16, 17, 33, 64])
def test_attention_window_edge(d, page, dtype, kernel, window):
    """With a window w the query at p sees keys p-w+1..p; pages wholly before the window are
    absent from the table (-1) and hold garbage, as the cache manager leaves them."""
    n_q, n_kv, s, q_len = 4, 2, 77, 6
    q, k, v = (rounded(rnd(s, h, d, seed=80 + i), dtype) for i, h in enumerate((n_q, n_kv, n_kv)))
    pages = list(range(10, 10 + -(-s // page)))
    gone = max(0, (s - q_len) - window + 1) // page
    got = run_attention([q[-q_len:]], [k], [v], dtype, [pages], page, 32, [s], [q_len], d ** -0.5,
                        window=window, kernel=kernel, hide_before=[gone])
    want = plain.causal_attention(q, k, v, d ** -0.5, 0, window)[-q_len:]
    torch.testing.assert_close(got, want, **tol(dtype))


@pytest.mark.parametrize("tile_rows,d,n_q,n_kv", [(32, 64, 14, 2), (64, 64, 14, 2), (32, 128, 8, 2),
                                                  (64, 32, 6, 6), (32, 96, 3, 1), (16, 64, 14, 2)])
@pytest.mark.parametrize("window", [None, 40])
@pytest.mark.parametrize("split", [None, (3, 2), (5, 1), (4, 0)])
def test_attention_wide_tiles_for_prompts(tile_rows, d, n_q, n_kv, window, split):
    """Wavefronts that take 32 or 64 rows (several tiles sharing the key fragments): two prompt
    portions of different length, one over a cached prefix, beside a decoded token; with the
    keys unsplit, split into fixed stretches of blocks (some splits then empty), and split
    evenly."""
    page = 16
    lens, q_lens = [150, 77, 90], [150, 33, 1]
    qs, ks, vs = [], [], []
    for i, s in enumerate(lens):
        ks.append(rounded(rnd(s, n_kv, d, seed=500 + i), torch.bfloat16))
        vs.append(rounded(rnd(s, n_kv, d, seed=510 + i), torch.bfloat16))
        qs.append(rounded(rnd(s, n_q, d, seed=520 + i), torch.bfloat16))
    pages = [list(range(0, 10)), list(range(20, 25)), list(range(30, 36))]
    got = run_attention([q[-ql:] for q, ql in zip(qs, q_lens)], ks, vs, torch.bfloat16, pages, page,
                        40, lens, q_lens, d ** -0.5, window=window, poison=1e4, kernel="mfma",
                        tile_rows=tile_rows, split_override=split)
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, 0, window)[-ql:]
                      for q, k, v, ql in zip(qs, ks, vs, q_lens)])
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


@pytest.mark.parametrize("tile_rows,d,n_q,n_kv,page,groups", [
    (16, 64, 14, 2, 16, 1), (32, 64, 14, 2, 16, 1), (16, 128, 8, 2, 32, 1), (32, 128, 4, 4, 16, 1),
    (32, 64, 3, 1, 64, 1), (16, 64, 14, 2, 16, 2), (16, 64, 14, 2, 16, 4), (16, 128, 8, 2, 32, 2),
    (16, 64, 3, 1, 64, 4),
    # the kernel of 32-row wavefronts and 64-key blocks (32 x 32 x 16 products)
    (32, 64, 14, 2, 16, 8), (32, 64, 3, 1, 64, 8), (32, 64, 8, 8, 32, 8), (32, 64, 16, 1, 128, 8),
    (32, 128, 8, 2, 32, 8), (32, 128, 3, 1, 16, 8), (32, 128, 4, 4, 16, 16), (32, 128, 14, 2, 64, 16),
    (32, 64, 14, 2, 16, 24), (32, 64, 5, 1, 32, 24)])
@pytest.mark.parametrize("window", [None, 40])
def test_attention_through_lds_for_prompts(tile_rows, d, n_q, n_kv, page, groups, window):
    """Workgroups whose wavefronts share the keys and values of one sequence through LDS, in
    one, two or four groups that take the key blocks in turn (with a window of 40 some groups
    get no block at all): prompt portions of different length, one over a cached prefix, one
    ending inside a workgroup's rows, beside a decoded token; pages scattered and poisoned
    outside."""
    lens, q_lens = [333, 150, 77, 90], [333, 150, 33, 1]
    qs, ks, vs = [], [], []
    for i, s in enumerate(lens):
        ks.append(rounded(rnd(s, n_kv, d, seed=600 + i), torch.bfloat16))
        vs.append(rounded(rnd(s, n_kv, d, seed=610 + i), torch.bfloat16))
        qs.append(rounded(rnd(s, n_q, d, seed=620 + i), torch.bfloat16))
    per = [-(-s // page) for s in lens]
    order = torch.randperm(sum(per) + 5, generator=torch.Generator().manual_seed(7)).tolist()
    pages, at = [], 0
    for n in per:
        pages.append(order[at:at + n])
        at += n
    got = run_attention([q[-ql:] for q, ql in zip(qs, q_lens)], ks, vs, torch.bfloat16, pages, page,
                        sum(per) + 5, lens, q_lens, d ** -0.5, window=window, poison=1e4,
                        kernel="mfma", tile_rows=tile_rows, staged=groups)
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, 0, window)[-ql:]
                      for q, k, v, ql in zip(qs, ks, vs, q_lens)])
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


@pytest.mark.parametrize("d,n_q,n_kv,page,groups", [
    (64, 14, 2, 16, 8), (128, 6, 2, 16, 8), (128, 6, 2, 64, 16), (64, 6, 2, 32, 24),
    (64, 14, 2, 16, 36), (64, 6, 2, 32, 20)])
@pytest.mark.parametrize("window", [None, 200, 700])
def test_attention_of_32_row_wavefronts_over_long_prompts(d, n_q, n_kv, page, groups, window):
    """The prompt kernel of 32-row wavefronts walks its key blocks in three stretches: blocks
    that a window's far edge cuts, blocks that every row sees whole, blocks that the diagonal
    cuts.  Long sequences give each stretch several blocks, with one and with two chains of
    blocks side by side, in tiles of 128 rows and (groups 20 and 36) of 64; in each sequence one far key carries a score that stands out for the
    rows that may see it, so a block dropped or taken twice shows."""
    lens, q_lens = [1500, 700, 260], [1500, 300, 129]
    qs, ks, vs = [], [], []
    for i, s in enumerate(lens):
        k = rnd(s, n_kv, d, seed=900 + i)
        q = rnd(s, n_q, d, seed=920 + i)
        far = s // 3 + 5
        k[far] *= 3.0
        q[far + 150:] += 6.0 / (9 * d ** 0.5) * k[far].repeat_interleave(n_q // n_kv, 0)
        ks.append(rounded(k, torch.bfloat16))
        vs.append(rounded(rnd(s, n_kv, d, seed=910 + i), torch.bfloat16))
        qs.append(rounded(q, torch.bfloat16))
    per = [-(-s // page) for s in lens]
    order = torch.randperm(sum(per) + 3, generator=torch.Generator().manual_seed(11)).tolist()
    pages, at = [], 0
    for n in per:
        pages.append(order[at:at + n])
        at += n
    got = run_attention([q[-ql:] for q, ql in zip(qs, q_lens)], ks, vs, torch.bfloat16, pages, page,
                        sum(per) + 3, lens, q_lens, d ** -0.5, window=window, poison=1e4,
                        kernel="mfma", tile_rows=32, staged=groups)
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, 0, window)[-ql:]
                      for q, k, v, ql in zip(qs, ks, vs, q_lens)])
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


def test_attention_through_lds_is_refused_where_it_does_not_fit():
    from mercury_amd.kernels.ops import KernelArgumentError

    q = rounded(rnd(40, 2, 96, seed=1), torch.bfloat16)
    with pytest.raises((KernelArgumentError, RuntimeError)):
        run_attention([q], [q], [q], torch.bfloat16, [[0, 1, 2]], 16, 4, [40], [40], 0.1,
                      kernel="mfma", staged=True)
    # two chains of key blocks exist for 128-wide heads only, three for 64-wide only
    for d, groups in ((64, 16), (128, 24), (128, 20), (64, 28), (64, 12)):
        q = rounded(rnd(40, 2, d, seed=1), torch.bfloat16)
        with pytest.raises((KernelArgumentError, RuntimeError)):
            run_attention([q], [q], [q], torch.bfloat16, [[0, 1, 2]], 16, 4, [40], [40], 0.1,
                          kernel="mfma", tile_rows=32, staged=groups)


@pytest.mark.parametrize("batch,context", [(1, 4096), (3, 1500), (64, 300)])
def test_attention_decode_with_split_keys(batch, context):
    """Decoded tokens over long contexts: the matrix-core kernel splits the keys over many
    wavefronts and merges the partial results; the float32 kernel does not."""
    n_q, n_kv, d, page = 14, 2, 64, 16
    lens = [context - 37 * i for i in range(batch)] if batch < 10 else [context - i for i in range(batch)]
    per = -(-context // page)
    qs = [rounded(rnd(1, n_q, d, seed=200 + i), torch.bfloat16) for i in range(batch)]
    ks = [rounded(rnd(n, n_kv, d, seed=300 + i), torch.bfloat16) for i, n in enumerate(lens)]
    vs = [rounded(rnd(n, n_kv, d, seed=400 + i), torch.bfloat16) for i, n in enumerate(lens)]
    pages = [list(range(i * per, (i + 1) * per)) for i in range(batch)]
    got = run_attention(qs, ks, vs, torch.bfloat16, pages, page, batch * per, lens, [1] * batch,
                        d ** -0.5, kernel="mfma")
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, n - 1)
                      for q, k, v, n in zip(qs, ks, vs, lens)])
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


@pytest.mark.parametrize("n_q,n_kv,d,page,lens", [
    (14, 2, 64, 16, [3000, 5, 70, 1, 33, 1024]), (8, 2, 128, 32, [2500, 1, 64, 31]),
    (6, 3, 32, 64, [130, 4000, 2]), (4, 4, 96, 16, [700, 17]), (8, 1, 256, 64, [900, 3, 200]),
    (6, 2, 192, 32, [1500, 40])])
def test_attention_decode_of_sequences_of_very_different_lengths(n_q, n_kv, d, page, lens):
    """Decoding takes the parts of a sequence's keys as every n-th block and asks for a part's
    first block before it knows the sequence's length: most parts of the short sequences here
    start past their end, where the block table holds -1 (and the cache poison); one key far
    back in each longer sequence carries a score that stands out, so a block that is skipped or
    taken twice shows."""
    bf = torch.bfloat16
    batch = len(lens)
    per = -(-max(lens) // page)
    qs, ks, vs = [], [], []
    for i, n in enumerate(lens):
        k = rnd(n, n_kv, d, seed=330 + i)
        q = rnd(1, n_q, d, seed=230 + i)
        if n > 40:
            far = n // 3
            k[far] *= 3.0
            q[0] += 6.0 / (9 * d ** 0.5) * k[far].repeat_interleave(n_q // n_kv, 0)
        qs.append(rounded(q, bf))
        ks.append(rounded(k, bf))
        vs.append(rounded(rnd(n, n_kv, d, seed=430 + i), bf))
    order = torch.randperm(batch * per + 3, generator=torch.Generator().manual_seed(5)).tolist()
    pages, at = [], 0
    for n in lens:
        need = -(-n // page)
        pages.append(order[at:at + need])
        at += need
    from mercury_amd.hostcore import core
    from mercury_amd.kernels import lib
    lib.load("core"), lib.load("mfma")
    plan = core.plan_attention(ops().BF16, d, page, n_q, n_kv, 0, [1] * batch, 1, max(lens))
    assert plan["mfma"] and plan["direct"] and plan["splits"] > 1, plan
    got = run_attention(qs, ks, vs, bf, pages, page, batch * per + 3, lens, [1] * batch,
                        d ** -0.5, poison=1e4, kernel="mfma")
    want = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, n - 1)
                      for q, k, v, n in zip(qs, ks, vs, lens)])
    torch.testing.assert_close(got, want, **tol(bf))


@pytest.mark.parametrize("n_q,n_kv,d,hidden,batch,context", [
    (14, 2, 64, 896, 8, 4096), (14, 2, 64, 896, 1, 700), (14, 2, 64, 896, 64, 1100),
    (8, 2, 128, 1024, 3, 2000), (28, 4, 128, 200, 17, 900), (6, 3, 64, 1000, 33, 520),
    (40, 8, 128, 264, 2, 3000)])
def test_decode_attention_with_the_merge_folded_into_the_output_projection(n_q, n_kv, d, hidden,
                                                                          batch, context):
    """Decoding with split keys as two kernels (attention leaving its partial results; their
    merge inside the output projection) gives what the three kernels give, and what the plain
    attention followed by the library product gives: partial sums per slice of heads, or
    nothing left over when the step is not one the folded kernel takes."""
    page = 16
    lens = [context - 13 * i for i in range(batch)]
    per = -(-context // page)
    bf = torch.bfloat16
    qs = [rounded(rnd(1, n_q, d, seed=200 + i), bf) for i in range(batch)]
    ks = [rounded(rnd(n, n_kv, d, seed=300 + i), bf) for i, n in enumerate(lens)]
    vs = [rounded(rnd(n, n_kv, d, seed=400 + i), bf) for i, n in enumerate(lens)]
    w_o = rounded(rnd(hidden, n_q * d, seed=9, scale=0.05), bf)
    k_cache = torch.zeros(batch * per, n_kv, page, d, dtype=bf)
    v_cache = torch.zeros_like(k_cache)
    table = torch.zeros((batch, per), dtype=torch.int32)
    for s in range(batch):
        table[s] = torch.arange(s * per, (s + 1) * per, dtype=torch.int32)
        for pos in range(lens[s]):
            k_cache[s * per + pos // page, :, pos % page] = ks[s][pos].to(bf)
            v_cache[s * per + pos // page, :, pos % page] = vs[s][pos].to(bf)
    v_cache = v_cache.transpose(2, 3).contiguous()
    from tests.helpers import context_from_spans

    step = context_from_spans([(1, n - 1) for n in lens], DEV)
    q_flat = torch.cat([q.reshape(1, n_q * d) for q in qs]).to(bf).to(DEV)
    attended = torch.cat([plain.causal_attention(q, k, v, d ** -0.5, n - 1)
                          for q, k, v, n in zip(qs, ks, vs, lens)]).reshape(batch, n_q * d)
    start = rnd(batch, hidden, seed=77)
    want = start + rounded(attended, bf) @ w_o.T
    results = {}
    for fold in (True, False):
        h = start.clone().to(DEV)
        left = ops().attention_project(q_flat, n_q * d, k_cache.to(DEV), v_cache.to(DEV), step,
                                       table.to(DEV), n_q, n_kv, d, d ** -0.5, None,
                                       w_o.to(bf).to(DEV), None, h, fold=fold)
        if fold:
            assert left is not None and left.shape[1:] == (batch, hidden) and 1 < left.shape[0] <= 16
        results[fold] = (h + (left.sum(0) if left is not None else 0)).cpu()
    torch.testing.assert_close(results[True], want, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(results[False], want, atol=2e-2, rtol=2e-2)
    # the two paths round the merged rows to bfloat16 alike and differ in the order of sums only
    torch.testing.assert_close(results[True], results[False], atol=2e-3, rtol=2e-3)
    # steps the folded kernel does not take are refused when it is asked for by name
    prompt = context_from_spans([(5, 100)], DEV)
    with pytest.raises(RuntimeError, match="do not take the folded merge"):
        ops().attention_project(q_flat[:5].contiguous(), n_q * d, k_cache.to(DEV), v_cache.to(DEV),
                                prompt, table[:1].to(DEV), n_q, n_kv, d, d ** -0.5, None,
                                w_o.to(bf).to(DEV), None, torch.zeros(5, hidden, device=DEV), fold=True)


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "generic"), (torch.bfloat16, "mfma")])
@pytest.mark.parametrize("q_len", [1, 40])
def test_attention_over_a_very_long_context(dtype, kernel, q_len):
    """20,000 cached keys (block tables of 1,250 pages, far more than the 64 entries a
    wavefront holds at a time), a decoded token or a short portion at the end; one key far
    back is made to stand out for the last query, so it has to be found."""
    n_q, n_kv, d, page, s = 4, 2, 64, 16, 20000
    k = rounded(rnd(s, n_kv, d, seed=701), dtype)
    v = rounded(rnd(s, n_kv, d, seed=702), dtype)
    q = rounded(rnd(q_len, n_q, d, seed=703), dtype)
    far = 1234
    k[far, 0] = rounded(q[-1, 0] * 4.0, dtype)            # head 0 of the last query looks there
    v[far, 0] = 7.0
    pages = torch.randperm(1300, generator=torch.Generator().manual_seed(5)).tolist()[: -(-s // page)]
    got = run_attention([q], [k], [v], dtype, [pages], page, 1300, [s], [q_len], d ** -0.5,
                        kernel=kernel)
    want = plain.causal_attention(q, k, v, d ** -0.5, s - q_len)
    torch.testing.assert_close(got, want, **tol(dtype))
    assert got[-1, 0].mean() > 6.0                       # the far value dominates that head


def slow_attention_with_score_terms(q, k, v, scale, cap, slopes):
    """q [n_q, d] at the last position of k, v [S, n_kv, d]: softmax over
    cap * tanh(score / cap) - slope[head] * distance, written out."""
    n_q, n_kv = q.shape[0], k.shape[1]
    group = n_q // n_kv
    last = k.shape[0] - 1
    out = torch.zeros_like(q)
    for head in range(n_q):
        scores = (k[:, head // group] @ q[head]) * scale
        if cap:
            scores = cap * torch.tanh(scores / cap)
        if slopes is not None:
            scores = scores - slopes[head] * (last - torch.arange(k.shape[0])).float()
        out[head] = torch.softmax(scores, dim=0) @ v[:, head // group]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cap,with_slopes", [(5.0, False), (None, True), (3.0, True)])
def test_attention_with_a_capped_score_and_a_distance_penalty(dtype, cap, with_slopes):
    """What the reference's attention does not have and another mixer may want: the score
    bounded by cap * tanh(. / cap), and slope[head] * distance subtracted from it (a position
    encoding that lives in the score).  The float32-arithmetic kernel computes both, in
    either dtype; the matrix-core kernel refuses them."""
    n_q, n_kv, d, page = 6, 2, 32, 16
    lens = [70, 33, 5]
    slopes = torch.tensor([0.5 ** (i + 1) for i in range(n_q)]) if with_slopes else None
    qs = [rounded(rnd(1, n_q, d, seed=20 + i, scale=2.0), dtype) for i in range(len(lens))]
    ks = [rounded(rnd(n, n_kv, d, seed=30 + i, scale=2.0), dtype) for i, n in enumerate(lens)]
    vs = [rounded(rnd(n, n_kv, d, seed=40 + i), dtype) for i, n in enumerate(lens)]
    per = -(-max(lens) // page)
    k_cache = torch.zeros(len(lens) * per, n_kv, page, d, dtype=dtype)
    v_cache = torch.zeros_like(k_cache)
    table = torch.zeros((len(lens), per), dtype=torch.int32)
    for s, n in enumerate(lens):
        table[s] = torch.arange(s * per, (s + 1) * per, dtype=torch.int32)
        for pos in range(n):
            k_cache[s * per + pos // page, :, pos % page] = ks[s][pos].to(dtype)
            v_cache[s * per + pos // page, :, pos % page] = vs[s][pos].to(dtype)
    from tests.helpers import context_from_spans

    step = context_from_spans([(1, n - 1) for n in lens], DEV)
    q_flat = torch.cat([q.reshape(1, n_q * d) for q in qs]).to(dtype).to(DEV)
    args = (q_flat, n_q * d, k_cache.to(DEV), v_cache.transpose(2, 3).contiguous().to(DEV), step,
            table.to(DEV), n_q, n_kv, d, d ** -0.5, None)
    got = ops().attention(*args, score_cap=cap,
                          distance_slopes=None if slopes is None else slopes.to(DEV))
    want = torch.stack([slow_attention_with_score_terms(q[0], k, v, d ** -0.5, cap, slopes)
                        for q, k, v in zip(qs, ks, vs)])
    torch.testing.assert_close(got.float().cpu().view(-1, n_q, d), want, **tol(dtype))
    # the terms matter: without them the result is another
    bare = ops().attention(*args).float().cpu().view(-1, n_q, d)
    assert float((bare - want).abs().max()) > 10 * tol(dtype)["atol"]
    if dtype == torch.bfloat16:
        with pytest.raises(RuntimeError, match="neither cap nor bias"):
            ops().attention(*args, score_cap=cap or 1.0, kernel="mfma")


def test_attention_gqa_equals_mha_with_repeated_heads():
    n_q, n_kv, d, page, s = 6, 2, 16, 16, 37
    q, k, v = (rnd(s, h, d, seed=90 + i) for i, h in enumerate((n_q, n_kv, n_kv)))
    grouped = run_attention([q], [k], [v], torch.float32, [[1, 2, 3]], page, 8, [s], [s], 0.25)
    repeated = run_attention([q], [k.repeat_interleave(3, 1)], [v.repeat_interleave(3, 1)],
                             torch.float32, [[1, 2, 3]], page, 8, [s], [s], 0.25)
    assert torch.equal(grouped, repeated)


# ----------------------------------------------------------------------------------- sampling


def test_argmax_takes_the_lowest_index_among_equals():
    logits = rnd(5, 1003, seed=100)
    logits[2, 77] = logits[2, 900] = 50.0
    logits[4, 1002] = 60.0
    got = ops().argmax(logits.to(DEV)).cpu()
    assert got.tolist() == logits.argmax(-1).tolist()
    assert got[2] == 77 and got[4] == 1002


def test_argmax_in_two_stages_over_a_large_vocabulary():
    vocab = 151936
    logits = rnd(9, vocab, seed=103)
    logits[1, 0] = logits[1, vocab - 1] = 70.0         # equal maxima at both ends
    logits[2, 2373] = logits[2, 2374] = 70.0           # and across a stage boundary
    logits[3, vocab - 1] = 80.0
    logits[4] = -1e30
    logits[4, 77777] = -1e29
    got = ops().argmax(logits.to(DEV)).cpu().tolist()
    assert got == logits.argmax(-1).tolist()
    assert got[1] == 0 and got[2] == 2373 and got[3] == vocab - 1 and got[4] == 77777


def test_sampling_rules():
    """(reference: mercury/sampling.py:17-35)  Greedy rows take the argmax whatever top_p says;
    sampled rows follow the inverse CDF of the plain distribution for their own uniform."""
    vocab = 1003
    logits = rnd(6, vocab, seed=101, scale=2.0)
    temps = torch.tensor([0.0, 0.8, 0.8, 1.5, 1e-7, 0.8])
    top_ps = torch.tensor([0.5, 1.0, 0.9, 0.3, 1.0, 0.9])
    us = torch.tensor([0.3, 0.999, 0.5, 0.01, 0.7, 0.0])
    got = ops().sample(logits.to(DEV), temps.to(DEV), top_ps.to(DEV), us.to(DEV)).cpu().tolist()
    assert got[0] == int(logits[0].argmax())
    assert got[4] == int(logits[4].argmax())       # temperature -> 0 is the argmax
    for r in (1, 2, 3, 5):
        probs = plain.sampling_distribution(logits[r], float(temps[r]), float(top_ps[r]))
        want = plain.inverse_cdf_draw(probs, float(us[r]))
        assert probs[got[r]] > 0, "drew a token outside the nucleus"
        if got[r] != want:  # only a rounding of the cumulative sum may move the draw
            cum = probs.double().cumsum(-1)
            lo, hi = sorted((got[r], want))
            assert abs(float(cum[hi - 1] - float(us[r]))) < 1e-5 or float(cum[hi] - cum[lo]) < 1e-5


@pytest.mark.parametrize("vocab", [50, 1003, 151936])
def test_sampling_without_a_nucleus_over_many_workgroups(vocab):
    """With no row restricting its nucleus the vocabulary is shared out over 64 workgroups per
    row: the same draws as the one-workgroup kernel told that every top_p is 1, greedy rows
    and tiny temperatures included."""
    rows = 9
    logits = rnd(rows, vocab, seed=103, scale=2.5)
    logits[3, vocab - 1] = 40.0                  # all the mass in the last stretch
    logits[4, 0] = 40.0                          # ... or in the first
    temps = torch.tensor([0.8, 0.0, 1.3, 0.7, 0.7, 1e-7, 0.8, 0.8, 2.0])
    us = torch.tensor([0.5, 0.3, 0.999999, 0.2, 0.9, 0.4, 0.0, 0.25, 0.75])
    ones = torch.ones(rows)
    fast = ops().sample(logits.to(DEV), temps.to(DEV), None, us.to(DEV)).cpu().tolist()
    slow = ops().sample(logits.to(DEV), temps.to(DEV), ones.to(DEV), us.to(DEV)).cpu().tolist()
    assert fast[1] == int(logits[1].argmax()) and fast[5] == int(logits[5].argmax())
    assert fast[3] == vocab - 1 and fast[4] == 0
    for r in range(rows):
        if fast[r] == slow[r] or temps[r] <= 0:
            continue
        # only a rounding of the cumulative sum may move the draw: both tokens are where the
        # running mass crosses u
        probs = plain.sampling_distribution(logits[r], float(temps[r]), 1.0)
        cum = probs.double().cumsum(-1)
        lo, hi = sorted((fast[r], slow[r]))
        assert float(cum[hi] - cum[lo]) < 1e-5 or abs(float(cum[hi - 1]) - float(us[r])) < 1e-5


@pytest.mark.parametrize("vocab", [1003, 151936])
def test_nucleus_over_a_large_vocabulary(vocab):
    """The nucleus is found by histograms of the probability mass over the bits of the
    probabilities: for several top_p, temperatures and uniforms per row the draw is the plain
    implementation's (or its neighbour where a rounding of the running sum decides), and never
    a token outside the plain nucleus."""
    top_ps = [0.05, 0.5, 0.9, 0.999, 0.5, 1e-6, 0.9, 0.9]
    temps = [0.8, 0.8, 1.3, 0.6, 2.0, 0.8, 0.8, 0.8]
    us = [0.0, 0.37, 0.81, 0.999, 0.5, 0.9, 0.25, 0.75]
    rows = len(us)
    logits = rnd(rows, vocab, seed=104, scale=2.0)
    logits[6, :] = 0.0
    logits[6, 100:700] = 12.0                      # a plateau with nearly all the mass, across the edge: kept together
    logits[7, :] = 1.25                            # all equal: everything is kept
    got = ops().sample(logits.to(DEV), torch.tensor(temps).to(DEV), torch.tensor(top_ps).to(DEV),
                       torch.tensor(us).to(DEV)).cpu().tolist()
    assert got[5] == int(logits[5].argmax())       # a nucleus of one token
    assert 100 <= got[6] < 700
    assert got[7] == min(vocab - 1, int(0.75 * vocab))
    for r in range(6):      # rows 6 and 7 are ties, which a sort cuts anywhere and we keep whole
        probs = plain.sampling_distribution(logits[r], temps[r], top_ps[r])
        want = plain.inverse_cdf_draw(probs, us[r])
        assert probs[got[r]] > 0, f"row {r} drew a token outside the nucleus"
        if got[r] != want:
            cum = probs.double().cumsum(-1)
            lo, hi = sorted((got[r], want))
            assert float(cum[hi] - cum[lo]) < 1e-4 or abs(float(cum[hi - 1]) - us[r]) < 1e-4, r


def test_sampling_frequencies_follow_the_distribution():
    vocab = 50
    logits = rnd(1, vocab, seed=102, scale=1.5).repeat(4000, 1)
    g = torch.Generator().manual_seed(5)
    us = torch.rand(4000, generator=g)
    temps, top_ps = torch.full((4000,), 0.7), torch.full((4000,), 0.8)
    got = ops().sample(logits.to(DEV), temps.to(DEV), top_ps.to(DEV), us.to(DEV)).cpu()
    probs = plain.sampling_distribution(logits[0], 0.7, 0.8)
    freq = torch.bincount(got.long(), minlength=vocab).float() / 4000
    assert torch.all(freq[probs == 0] == 0)
    assert (freq - probs).abs().max() < 0.03
    # the crossing token stays: the kept mass reaches top_p
    full = torch.softmax(logits[0] / 0.7, -1)
    assert full[probs > 0].sum() >= 0.8

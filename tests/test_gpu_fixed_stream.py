"""Steps of a few tokens keep the residual stream in fixed point (64-bit integers in units of
2^-32 that projections add into with integer atomics, the norms folded into the projections
behind them): each kernel of that path alone against the kernel it replaces and against plain
arithmetic, at other sizes than the engine's; then whole models with the path on, off and
forced on where no kernel folds anything, against the plain implementation
(the residual sum and the norm's formula: /root/reference mercury/model/qwen2.py:27-31, 107-117)."""

from __future__ import annotations

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain
from tests.test_gpu_replay import Case, check, entry

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF = torch.bfloat16
UNIT = 2.0 ** 32


def libs():
    from mercury_amd.kernels import lib

    return lib, lib.load("core"), lib.load("mfma")


def stream():
    return torch.cuda.current_stream().cuda_stream


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def to_fixed(h: torch.Tensor) -> torch.Tensor:
    return (h.double() * UNIT).round().long()


def from_fixed(a: torch.Tensor) -> torch.Tensor:
    return (a.double() / UNIT).float()


@pytest.mark.parametrize("hidden", [8, 168, 896, 1000, 4100])
def test_the_stream_starts_from_the_embedding_and_its_norm_is_the_norm(hidden):
    lib, core, _ = libs()
    table = rnd(301, hidden, seed=1).to(BF).to(DEV)
    ids = torch.tensor([0, 300, 5, 5, 77], dtype=torch.int32, device=DEV)
    h64 = torch.zeros(5, hidden, dtype=torch.long, device=DEV)
    lib.check(core, core.mk_embed_fixed(ids.data_ptr(), table.data_ptr(), 1, h64.data_ptr(), 5, hidden,
                                        301, 1.0, stream()), "embed_fixed")
    assert torch.equal(from_fixed(h64), table[ids.long()].float())     # bfloat16 values are exact
    # values of every size a stream holds, beside the float32 stream's own norm
    h = rnd(5, hidden, seed=2) * torch.logspace(-4, 3, hidden)
    h64 = to_fixed(h).to(DEV)
    h_d = from_fixed(h64).to(DEV)               # the float32 values the fixed ones round to
    w = (1 + 0.1 * rnd(hidden, seed=3)).to(BF).to(DEV)
    rows = torch.tensor([4, 0, 2], dtype=torch.int32, device=DEV)
    for selected in (None, rows):
        n = 5 if selected is None else 3
        got = torch.zeros(n, hidden, dtype=BF, device=DEV)
        want = torch.zeros_like(got)
        at = 0 if selected is None else selected.data_ptr()
        lib.check(core, core.mk_rmsnorm_fixed(h64.data_ptr(), w.data_ptr(), 1, 1e-6, at, got.data_ptr(),
                                              1, n, hidden, stream()), "rmsnorm_fixed")
        lib.check(core, core.mk_rmsnorm(h_d.data_ptr(), 0, 0, 0, w.data_ptr(), 1, 1e-6, at,
                                        want.data_ptr(), 1, n, hidden, stream()), "rmsnorm")
        # the same formula and roundings; the sums of squares are added up in another order
        torch.testing.assert_close(got.float(), want.float(), atol=0, rtol=2.0 ** -7)
        assert (got != want).float().mean() < 0.01
    ref = plain.rms_norm(h_d.cpu(), w.float().cpu(), 1e-6)[0]
    torch.testing.assert_close(got.float().cpu(), ref[rows.cpu().long()], atol=1e-6, rtol=2.0 ** -6)


@pytest.mark.parametrize("m,n,k", [(1, 896, 4864), (8, 896, 896), (3, 1003, 168), (16, 130, 264), (5, 64, 2048)])
@pytest.mark.parametrize("bias_dtype", [None, torch.float32, BF])
def test_a_projection_adds_into_the_fixed_stream(m, n, k, bias_dtype):
    lib, core, mfma = libs()
    x = rnd(m, k, seed=11).to(BF)
    w = rnd(n, k, seed=12, scale=0.1).to(BF)
    h = rnd(m, n, seed=13, scale=3.0)
    want = h.double() + x.double() @ w.double().T
    x_d, w_d = x.to(DEV), w.to(DEV)
    bias_at, code = 0, 0
    if bias_dtype is not None:
        bias = rnd(n, seed=14).to(bias_dtype).to(DEV)
        want = want + bias.double().cpu()
        bias_at, code = bias.data_ptr(), 1 if bias_dtype == BF else 0
    slices = mfma.mk_linear_skinny_slices(m, n, k)
    runs = []
    for count in sorted({1, slices, min(3, (k + 127) // 128)}):
        per = -(-((k + 127) // 128) // count)
        if per * (count - 1) >= (k + 127) // 128:
            continue                              # a count the steps do not divide into
        h64 = to_fixed(h).to(DEV)
        lib.check(mfma, mfma.mk_linear_skinny_fixed(x_d.data_ptr(), w_d.data_ptr(), bias_at,
                                                    code, h64.data_ptr(), m, n, k, count, stream()),
                  "linear_skinny_fixed")
        runs.append(h64.cpu())
        # float32 sums of bfloat16 products over K, then one rounding to 2^-32
        torch.testing.assert_close(from_fixed(h64).cpu().double(), want, atol=3e-5 * k ** 0.5, rtol=1e-5)
    again = to_fixed(h).to(DEV)
    lib.check(mfma, mfma.mk_linear_skinny_fixed(x_d.data_ptr(), w_d.data_ptr(), bias_at, code,
                                                again.data_ptr(), m, n, k, count, stream()), "again")
    assert torch.equal(again.cpu(), runs[-1])     # whatever order the slices' atomics arrive in
    # float32 partial sums owed to the stream
    parts = rnd(3, m, n, seed=15).to(DEV)
    h64 = to_fixed(h).to(DEV)
    lib.check(core, core.mk_fixed_add(h64.data_ptr(), parts.data_ptr(), 3, m * n, m * n, stream()), "fixed_add")
    torch.testing.assert_close(from_fixed(h64).cpu().double(), h.double() + parts.double().sum(0).cpu(),
                               atol=1e-6, rtol=1e-6)
    with pytest.raises(lib.KernelLibraryError, match="outside 1..16"):
        lib.check(mfma, mfma.mk_linear_skinny_fixed(x_d.data_ptr(), w_d.data_ptr(), 0, 0,
                                                    h64.data_ptr(), 17, n, k, 1, stream()), "too many rows")


@pytest.mark.parametrize("m,k,inter", [(1, 896, 4864), (8, 896, 4864), (3, 168, 410), (16, 64, 176),
                                       (4, 1024, 96), (13, 1000, 24), (2, 1536, 200), (4, 2048, 48),
                                       (7, 1032, 64), (11, 2000, 32), (16, 256, 704), (12, 896, 64),
                                       (8, 256, 704), (5, 1000, 4864), (6, 896, 410), (16, 1024, 704)])
def test_the_gated_projection_makes_its_own_normalised_rows(m, k, inter):
    lib, core, mfma = libs()
    h = rnd(m, k, seed=21) * torch.logspace(-3, 2, k)
    h64 = to_fixed(h).to(DEV)
    g = (1 + 0.1 * rnd(k, seed=22)).to(BF).to(DEV)
    w = rnd(2 * inter, k, seed=23, scale=0.05).to(BF).to(DEV)
    x = torch.zeros(m, k, dtype=BF, device=DEV)
    lib.check(core, core.mk_rmsnorm_fixed(h64.data_ptr(), g.data_ptr(), 1, 1e-5, 0, x.data_ptr(), 1, m, k,
                                          stream()), "rmsnorm_fixed")
    want = torch.zeros(m, inter, dtype=BF, device=DEV)
    got = torch.zeros_like(want)
    lib.check(mfma, mfma.mk_gated_skinny(x.data_ptr(), w.data_ptr(), want.data_ptr(), m, inter, k, stream()),
              "gated_skinny")
    for weight_dtype in (1, 0):
        weight = g if weight_dtype else g.float()
        lib.check(mfma, mfma.mk_gated_skinny_normed(h64.data_ptr(), weight.data_ptr(), weight_dtype, 1e-5,
                                                    w.data_ptr(), got.data_ptr(), m, inter, k, stream()),
                  "gated_skinny_normed")
        # the rows it makes differ from the norm kernel's by the order of the sum of squares,
        # its products by how many wavefronts share K: one rounding here and there
        scale = float(want.float().abs().max())
        torch.testing.assert_close(got.float(), want.float(), atol=scale * 2.0 ** -7, rtol=2.0 ** -6)
        assert (got != want).float().mean() < 0.02
        for _ in range(4):                      # the same bits run after run
            again = torch.full_like(got, 3.0)
            lib.check(mfma, mfma.mk_gated_skinny_normed(h64.data_ptr(), weight.data_ptr(), weight_dtype, 1e-5,
                                                        w.data_ptr(), again.data_ptr(), m, inter, k, stream()),
                      "gated_skinny_normed")
            assert torch.equal(again, got)
    # and from the formulas
    xn = plain.rms_norm(from_fixed(h64).cpu(), g.float().cpu(), 1e-5)[0].to(BF).float()
    y = xn @ w.float().cpu().T
    ref = torch.nn.functional.silu(y[:, :inter].to(BF).float()).to(BF).float() * y[:, inter:].to(BF).float()
    torch.testing.assert_close(got.float().cpu(), ref, atol=float(ref.abs().max()) * 2.0 ** -6, rtol=2.0 ** -5)


@pytest.mark.parametrize("n_q,n_kv,d,page,k,m", [(14, 2, 64, 16, 896, 8), (6, 1, 32, 8, 168, 1),
                                                 (4, 4, 128, 32, 264, 16), (3, 1, 96, 16, 72, 5),
                                                 (2, 2, 64, 16, 1024, 3), (2, 1, 128, 16, 1536, 4),
                                                 (1, 1, 64, 16, 2048, 9), (3, 1, 32, 8, 1096, 2), (8, 1, 32, 8, 256, 16),
                                                 (14, 2, 64, 16, 896, 13)])
def test_the_qkv_projection_makes_its_own_normalised_rows(n_q, n_kv, d, page, k, m):
    """Against the same kernel on rows the norm kernel made: the same wavefronts take the same
    k-steps, so wherever the rows agree the results are the same bits; rotation, bias and the
    cache write are the kernel's own either way (tested with it)."""
    lib, core, mfma = libs()
    width = (n_q + 2 * n_kv) * d
    h64 = to_fixed(rnd(m, k, seed=31) * torch.logspace(-2, 2, k)).to(DEV)
    g = (1 + 0.1 * rnd(k, seed=32)).to(BF).to(DEV)
    w = rnd(width, k, seed=33, scale=0.05).to(BF).to(DEV)
    bias = rnd(width, seed=34).to(BF).to(DEV)
    half = d // 2
    angles = torch.arange(8 * page).float()[:, None] * (10000.0 ** (-torch.arange(half).float() / half))[None]
    cos, sin = angles.cos().contiguous().to(DEV), angles.sin().contiguous().to(DEV)
    positions = torch.tensor([(page - 1 + 3 * i) % (8 * page) for i in range(m)], dtype=torch.int32, device=DEV)
    seq = torch.tensor([i % 3 for i in range(m)], dtype=torch.int32, device=DEV)
    table = torch.arange(1, 25, dtype=torch.int32).view(3, 8).contiguous().to(DEV)
    x = torch.zeros(m, k, dtype=BF, device=DEV)
    lib.check(core, core.mk_rmsnorm_fixed(h64.data_ptr(), g.data_ptr(), 1, 1e-6, 0, x.data_ptr(), 1, m, k,
                                          stream()), "rmsnorm_fixed")
    out = []
    for folded in (False, True):
        kc = torch.zeros(32, n_kv, page, d, dtype=BF, device=DEV)
        vc = torch.zeros(32, n_kv, d, page, dtype=BF, device=DEV)
        q = torch.zeros(m, n_q * d, dtype=BF, device=DEV)
        tail = (w.data_ptr(), bias.data_ptr(), 1, q.data_ptr(), cos.data_ptr(), sin.data_ptr(), 8 * page,
                positions.data_ptr(), seq.data_ptr(), table.data_ptr(), 8, kc.data_ptr(), vc.data_ptr(), page,
                n_q, n_kv, d, 1, m, k, stream())
        if folded:
            lib.check(mfma, mfma.mk_qkv_skinny_normed(h64.data_ptr(), g.data_ptr(), 1, 1e-6, *tail), "normed")
        else:
            lib.check(mfma, mfma.mk_qkv_skinny(x.data_ptr(), *tail), "qkv_skinny")
        out.append((q, kc, vc))
    for a, b in zip(out[0], out[1]):
        scale = float(a.float().abs().max())
        torch.testing.assert_close(b.float(), a.float(), atol=scale * 2.0 ** -7, rtol=2.0 ** -6)
        assert (a != b).float().mean() < 0.02
        assert (a != 0).eq(b != 0).all() and a.abs().sum() > 0


def test_rows_too_wide_or_too_many_are_refused():
    lib, core, mfma = libs()
    # a lane holds at most 16 pairs of a row; 16 rows of LDS leave room for 1,528 values each
    assert mfma.mk_skinny_normed_max_k(8) == 2048 and mfma.mk_skinny_normed_max_k(16) == 1528
    assert mfma.mk_skinny_normed_max_k(17) == 0
    h64 = torch.zeros(16, 2056, dtype=torch.long, device=DEV)
    g = torch.ones(2056, dtype=BF, device=DEV)
    w = torch.zeros(64, 2056, dtype=BF, device=DEV)
    act = torch.zeros(16, 32, dtype=BF, device=DEV)
    for rows, width in ((16, 2048), (2, 2056)):
        with pytest.raises(lib.KernelLibraryError, match="more than its workgroups hold"):
            lib.check(mfma, mfma.mk_gated_skinny_normed(h64.data_ptr(), g.data_ptr(), 1, 1e-6, w.data_ptr(),
                                                        act.data_ptr(), rows, 32, width, stream()), "too wide")
    with pytest.raises(lib.KernelLibraryError, match="more than its workgroups hold"):
        lib.check(mfma, mfma.mk_gated_skinny_normed(h64.data_ptr(), g.data_ptr(), 1, 1e-6, w.data_ptr(),
                                                    act.data_ptr(), 17, 32, 64, stream()), "too many")
    with pytest.raises(lib.KernelLibraryError, match="16-byte aligned"):
        lib.check(mfma, mfma.mk_gated_skinny_normed(h64.data_ptr() + 8, g.data_ptr(), 1, 1e-6, w.data_ptr(),
                                                    act.data_ptr(), 2, 32, 64, stream()), "misaligned")


# ---- whole models


@pytest.fixture
def limit():
    from mercury_amd.hostcore import core

    before = core.set_fixed_stream_limit(-1)

    def set_to(n):
        core.set_fixed_stream_limit(n)

    yield set_to
    core.set_fixed_stream_limit(before)


@pytest.mark.parametrize("name,page", [("S64", 16), ("S128", 32), ("A", 16)])
def test_decoding_with_the_stream_in_fixed_point_and_without(name, page, limit):
    """The same requests decoded in steps of 1, 3 and 8 tokens with the path on (the kernels'
    own rule) and off: both within what bfloat16 costs the plain implementation, and closer
    to each other than either has to be to it."""
    case = Case(name, page)
    keys = ("a", "b", "c")
    got = {}
    for mode, n in (("fixed", -1), ("float", 0)):
        limit(n)
        s = case.session("bfloat16", 1024)
        assert s.runner.program.fixed_stream(1) == (mode == "fixed")
        assert s.runner.program.fixed_stream(8) == (mode == "fixed") and not s.runner.program.fixed_stream(9)
        rows = {k: [] for k in keys}
        for k in keys:                                        # most of each prompt whole
            rows[k].append(s.step([entry(k, case.reqs[k][:40])], []))
        for at in range(40, 72):                              # then 3 sequences a token each
            rows_now = s.step([entry(k, case.reqs[k][at:at + 1]) for k in keys], [])
            for i, k in enumerate(keys):
                rows[k].append(rows_now[i:i + 1])
        rows["a"].append(s.step([entry("a", case.reqs["a"][72:80])], []))     # a portion of 8
        rows["a"].append(s.step([entry("a", case.reqs["a"][80:81])], []))     # one alone
        s.step([], list(keys))
        assert s.manager.leaked_pages() == 0
        got[mode] = {k: torch.cat(v) for k, v in rows.items()}
        for k in keys:
            case.check(got[mode][k], k, "bfloat16", f"{mode} stream", rows=slice(0, got[mode][k].shape[0]))
    for k in keys:
        apart = float((got["fixed"][k] - got["float"][k]).abs().max())
        assert apart <= case.cost[k], (k, apart, case.cost[k])


def test_a_model_1536_wide_decodes_in_fixed_point_up_to_four_tokens(limit):
    """Rows of more than 1,024 values take the projections' instantiation of sixteen pairs a
    lane, and the rule stops at four tokens there."""
    from tests.test_gpu_replay_bench_sizes import folder_for, session

    limit(-1)
    folder = folder_for("S128", hidden_size=1536, num_attention_heads=12, intermediate_size=1288,
                        vocab_size=1003)
    weights, cfg = helpers.plain_model(folder)
    tokens = helpers.random_tokens(cfg["vocab_size"], 90, seed=5)
    want = plain.forward_logits(weights, cfg, tokens)
    from tests.test_gpu_replay import bf16_cost

    cost = bf16_cost(folder, cfg, tokens, want)
    s = session(folder, "bfloat16", 256, 32)
    assert s.runner.program.fixed_stream(4) and not s.runner.program.fixed_stream(5)
    rows, done = [], 0
    for size in (50, 1, 1, 4, 3, 1, 2, 5, 1, 4, 1, 8, 1, 1, 4, 3):
        rows.append(s.step([entry("x", tokens[done:done + size])], []))
        done += size
    assert done == len(tokens)
    check(torch.cat(rows), want, "bfloat16", "1536 wide", cost)
    s.step([], ["x"])
    assert s.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 8), ("S128", 32)])
def test_the_stream_in_fixed_point_where_no_kernel_folds_anything(name, page, dtype, limit):
    """Forced on for steps of up to 16 tokens, in float32 and at widths and row counts the
    norm-folding projections do not take: the norm kernel on the fixed stream, projections
    into a buffer and that added to the stream."""
    limit(16)
    case = Case(name, page)
    s = case.session(dtype, 512)
    assert s.runner.program.fixed_stream(16) and not s.runner.program.fixed_stream(17)
    for key in ("d", "f"):
        tokens = case.reqs[key]
        rows, done = [], 0
        for size in (16, 7, 2, 9, 1, 1, 12):                  # portions of at most 16 tokens
            part = tokens[done:done + size]
            if not part:
                break
            rows.append(s.step([entry(key, part)], []))
            done += len(part)
        s.step([], [key])
        case.check(torch.cat(rows), key, dtype, "forced fixed stream", rows=slice(0, done))
    assert s.manager.leaked_pages() == 0

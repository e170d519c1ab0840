"""Pins of the plain implementation beside the reference's text: vectors the reference's own
tests hold, special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake fails it."""

from __future__ import annotations

import math

import torch

from tests import helpers
from tests.plain import qwen2_plain as plain


def test_rotate_half_vector():
    """(reference: tests/test_attention.py:177-179)"""
    assert torch.equal(plain.rotate_half(torch.tensor([[1.0, 2.0, 3.0, 4.0]])),
                       torch.tensor([[-3.0, -4.0, 1.0, 2.0]]))


def test_rotary_table_from_libm_and_identity_at_zero():
    cos, sin = plain.rotary_table(8, [0, 1, 7], 10000.0)
    assert torch.equal(cos[0], torch.ones(8)) and torch.equal(sin[0], torch.zeros(8))
    for row, pos in ((1, 1), (2, 7)):
        for j in range(4):
            angle = pos * 10000.0 ** (-2 * j / 8)
            assert abs(cos[row, j] - math.cos(angle)) < 1e-6 and abs(sin[row, j + 4] - math.sin(angle)) < 1e-6


def test_rotary_keeps_pair_norms_and_depends_on_distance_only():
    """(reference: tests/test_attention.py:182-197)"""
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(1, 1, 8, generator=g), torch.randn(1, 1, 8, generator=g)
    dots = []
    for pos in (3, 9):
        cos, sin = plain.rotary_table(8, [pos], 10000.0)
        qa, ka = plain.apply_rotary(q, k, cos, sin)
        dots.append(float((qa * ka).sum()))
        pairs = qa[0, 0, :4] ** 2 + qa[0, 0, 4:] ** 2
        torch.testing.assert_close(pairs, q[0, 0, :4] ** 2 + q[0, 0, 4:] ** 2)
    assert abs(dots[0] - dots[1]) < 1e-5
    cos_q, sin_q = plain.rotary_table(8, [5], 10000.0)
    cos_k, sin_k = plain.rotary_table(8, [2], 10000.0)
    fwd = float((plain.apply_rotary(q, q, cos_q, sin_q)[0] * plain.apply_rotary(k, k, cos_k, sin_k)[1]).sum())
    bwd = float((plain.apply_rotary(q, q, cos_k, sin_k)[0] * plain.apply_rotary(k, k, cos_q, sin_q)[1]).sum())
    assert abs(fwd - bwd) > 1e-3          # a sign error in the rotation would make these equal


def test_rms_norm_is_the_library_routine_with_eps_inside_the_root():
    g = torch.Generator().manual_seed(1)
    x, w, r = torch.randn(5, 64, generator=g), torch.randn(64, generator=g), torch.randn(5, 64, generator=g)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6)[0], torch.nn.functional.rms_norm(x, (64,), w, 1e-6))
    out, summed = plain.rms_norm(x, w, 1e-6, residual=r)
    assert torch.equal(summed, x + r)
    torch.testing.assert_close(out, torch.nn.functional.rms_norm(x + r, (64,), w, 1e-6))
    c = torch.full((1, 16), 3.0)
    torch.testing.assert_close(plain.rms_norm(c, torch.ones(16), 0.5)[0],
                               torch.full((1, 16), 3.0 / math.sqrt(9.5)))
    assert torch.equal(plain.rms_norm(torch.zeros(1, 16), torch.ones(16), 1e-6)[0], torch.zeros(1, 16))


def test_attention_reduces_to_the_library_routine_and_to_means():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(12, h, 8, generator=g) for h in (4, 2, 2))
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(2, 1).transpose(0, 1)[None],
        v.repeat_interleave(2, 1).transpose(0, 1)[None], is_causal=True, scale=0.3)[0].transpose(0, 1)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3), lib, atol=1e-6, rtol=1e-5)
    # a suffix over a prefix equals the rows of the whole (reference: tests/test_attention.py:84-102)
    torch.testing.assert_close(plain.causal_attention(q[8:], k, v, 0.3, query_offset=8),
                               plain.causal_attention(q, k, v, 0.3)[8:])
    # grouping: head h reads kv head h // 2, not h % 2
    one_hot_v = torch.zeros(12, 2, 8)
    one_hot_v[:, 1] = 1.0
    out = plain.causal_attention(q, k, one_hot_v, 0.3)
    assert torch.equal(out[:, :2], torch.zeros(12, 2, 8)) and torch.allclose(out[:, 2:], torch.ones(12, 2, 8))
    # equal scores -> running mean; a window of one -> the token's own value
    flat = plain.causal_attention(q, torch.zeros_like(k), v, 0.3)
    torch.testing.assert_close(flat[5, 0], v[:6, 0].mean(0))
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=1)[:, 0], v[:, 0])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=12), plain.causal_attention(q, k, v, 0.3))


def test_mlp_and_silu():
    g = torch.Generator().manual_seed(3)
    x, wg, wu, wd = (torch.randn(*s, generator=g) for s in ((4, 16), (24, 16), (24, 16), (16, 24)))
    F = torch.nn.functional
    torch.testing.assert_close(plain.gated_mlp(x, wg, wu, wd),
                               F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd))
    assert float(plain.silu(torch.tensor(0.0))) == 0.0


def test_slot_mapping_vectors():
    """(reference: tests/test_attention.py:38-51)"""
    blocks = [5, 9, 2]
    assert [plain.slot_mapping(blocks, p, p + 1, 16)[0] for p in (15, 16, 17, 31, 32)] == \
        [5 * 16 + 15, 9 * 16, 9 * 16 + 1, 9 * 16 + 15, 2 * 16]
    slots = plain.slot_mapping([7, 1], 0, 20, 16)
    assert slots[:16] == [7 * 16 + i for i in range(16)] and slots[16:] == [16 + i for i in range(4)]


def _library_attention(x, w, prefix, cfg, cos, sin):
    """The attention layer from library routines only: `F.linear`, the rotation (pinned
    above), and `F.scaled_dot_product_attention` with its default scale, which is
    1 / sqrt(head size): the reference's `head_dim ** -0.5` (mercury/model/qwen2.py:54)."""
    F = torch.nn.functional
    n_q, n_kv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    t = x.shape[0]
    q = F.linear(x, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"]).view(t, n_q, d)
    k = F.linear(x, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"]).view(t, n_kv, d)
    v = F.linear(x, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"]).view(t, n_kv, d)
    q, k = plain.apply_rotary(q, k, cos, sin)
    k, v = (z.repeat_interleave(n_q // n_kv, 1) for z in (k, v))
    out = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                         v.transpose(0, 1)[None], is_causal=True)[0]
    return F.linear(out.transpose(0, 1).reshape(t, n_q * d), w[prefix + "o_proj.weight"])


def test_the_score_scale_is_the_library_default():
    """A scale of 1, of 1/d or a missing scale fails this; so does a bias on the output
    projection or none on q/k/v."""
    for name in ("A", "C"):
        w, cfg = helpers.plain_model(helpers.model_folder(name, std=0.3))
        g = torch.Generator().manual_seed(4)
        x = torch.randn(19, cfg["hidden_size"], generator=g)
        cos, sin = plain.rotary_table(cfg["head_dim"], range(19), cfg["rope_theta"])
        prefix = "model.layers.0.self_attn."
        want = _library_attention(x, w, prefix, cfg, cos, sin)
        got = plain.attention_layer(x, w, prefix, cfg, cos, sin)
        torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-4)


def test_the_layers_are_pre_norm_around_a_running_sum():
    """The reference carries `residual` through its norms (mercury/model/qwen2.py:82-94,
    :110-114).  Written out, that is h <- h + attention(norm(h)); h <- h + mlp(norm(h)) from
    h = embedding, and norm(h) at the end: composed here from library routines
    (`F.rms_norm`, `F.linear`, `F.silu`, library attention).  A norm after the sum instead of
    before it, a forgotten sum, or the final norm applied to the last layer's output alone
    fails this."""
    F = torch.nn.functional
    for name in ("A", "B", "C"):
        w, cfg = helpers.plain_model(helpers.model_folder(name, std=0.2))
        eps, width = cfg["rms_norm_eps"], (cfg["hidden_size"],)
        tokens = helpers.random_tokens(cfg["vocab_size"], 23, seed=8)
        cos, sin = plain.rotary_table(cfg["head_dim"], range(len(tokens)), cfg["rope_theta"])
        h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            a = F.rms_norm(h, width, w[p + "input_layernorm.weight"], eps)
            h = h + _library_attention(a, w, p + "self_attn.", cfg, cos, sin)
            m = F.rms_norm(h, width, w[p + "post_attention_layernorm.weight"], eps)
            h = h + F.linear(F.silu(F.linear(m, w[p + "mlp.gate_proj.weight"]))
                             * F.linear(m, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
        y = F.rms_norm(h, width, w["model.norm.weight"], eps)
        head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
        want = F.linear(y, head)
        got = plain.forward_logits(w, cfg, tokens)
        assert want.abs().max() > 0.5       # weights wide enough that every part matters
        torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-4)
        # and every part does matter: without the sums the logits are others
        for drop in ("self_attn.o_proj.weight", "mlp.down_proj.weight"):
            cut = {k: (torch.zeros_like(v) if k.endswith(drop) else v) for k, v in w.items()}
            assert (plain.forward_logits(cut, cfg, tokens) - got).abs().max() > 1e-2


def test_bfloat16_run_rounds_where_the_reference_rounds():
    """Read in bfloat16 the plain implementation keeps every tensor in bfloat16 (the
    reference's casts, mercury/model/qwen2.py:27-31, mercury/model/rope.py:46-47) and stays
    close to the float32 run: a fraction of a per cent of the logits' range, not more."""
    folder = helpers.model_folder("B")
    w, cfg = helpers.plain_model(folder)
    tokens = helpers.random_tokens(cfg["vocab_size"], 60, seed=3)
    exact = plain.forward_logits(w, cfg, tokens)
    rounded = plain.forward_logits(plain.read_weights(folder, torch.bfloat16), cfg, tokens)
    assert rounded.dtype == torch.bfloat16
    gap = float((rounded.float() - exact).abs().max())
    assert 0 < gap < 0.03 * float(exact.abs().max())
    normed, summed = plain.rms_norm(torch.full((1, 8), 3.0, dtype=torch.bfloat16),
                                    torch.ones(8, dtype=torch.bfloat16), 1e-6,
                                    residual=torch.full((1, 8), 0.0078125, dtype=torch.bfloat16))
    assert summed.dtype == normed.dtype == torch.bfloat16
    assert float(summed[0, 0]) == 3.0       # the sum itself is rounded to bfloat16 first


def test_whole_model_invariants():
    folder = helpers.model_folder("B")
    w, cfg = helpers.plain_model(folder)
    tokens = helpers.random_tokens(cfg["vocab_size"], 20, seed=1)
    logits = plain.forward_logits(w, cfg, tokens)
    # causal: a later token does not change earlier logits
    changed = list(tokens)
    changed[-1] = (changed[-1] + 1) % cfg["vocab_size"]
    torch.testing.assert_close(plain.forward_logits(w, cfg, changed)[:-1], logits[:-1])
    # shifting every position changes nothing (only distances count)
    torch.testing.assert_close(plain.forward_logits(w, cfg, tokens, first_position=50), logits,
                               atol=3e-5, rtol=1e-4)
    # the q/k/v biases matter (they are zero in no layer of the random model)
    no_bias = {k: (torch.zeros_like(v) if k.endswith("_proj.bias") else v) for k, v in w.items()}
    assert (plain.forward_logits(no_bias, cfg, tokens) - logits).abs().max() > 1e-3
    # untied head: logits use lm_head, not the embedding
    swapped = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"]})
    assert (plain.forward_logits(swapped, cfg, tokens) - logits).abs().max() > 1e-3
    assert plain.kv_bytes_per_token(cfg, 2) == 2 * 3 * 1 * 32 * 2
    # float64 agrees with float32 to float32 rounding
    w64, _ = plain.read_weights(folder, torch.float64), None
    torch.testing.assert_close(plain.forward_logits(w64, cfg, tokens).float(), logits, atol=2e-5, rtol=1e-4)


def test_sampling_rules():
    """(reference: mercury/sampling.py:6-35)"""
    probs = torch.tensor([0.5, 0.3, 0.15, 0.05])
    kept = lambda p: (plain.nucleus_mask(probs, p) > 0).tolist()
    assert kept(0.6) == [True, True, False, False]        # the crossing token stays
    assert kept(0.5) == [True, True, False, False]
    assert kept(0.49) == [True, False, False, False]
    assert torch.equal(plain.nucleus_mask(probs, 0.6)[:2], probs[:2])
    logits = torch.log(probs)
    torch.testing.assert_close(plain.sampling_distribution(logits, 1.0, 1.0), probs)
    torch.testing.assert_close(plain.sampling_distribution(logits, 1.0, 0.6), torch.tensor([0.625, 0.375, 0, 0]))
    sharp = plain.sampling_distribution(logits, 1e-9, 1.0)           # temperature clamps at 1e-5
    assert sharp[0] > 0.999
    assert [plain.inverse_cdf_draw(probs, u) for u in (0.0, 0.49, 0.5, 0.79, 0.81, 0.999)] == [0, 0, 1, 1, 2, 3]

"""Operation kinds registered from outside the package run inside the host core's program:
a feed-forward and a mixer with per-request state whose operations are written here, over the
kernel libraries' C entry points, beside an embedding with a scale and a head with a bias and
a cap.  And the other way round: a subclass that overrides `forward` is not lowered."""

from __future__ import annotations

import ctypes
import math

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

NAMES = {"mixer": "mixer.", "ffn": "ffn.", "norm_mixer": "norm1.", "norm_ffn": "norm2."}
SCALE, CAP = 3.0, 2.5


class SelfGateParams(ctypes.Structure):
    _fields_ = [("w_down", ctypes.c_void_p), ("half", ctypes.c_int)]


class FirstTokenParams(ctypes.Structure):
    _fields_ = [("w", ctypes.c_void_p), ("state", ctypes.c_void_p)]


def register(native: bool):
    """The toy parts and the architecture that uses them; with `native` their operations run
    inside the program, otherwise their `forward` does the same from Python."""
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.kernels import lib as kernel_lib
    from mercury_amd.kernels import ops
    from mercury_amd.parts import (Attention, DecoderModel, FeedForward, GatedMLP, Mixer, OutputHead,
                                   PreNormBlock, RMSNorm, RotaryPosition, StateSpec, TensorSpec,
                                   TokenEmbedding, op_abi, register_ffn, register_mixer)

    core_lib = kernel_lib.load("core")

    def check(code, what):
        if code:
            raise RuntimeError(f"{what}: {core_lib.mk_last_error().decode()}")

    def self_gate(params, ctx):
        """h += (silu(x[:, :half]) * x[:, half:]) Wd^T: the gating kernel, then the float32
        multiply-add projection added into the stream."""
        p = SelfGateParams.from_address(params)
        tokens = ctx.step.contents.num_tokens
        act = ctx.allocate(tokens * p.half * (2 if ctx.dtype else 4))
        if ctx.dry:
            return
        check(core_lib.mk_silu_mul(ctx.x, act, ctx.dtype, tokens, p.half, ctx.stream), "silu_mul")
        check(core_lib.mk_linear_generic(act, p.w_down, ctx.dtype, None, 0, ctx.h, 0, 1, tokens,
                                         ctx.hidden, p.half, p.half, ctx.hidden, ctx.stream), "linear")

    def first_token(params, ctx):
        """h += x_0 W^T for every token of a sequence, x_0 being the sequence's first token's
        input, kept in the sequence's state slot from the step that ran position 0."""
        p = FirstTokenParams.from_address(params)
        step = ctx.step.contents
        tokens = step.num_tokens
        rows = ctx.allocate(tokens * ctx.hidden * (2 if ctx.dtype else 4))
        if ctx.dry:
            return
        check(core_lib.mk_state_store(ctx.x, ctx.dtype, p.state, step.state_slots, step.token_seq,
                                      step.positions, 0, tokens, ctx.hidden, ctx.stream), "state_store")
        check(core_lib.mk_state_load(p.state, step.state_slots, step.token_seq, rows, ctx.dtype,
                                     tokens, ctx.hidden, ctx.stream), "state_load")
        check(core_lib.mk_linear_generic(rows, p.w, ctx.dtype, None, 0, ctx.h, 0, 1, tokens,
                                         ctx.hidden, ctx.hidden, ctx.hidden, ctx.hidden, ctx.stream),
              "linear")

    op_abi.register_python_op("test_self_gate", self_gate, op_abi.READS_X)
    op_abi.register_python_op("test_first_token", first_token, op_abi.READS_X)

    @register_ffn("test_self_gate")
    class SelfGate(FeedForward):
        graph_safe = True
        lowerable = native

        def __init__(self, hidden):
            self.hidden = hidden

        def param_specs(self):
            return {"down.weight": TensorSpec((self.hidden, self.hidden // 2))}

        def bind(self, params, dtype, device):
            self.w = params["down.weight"]

        def lower(self, program):
            program.append("test_self_gate", bytes(SelfGateParams(self.w.data_ptr(), self.hidden // 2)))

        def forward(self, x, step, accum):
            ops.linear(ops.silu_mul(x), self.w, out=accum, accumulate=True, kernel="generic")

    @register_mixer("test_first_token")
    class FirstToken(Mixer):
        graph_safe = native     # its `forward` reads the slots on the host
        lowerable = native
        lowers_state = True

        def __init__(self, hidden):
            self.hidden = hidden

        def state_spec(self):
            return StateSpec((self.hidden,), torch.float32)

        def param_specs(self):
            return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

        def bind(self, params, dtype, device):
            self.w = params["mix.weight"]

        def lower(self, program, cache, state):
            program.append("test_first_token",
                           bytes(FirstTokenParams(self.w.data_ptr(), state.data_ptr())))

        def forward(self, x, step, cache, state, accum):
            slots = step.state_slots.tolist()
            for s, (first, count, start) in enumerate(step.spans):
                if start == 0:
                    state[slots[s]] = x[first].float()
                row = state[slots[s]].to(x.dtype)
                accum[first:first + count] += (row @ self.w.T).float()

    @register_architecture("TestOpenOpsLM", Qwen2Config)
    def build(cfg):
        h, eps = cfg.hidden_size, cfg.rms_norm_eps
        attention = Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                              RotaryPosition(cfg.head_dim, cfg.rope_theta), qkv_bias=False,
                              names={"q": "wq", "k": "wk", "v": "wv", "o": "wo"})
        layers = [
            PreNormBlock(attention, SelfGate(h), RMSNorm(h, eps), RMSNorm(h, eps), NAMES),
            PreNormBlock(FirstToken(h), GatedMLP(h, cfg.intermediate_size,
                                                 names={"gate": "w1", "up": "w3", "down": "w2"}),
                         RMSNorm(h, eps), RMSNorm(h, eps), NAMES),
        ]
        return DecoderModel(
            cfg.vocab_size, h, layers, RMSNorm(h, eps), tied_head=False, layer_prefix="blocks.{}.",
            embed_name="tok.weight", norm_prefix="final.", head_name="out.weight",
            max_positions=cfg.max_position_embeddings, config=cfg,
            embedding=TokenEmbedding(cfg.vocab_size, h, scale=SCALE),
            head=OutputHead(cfg.vocab_size, h, bias=True, cap=CAP))

    return build


def slow_logits(w, cfg, tokens):
    """The toy model the slow way, from the plain parts, in the tensors' own dtype."""
    eps, d, h_size = cfg["rms_norm_eps"], cfg["head_dim"], cfg["hidden_size"]
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    dtype = w["tok.weight"].dtype
    cos, sin = plain.rotary_table(d, range(len(tokens)), cfg["rope_theta"])
    h = (w["tok.weight"][torch.tensor(tokens)].float() * SCALE)

    def norm(h, name):
        return plain.rms_norm(h.to(dtype), w[name], eps)[0]

    x = norm(h, "blocks.0.norm1.weight")
    q = (x @ w["blocks.0.mixer.wq.weight"].T).view(-1, n_q, d)
    k = (x @ w["blocks.0.mixer.wk.weight"].T).view(-1, n_kv, d)
    v = (x @ w["blocks.0.mixer.wv.weight"].T).view(-1, n_kv, d)
    q, k = plain.apply_rotary(q, k, cos.to(dtype), sin.to(dtype))
    attended = plain.causal_attention(q, k, v, d ** -0.5).reshape(len(tokens), -1)
    h = h + (attended @ w["blocks.0.mixer.wo.weight"].T).float()
    x = norm(h, "blocks.0.norm2.weight")
    half = h_size // 2
    h = h + ((plain.silu(x[:, :half]) * x[:, half:]) @ w["blocks.0.ffn.down.weight"].T).float()
    x = norm(h, "blocks.1.norm1.weight")
    h = h + (x[0] @ w["blocks.1.mixer.mix.weight"].T).float()[None, :]
    x = norm(h, "blocks.1.norm2.weight")
    h = h + plain.gated_mlp(x, w["blocks.1.ffn.w1.weight"], w["blocks.1.ffn.w3.weight"],
                            w["blocks.1.ffn.w2.weight"]).float()
    x = norm(h, "final.weight")
    logits = (x @ w["out.weight"].T).float() + w["out.bias"].float()
    return CAP * torch.tanh(logits / CAP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("native", [True, False], ids=["in-the-program", "from-python"])
def test_parts_from_outside_with_operations_of_their_own(tmp_path, native, dtype):
    from safetensors.torch import load_file

    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model

    register(native)
    config = {**helpers.TINY_A, "architectures": ["TestOpenOpsLM"], "hidden_size": 96,
              "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
              "intermediate_size": 136, "vocab_size": 301, "max_position_embeddings": 512}
    folder = write_random_model(tmp_path / "open", config, seed=4, std=0.08, dtype=torch.bfloat16)
    stored = load_file(str(folder / "model.safetensors"))
    assert "blocks.0.mixer.wq.weight" in stored and "blocks.1.ffn.w3.weight" in stored
    assert "out.bias" in stored and "tok.weight" in stored
    cfg = plain.read_config(folder)
    reqs = {"a": helpers.random_tokens(301, 75, 1), "b": helpers.random_tokens(301, 40, 2)}
    exact = {k: slow_logits({n: t.float() for n, t in stored.items()}, cfg, v) for k, v in reqs.items()}
    tol = dict(atol=2e-5, rtol=1e-4)
    if dtype == "bfloat16":
        # what bfloat16 costs the slow version itself, times the slack the replay tests use
        cost = max(float((slow_logits(stored, cfg, v) - exact[k]).abs().max()) for k, v in reqs.items())
        tol = dict(atol=1.5 * cost, rtol=0)

    s = ReplaySession(folder, dtype, 256)
    kinds = s.runner.program.kinds
    if native:
        assert "host" not in kinds and kinds.count("test_self_gate") == 1
        assert kinds.count("test_first_token") == 1, kinds
        assert s.runner.use_graphs
    else:
        assert kinds.count("host") == 2
    assert list(s.runner.states) == [1] and not s.manager.prefix_sharing

    def entry(key, part):
        return {"id": key, "tokens": part, "want": list(range(len(part)))}

    # whole
    for key, tokens in reqs.items():
        got = s.step([entry(key, tokens)], [key])
        torch.testing.assert_close(got, exact[key], **tol)
    # both requests in portions side by side, then token by token (captured graphs when native)
    done, rows = {"a": 0, "b": 0}, {"a": [], "b": []}
    sizes = [9, 2, 17, 5, 3]
    n = 0
    while any(done[k] < len(reqs[k]) for k in reqs):
        entries = []
        for i, key in enumerate(reqs):
            if done[key] >= len(reqs[key]):
                continue
            size = sizes[(n + i) % len(sizes)] if done[key] < 30 else 1
            entries.append(entry(key, reqs[key][done[key]:done[key] + size]))
        out = s.step(entries, [])
        at = 0
        for e in entries:
            rows[e["id"]].append(out[at:at + len(e["tokens"])])
            at += len(e["tokens"])
            done[e["id"]] += len(e["tokens"])
        n += 1
    for key in reqs:
        torch.testing.assert_close(torch.cat(rows[key]), exact[key], **tol)
    if native:
        assert s.runner.graphs, "the decoded tail did not go through a captured graph"
    s.step([], ["a", "b"])
    assert s.manager.leaked_pages() == 0


def test_embedding_scale_head_bias_and_cap_change_the_logits(tmp_path):
    """The three options of the embedding and head parts are not decoration: the same weights
    under a plain embedding and head give other logits, and the capped ones stay inside the
    cap."""
    from safetensors.torch import load_file

    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model

    register(True)
    config = {**helpers.TINY_A, "architectures": ["TestOpenOpsLM"], "hidden_size": 96,
              "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
              "intermediate_size": 136, "vocab_size": 301, "max_position_embeddings": 512}
    folder = write_random_model(tmp_path / "open", config, seed=4, std=0.3, dtype=torch.float32)
    tokens = helpers.random_tokens(301, 20, 3)
    got = ReplaySession(folder, "float32", 64).step(
        [{"id": "a", "tokens": tokens, "want": list(range(20))}], ["a"])
    assert float(got.abs().max()) < CAP and float(got.abs().max()) > 0.9 * CAP
    w = load_file(str(folder / "model.safetensors"))
    want = slow_logits(w, plain.read_config(folder), tokens)
    torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-4)
    assert math.isclose(SCALE, 3.0)


def test_a_position_encoding_that_lives_in_the_score(tmp_path):
    """Another position encoding, registered from outside: no rotation, but a penalty
    slope[head] * distance in the score (and a cap on the score beside it).  It describes
    itself to the kernels, so its layers stay inside the program; the slow version is written
    out here.  Only distances enter, so shifting all positions changes nothing."""
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.parts import (Attention, DecoderModel, GatedMLP, PositionDescriptor,
                                   PositionEncoding, PreNormBlock, RMSNorm, register_position)
    from mercury_amd.weights import write_random_model

    cap = 4.0

    @register_position("test_distance_penalty")
    class DistancePenalty(PositionEncoding):
        def __init__(self, heads):
            self.values = [2.0 ** -(i + 1) for i in range(heads)]
            self.slopes = None

        def prepare(self, max_positions, device):
            self.slopes = torch.tensor(self.values, dtype=torch.float32, device=device)

        def describe(self):
            return PositionDescriptor(distance_slopes=self.slopes)

    @register_architecture("TestDistanceLM", Qwen2Config)
    def build(cfg):
        h, eps = cfg.hidden_size, cfg.rms_norm_eps
        layers = [PreNormBlock(
            Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                      DistancePenalty(cfg.num_attention_heads), qkv_bias=False, score_cap=cap),
            GatedMLP(h, cfg.intermediate_size), RMSNorm(h, eps), RMSNorm(h, eps),
            {"mixer": "self_attn.", "ffn": "mlp.", "norm_mixer": "input_layernorm.",
             "norm_ffn": "post_attention_layernorm."}) for _ in range(cfg.num_hidden_layers)]
        return DecoderModel(cfg.vocab_size, h, layers, RMSNorm(h, eps), tied_head=True,
                            max_positions=cfg.max_position_embeddings, config=cfg)

    config = {**helpers.TINY_A, "architectures": ["TestDistanceLM"], "hidden_size": 96,
              "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
              "intermediate_size": 136, "vocab_size": 301}
    folder = write_random_model(tmp_path / "distance", config, seed=6, std=0.15, dtype=torch.float32)
    w, cfg = helpers.plain_model(folder)
    tokens = helpers.random_tokens(301, 50, 5)

    def slow(tokens, w):
        """In the weights' own dtype, scores and softmax in float32, the stream in float32."""
        n_q, n_kv, d, eps = 3, 1, 32, cfg["rms_norm_eps"]
        dtype = w["model.embed_tokens.weight"].dtype
        slopes = torch.tensor([2.0 ** -(i + 1) for i in range(n_q)])
        h = w["model.embed_tokens.weight"][torch.tensor(tokens)].float()
        positions = torch.arange(len(tokens))
        distance = (positions[:, None] - positions[None, :]).float()
        for i in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{i}."
            x = plain.rms_norm(h.to(dtype), w[p + "input_layernorm.weight"], eps)[0]
            q = (x @ w[p + "self_attn.q_proj.weight"].T).view(-1, n_q, d).float()
            k = (x @ w[p + "self_attn.k_proj.weight"].T).view(-1, n_kv, d).float()
            v = (x @ w[p + "self_attn.v_proj.weight"].T).view(-1, n_kv, d).float()
            scores = torch.einsum("qhd,kd->hqk", q, k[:, 0]) * d ** -0.5
            scores = cap * torch.tanh(scores / cap) - slopes[:, None, None] * distance[None]
            scores = scores.masked_fill(distance[None] < 0, float("-inf"))
            attended = torch.einsum("hqk,kd->qhd", torch.softmax(scores, -1), v[:, 0]).to(dtype)
            h = h + (attended.reshape(len(tokens), -1) @ w[p + "self_attn.o_proj.weight"].T).float()
            x = plain.rms_norm(h.to(dtype), w[p + "post_attention_layernorm.weight"], eps)[0]
            h = h + plain.gated_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                    w[p + "mlp.down_proj.weight"]).float()
        x = plain.rms_norm(h.to(dtype), w["model.norm.weight"], eps)[0]
        return (x @ w["model.embed_tokens.weight"].T).float()

    want = slow(tokens, w)
    # what bfloat16 costs the slow version itself, times the slack the replay tests use
    cost = float((slow(tokens, {n: t.bfloat16() for n, t in w.items()}) - want).abs().max())
    for dtype, tol in (("float32", dict(atol=2e-5, rtol=1e-4)),
                       ("bfloat16", dict(atol=1.5 * cost, rtol=0))):
        s = ReplaySession(folder, dtype, 128)
        assert "host" not in s.runner.program.kinds
        whole = s.step([{"id": "a", "tokens": tokens, "want": list(range(50))}], ["a"])
        torch.testing.assert_close(whole, want, **tol)
        rows = [s.step([{"id": "b", "tokens": tokens[:31], "want": list(range(31))}], [])]
        for i in range(31, 50):
            rows.append(s.step([{"id": "b", "tokens": tokens[i:i + 1], "want": [0]}],
                               ["b"] if i == 49 else []))
        torch.testing.assert_close(torch.cat(rows), want, **tol)
        if dtype == "float32":
            assert torch.equal(torch.cat(rows), whole)     # the order of sums is the position's own


def test_a_subclass_that_overrides_forward_is_not_lowered():
    """`lower` describes the base class's work.  A subclass with a `forward` of its own must
    run through that `forward`, as a step the caller runs; one that also brings its own
    `lower` is lowered again."""
    from mercury_amd.parts import Attention, GatedMLP, RMSNorm, RotaryPosition

    class Doubled(GatedMLP):
        def forward(self, x, step, accum):
            super().forward(x, step, accum)
            super().forward(x, step, accum)

    class DoubledAndLowered(Doubled):
        def lower(self, program):
            super().lower(program)
            super().lower(program)

    class Renamed(GatedMLP):
        pass

    class OffsetNorm(RMSNorm):
        def forward(self, h, out_dtype, rows=None, partials=None):
            return super().forward(h, out_dtype, rows, partials) + 1

    class Biased(Attention):
        def forward(self, x, step, cache, state, accum):
            return super().forward(x, step, cache, state, accum)

    assert GatedMLP(8, 8).can_lower() and Renamed(8, 8).can_lower()
    assert not Doubled(8, 8).can_lower()
    assert DoubledAndLowered(8, 8).can_lower()
    assert RMSNorm(8, 1e-6).can_lower() and not OffsetNorm(8, 1e-6).can_lower()
    rotary = RotaryPosition(16, 1e4)
    assert Attention(32, 2, 1, 16, rotary).can_lower() and not Biased(32, 2, 1, 16, rotary).can_lower()


def test_a_forward_override_runs_inside_a_model(tmp_path):
    """The same through a model: a feed-forward subclass that runs its base twice gives the
    logits of a model whose feed-forward output is doubled, and its layer is a caller-run
    step of the program."""
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.models.qwen2 import build_qwen2
    from mercury_amd.parts import GatedMLP
    from mercury_amd.weights import write_random_model

    class Doubled(GatedMLP):
        def forward(self, x, step, accum):
            first = super().forward(x, step, accum)
            if first is not None:
                accum += first.sum(0)
            second = super().forward(x, step, accum)
            if second is not None:
                accum += second.sum(0)

    @register_architecture("TestDoubledLM", Qwen2Config)
    def build(cfg):
        model = build_qwen2(cfg)
        block = model.layers[0]
        block.ffn = Doubled(cfg.hidden_size, cfg.intermediate_size)
        return model

    config = {**helpers.TINY_A, "architectures": ["TestDoubledLM"]}
    folder = write_random_model(tmp_path / "doubled", config, seed=5, std=0.08, dtype=torch.float32)
    w, cfg = helpers.plain_model(folder)
    doubled = dict(w)
    doubled["model.layers.0.mlp.down_proj.weight"] = 2 * w["model.layers.0.mlp.down_proj.weight"]
    tokens = helpers.random_tokens(512, 33, 9)
    s = ReplaySession(folder, "float32", 64)
    assert s.runner.program.kinds.count("host") == 1
    got = s.step([{"id": "a", "tokens": tokens, "want": list(range(33))}], ["a"])
    torch.testing.assert_close(got, plain.forward_logits(doubled, cfg, tokens), atol=2e-5, rtol=1e-4)

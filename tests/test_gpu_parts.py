"""Each part of a layer alone against its plain function, and that a toy mixer with a state of
its own, a layer named twice and a layer that reads another layer's cache can be registered,
built and stepped from outside the package."""

from __future__ import annotations

import json

import pytest
import torch

from tests import helpers
from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def settle(acc, pending):
    """A part may hand back partial sums it has not added into the accumulator."""
    if pending is not None:
        acc += pending.sum(0)
    return acc


def one_sequence_step(tokens, start, manager, key="s"):
    from mercury_amd.engine.batch import SeqChunk, build_step

    if not manager.holds(key):
        manager.admit(key, [], start + tokens)
    manager.grow(key, start, start + tokens)
    return build_step([SeqChunk(key, [0] * tokens, start, [])], manager, 10, 4096, DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from mercury_amd.parts import RMSNorm

    part = RMSNorm(168, 3e-6)
    w = (1 + rnd(168, seed=1, scale=0.1)).to(dtype)
    part.bind({"weight": w.to(DEV)}, dtype, DEV)
    h = rnd(11, 168, seed=2)
    want, _ = plain.rms_norm(h, w.float(), 3e-6)
    got = part.forward(h.to(DEV), dtype).float().cpu()
    torch.testing.assert_close(got, want, atol=2e-6 if dtype == torch.float32 else 2e-2, rtol=1e-5 if dtype == torch.float32 else 2e-2)
    assert part.param_specs()["weight"].shape == (168,)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part_adds_into_the_accumulator(dtype):
    from mercury_amd.parts import GatedMLP

    part = GatedMLP(168, 410)
    params = {n: rnd(*s.shape, seed=i, scale=0.05).to(dtype) for i, (n, s) in enumerate(part.param_specs().items())}
    part.bind({n: t.to(DEV) for n, t in params.items()}, dtype, DEV)
    x = rnd(9, 168, seed=7).to(dtype)
    acc = rnd(9, 168, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    want = acc + plain.gated_mlp(x.float(), params["gate_proj.weight"].float(),
                                 params["up_proj.weight"].float(), params["down_proj.weight"].float())
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=5e-3, rtol=2e-2)
    torch.testing.assert_close(acc_d.cpu(), want, **tol)
    with pytest.raises(ValueError, match="activation"):
        GatedMLP(8, 8, activation="relu")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 12])
def test_attention_part_over_two_portions(dtype, window):
    """The mixer alone: a 21-token portion, then 9 more tokens of the same sequence, equal the
    plain attention layer over all 30 (with and without a window)."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.parts import Attention, LayerCache, RotaryPosition

    hidden, n_q, n_kv, d, page = 72, 6, 2, 16, 8
    part = Attention(hidden, n_q, n_kv, d, RotaryPosition(d, 50000.0), qkv_bias=True, window=window)
    params = {n: rnd(*s.shape, seed=10 + i, scale=0.08).to(dtype)
              for i, (n, s) in enumerate(part.param_specs().items())}
    part.bind({n: t.to(DEV) for n, t in params.items()}, dtype, DEV)
    part.prepare(64, DEV)
    manager = CacheManager({0: part.cache_spec()}, 16, page, 2)
    cache = LayerCache(torch.zeros(16, n_kv, page, d, dtype=dtype, device=DEV),
                       torch.zeros(16, n_kv, d, page, dtype=dtype, device=DEV), 0, page, True)
    x = rnd(30, hidden, seed=30).to(dtype)
    out = []
    for start, count in ((0, 21), (21, 9)):
        step = one_sequence_step(count, start, manager)
        acc = torch.zeros(count, hidden, device=DEV)
        settle(acc, part.forward(x[start:start + count].to(DEV).contiguous(), step, cache, None, acc))
        out.append(acc.cpu())
        manager.trim("s", start + count)
    cfg = {"num_attention_heads": n_q, "num_key_value_heads": n_kv, "head_dim": d}
    cos, sin = plain.rotary_table(d, range(30), 50000.0)
    want = plain.attention_layer(x.float(), {k: v.float() for k, v in params.items()}, "", cfg,
                                 cos, sin, window)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=5e-3, rtol=2e-2)
    torch.testing.assert_close(torch.cat(out), want, **tol)


def test_block_arrangement_is_pre_norm_residual():
    """One whole layer of configuration C equals plain.decoder_layer's running sum."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.config import build_model
    from mercury_amd.parts import LayerCache
    from mercury_amd.weights import FolderSource

    folder = helpers.model_folder("C")
    w, cfg = helpers.plain_model(folder)
    model = build_model(folder)
    block = model.layers[0]
    source = FolderSource(folder)
    prefix = "model.layers.0."
    block.bind({n[len(prefix):]: source.tensor(n).float().to(DEV) for n in source.names()
                if n.startswith(prefix)}, torch.float32, DEV)
    block.prepare(64, DEV)
    spec = block.mixer.cache_spec()
    manager = CacheManager({0: spec}, 8, 16, 2)
    k_pages = torch.zeros(8, spec.kv_heads, 16, spec.head_dim, device=DEV)
    v_pages = torch.zeros(8, spec.kv_heads, spec.head_dim, 16, device=DEV)
    h = rnd(20, cfg["hidden_size"], seed=40)
    h_d = h.clone().to(DEV)
    settle(h_d, block.forward(h_d, one_sequence_step(20, 0, manager),
                              LayerCache(k_pages, v_pages, 0, 16), None, torch.float32))
    cos, sin = plain.rotary_table(cfg["head_dim"], range(20), cfg["rope_theta"])
    x, residual = plain.decoder_layer(h, None, w, 0, cfg, cos, sin)
    torch.testing.assert_close(h_d.cpu(), x + residual, atol=1e-5, rtol=1e-5)


# ------------------------------------------------------------------ toy parts from outside


def register_toys():
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.parts import (Attention, DecoderModel, GatedMLP, LayerCall, Mixer, PreNormBlock,
                                   RMSNorm, RotaryPosition, StateSpec, TensorSpec, register_mixer)

    @register_mixer("test_running_mean")
    class RunningMean(Mixer):
        """out_t = W * mean(x_0..x_t): a mixer whose only memory is a per-request state
        (running sum and count), carried from portion to portion."""

        def __init__(self, hidden):
            self.hidden = hidden

        def state_spec(self):
            return StateSpec((self.hidden + 1,), torch.float32)

        def param_specs(self):
            return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

        def bind(self, params, dtype, device):
            self.w = params["mix.weight"]

        def forward(self, x, step, cache, state, accum):
            slots = step.state_slots.tolist()
            for s, (first, count, start) in enumerate(step.spans):
                rows = x[first:first + count].float()
                sums = state[slots[s], :-1] + rows.cumsum(0)
                counts = state[slots[s], -1] + torch.arange(1, count + 1, device=x.device)
                state[slots[s], :-1] = sums[-1]
                state[slots[s], -1] = counts[-1]
                accum[first:first + count] += (sums / counts[:, None]) @ self.w.float().T

    names = {"mixer": "mixer.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2."}

    @register_architecture("TestToyLM", Qwen2Config)
    def build(cfg):
        h, eps = cfg.hidden_size, cfg.rms_norm_eps
        rotary = RotaryPosition(cfg.head_dim, cfg.rope_theta)

        def attention(window=None):
            return Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                             rotary, qkv_bias=False, window=window)

        def block(mixer):
            return PreNormBlock(mixer, GatedMLP(h, cfg.intermediate_size), RMSNorm(h, eps),
                                RMSNorm(h, eps), names)

        layers = [block(attention()), block(RunningMean(h)), block(attention(window=24)), block(attention())]
        # layer 0 runs twice (second time on its own cache slot); layer 3 reads layer 0's first cache
        calls = [LayerCall(0, 0), LayerCall(1, None), LayerCall(2, 1), LayerCall(0, 2),
                 LayerCall(3, 0, writes=False)]
        return DecoderModel(cfg.vocab_size, h, layers, RMSNorm(h, eps), tied_head=True, calls=calls,
                            layer_prefix="layers.{}.", embed_name="embed.weight", norm_prefix="norm.",
                            max_positions=cfg.max_position_embeddings, config=cfg)

    return build


def plain_toy_logits(w, cfg, tokens):
    """The toy model written the slow way, from the plain parts."""
    eps, d = cfg["rms_norm_eps"], cfg["head_dim"]
    ids = torch.tensor(tokens)
    cos, sin = plain.rotary_table(d, range(len(tokens)), cfg["rope_theta"])
    h = w["embed.weight"][ids]

    def attn(x, i, window=None, kv_from=None):
        p = f"layers.{i}.mixer."
        zero = {p + f"{n}_proj.bias": torch.zeros(w[p + f"{n}_proj.weight"].shape[0]) for n in "qkv"}
        ww = {**w, **zero}
        if kv_from is None:
            return plain.attention_layer(x, ww, p, cfg, cos, sin, window)
        # queries from layer i, keys and values as layer 0 computed them from ITS input
        n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
        q = (x @ w[p + "q_proj.weight"].T).view(-1, n_q, d)
        k, v = kv_from
        q, _ = plain.apply_rotary(q, q[:, :n_kv], cos, sin)
        return plain.causal_attention(q, k, v, d ** -0.5).reshape(len(tokens), -1) @ w[p + "o_proj.weight"].T

    def ffn(x, i):
        p = f"layers.{i}.mlp."
        return plain.gated_mlp(x, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])

    def norm(x, name):
        return plain.rms_norm(x, w[name], eps)[0]

    def run(i, mixer):
        nonlocal h
        h = h + mixer(norm(h, f"layers.{i}.norm1.weight"))
        h = h + ffn(norm(h, f"layers.{i}.norm2.weight"), i)

    n_kv = cfg["num_key_value_heads"]
    x0 = norm(h, "layers.0.norm1.weight")
    k0 = (x0 @ w["layers.0.mixer.k_proj.weight"].T).view(-1, n_kv, d)
    v0 = (x0 @ w["layers.0.mixer.v_proj.weight"].T).view(-1, n_kv, d)
    _, k0 = plain.apply_rotary(k0, k0, cos, sin)
    run(0, lambda x: attn(x, 0))
    run(1, lambda x: (x.cumsum(0) / torch.arange(1, len(tokens) + 1)[:, None]) @ w["layers.1.mixer.mix.weight"].T)
    run(2, lambda x: attn(x, 2, window=24))
    run(0, lambda x: attn(x, 0))
    run(3, lambda x: attn(x, 3, kv_from=(k0, v0)))
    return norm(h, "norm.weight") @ w["embed.weight"].T


def test_toy_architecture_registered_built_and_stepped(tmp_path):
    """A mixer with per-request state, a windowed layer (pages of its own, given back as the
    window passes), a layer named twice and a layer reading another layer's cache: built from
    config.json through the registry, random weights written and loaded, replayed whole and
    in portions beside another request, against the slow version above."""
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model

    register_toys()
    config = {**helpers.TINY_A, "architectures": ["TestToyLM"], "hidden_size": 48,
              "num_attention_heads": 3, "num_key_value_heads": 1, "intermediate_size": 80}
    folder = write_random_model(tmp_path / "toy", config, seed=2, std=0.08, dtype=torch.float32)
    from safetensors.torch import load_file

    w = load_file(str(folder / "model.safetensors"))
    cfg = {**plain.read_config(folder)}
    reqs = {"a": helpers.random_tokens(512, 90, 1), "b": helpers.random_tokens(512, 47, 2)}
    want = {k: plain_toy_logits(w, cfg, v) for k, v in reqs.items()}

    s = ReplaySession(folder, "float32", 256)
    assert [g.window for g in s.manager.groups] == [None, 24]
    assert not s.manager.prefix_sharing and list(s.runner.states) == [1]
    for key, tokens in reqs.items():
        got = s.step([{"id": key, "tokens": tokens, "want": list(range(len(tokens)))}], [key])
        torch.testing.assert_close(got, want[key], atol=2e-5, rtol=1e-4)
    done = {"a": 0, "b": 0}
    rows = {"a": [], "b": []}
    sizes = [16, 7, 2, 5, 3, 2, 33, 9, 1, 1, 20]
    n = 0
    while any(done[k] < len(reqs[k]) for k in reqs):
        entries = []
        for i, k in enumerate(reqs):
            if done[k] >= len(reqs[k]):
                continue
            part = reqs[k][done[k]:done[k] + sizes[(n + 4 * i) % len(sizes)]]
            entries.append({"id": k, "tokens": part, "want": list(range(len(part)))})
        ends = [e["id"] for e in entries if done[e["id"]] + len(e["tokens"]) == len(reqs[e["id"]])]
        out = s.step(entries, ends)
        at = 0
        for e in entries:
            rows[e["id"]].append(out[at:at + len(e["tokens"])])
            at += len(e["tokens"])
            done[e["id"]] += len(e["tokens"])
        window_pool = s.manager.groups[1].pool
        assert window_pool.num_pages - window_pool.num_available() <= 2 * 4
        s.manager.check_invariants()
        n += 1
    for k in reqs:
        torch.testing.assert_close(torch.cat(rows[k]), want[k], atol=2e-5, rtol=1e-4)
    assert s.manager.leaked_pages() == 0


# ------------------------------------------- a routed feed-forward and other position encodings


def register_routed_toy():
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.kernels import ops
    from mercury_amd.parts import (Attention, DecoderModel, FeedForward, NoPosition, PreNormBlock,
                                   RMSNorm, RotaryPosition, TensorSpec, register_ffn)

    @register_ffn("test_top1_experts")
    class Top1Experts(FeedForward):
        """Every token goes to the one expert whose router logit (float32) is largest; an
        expert is a SiLU-gated projection pair; its output is scaled by the softmax weight of
        the chosen logit."""

        def __init__(self, hidden, inter, experts):
            self.hidden, self.inter, self.experts = hidden, inter, experts

        def param_specs(self):
            specs = {"router.weight": TensorSpec((self.experts, self.hidden))}
            for e in range(self.experts):
                specs[f"experts.{e}.gate_up.weight"] = TensorSpec((2 * self.inter, self.hidden))
                specs[f"experts.{e}.down.weight"] = TensorSpec((self.hidden, self.inter))
            return specs

        def bind(self, params, dtype, device):
            self.p = params

        def forward(self, x, step, accum):
            scores = torch.softmax(x.float() @ self.p["router.weight"].float().T, dim=-1)
            weight, choice = scores.max(dim=-1)
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                mine = x[rows].contiguous()
                act = ops.silu_mul(ops.linear(mine, self.p[f"experts.{e}.gate_up.weight"]))
                out = ops.linear(act, self.p[f"experts.{e}.down.weight"], out_dtype=torch.float32)
                accum.index_add_(0, rows, out * weight[rows, None])

    names = {"mixer": "mixer.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2."}

    @register_architecture("TestRoutedLM", Qwen2Config)
    def build(cfg):
        h, eps, d = cfg.hidden_size, cfg.rms_norm_eps, cfg.head_dim
        positions = [RotaryPosition(d, cfg.rope_theta, rotary_dim=d // 2), NoPosition(),
                     RotaryPosition(d, cfg.rope_theta)]
        layers = [PreNormBlock(Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, d,
                                         pos, qkv_bias=True),
                               Top1Experts(h, cfg.intermediate_size, 3), RMSNorm(h, eps),
                               RMSNorm(h, eps), names) for pos in positions]
        return DecoderModel(cfg.vocab_size, h, layers, RMSNorm(h, eps), tied_head=False,
                            layer_prefix="layers.{}.", embed_name="embed.weight",
                            norm_prefix="norm.", head_name="head.weight",
                            max_positions=cfg.max_position_embeddings, config=cfg)

    return build


def plain_routed_logits(w, cfg, tokens, margins=None):
    """Logits of the routed toy model; `margins`, a list, receives per layer the gap between
    every token's two largest router probabilities."""
    eps, d = cfg["rms_norm_eps"], cfg["head_dim"]
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    t = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    full_cos, full_sin = plain.rotary_table(d, range(t), cfg["rope_theta"])
    half_cos, half_sin = plain.rotary_table(d // 2, range(t), cfg["rope_theta"])

    def rotate(q, k, layer):
        if layer == 1:
            return q, k                                   # no position encoding
        if layer == 2:
            return plain.apply_rotary(q, k, full_cos, full_sin)
        # layer 0: only the first d/2 dims of a head turn, as a head of d/2 would
        q1, k1 = plain.apply_rotary(q[..., : d // 2], k[..., : d // 2], half_cos, half_sin)
        return torch.cat([q1, q[..., d // 2:]], -1), torch.cat([k1, k[..., d // 2:]], -1)

    for i in range(3):
        p = f"layers.{i}."
        x = plain.rms_norm(h, w[p + "norm1.weight"], eps)[0]
        q = (x @ w[p + "mixer.q_proj.weight"].T + w[p + "mixer.q_proj.bias"]).view(t, n_q, d)
        k = (x @ w[p + "mixer.k_proj.weight"].T + w[p + "mixer.k_proj.bias"]).view(t, n_kv, d)
        v = (x @ w[p + "mixer.v_proj.weight"].T + w[p + "mixer.v_proj.bias"]).view(t, n_kv, d)
        q, k = rotate(q, k, i)
        h = h + plain.causal_attention(q, k, v, d ** -0.5).reshape(t, -1) @ w[p + "mixer.o_proj.weight"].T
        x = plain.rms_norm(h, w[p + "norm2.weight"], eps)[0]
        scores = torch.softmax(x.float() @ w[p + "mlp.router.weight"].float().T, dim=-1)
        weight, choice = scores.max(-1)
        if margins is not None:
            top = scores.topk(2, dim=-1).values
            margins.append(top[:, 0] - top[:, 1])
        weight = weight.to(h.dtype)
        out = torch.zeros_like(h)
        for e in range(3):
            gu, down = w[p + f"mlp.experts.{e}.gate_up.weight"], w[p + f"mlp.experts.{e}.down.weight"]
            inter = gu.shape[0] // 2
            y = plain.gated_mlp(x, gu[:inter], gu[inter:], down)
            out = torch.where((choice == e)[:, None], y * weight[:, None], out)
        h = h + out
    return plain.rms_norm(h, w["norm.weight"], eps)[0] @ w["head.weight"].T


def test_routed_feed_forward_and_other_position_encodings(tmp_path):
    """A feed-forward that routes every token to one of three experts, attention with rotation
    over half of the head, and attention with no position encoding at all: registered from
    here, built through the registry, and stepped whole, in portions and token by token."""
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model
    from safetensors.torch import load_file

    register_routed_toy()
    config = {**helpers.TINY_A, "architectures": ["TestRoutedLM"], "hidden_size": 64, "head_dim": 32,
              "num_attention_heads": 2, "num_key_value_heads": 1, "intermediate_size": 48,
              "tie_word_embeddings": False}
    from mercury_amd.weights import save_file

    folder = write_random_model(tmp_path / "routed", config, seed=8, std=0.1, dtype=torch.float32)
    w = load_file(str(folder / "model.safetensors"))
    # routers with wide weights: most tokens' choice of expert is far from a tie
    # (copies: the loaded tensors are views of the very file that is rewritten here)
    w = {k: (v * 16 if "router" in k else v.clone()) for k, v in w.items()}
    save_file(w, folder / "model.safetensors")
    cfg = plain.read_config(folder)
    tokens = helpers.random_tokens(512, 70, 3)
    want = plain_routed_logits(w, cfg, tokens)
    # the router must actually route: every expert gets tokens in every layer
    for i in range(3):
        x = torch.randn(200, 64, generator=torch.Generator().manual_seed(i))
        assert len(set((x @ w[f"layers.{i}.mlp.router.weight"].T).argmax(-1).tolist())) == 3

    s = ReplaySession(folder, "float32", 256)
    whole = s.step([{"id": "w", "tokens": tokens, "want": list(range(70))}], ["w"])
    torch.testing.assert_close(whole, want, atol=1e-4, rtol=1e-4)
    parts, at = [], 0
    for size in (33, 2, 19, 1, 1, 1, 13):
        part = tokens[at:at + size]
        parts.append(s.step([{"id": "p", "tokens": part, "want": list(range(size))}],
                            ["p"] if at + size == 70 else []))
        at += size
    torch.testing.assert_close(torch.cat(parts), want, atol=1e-4, rtol=1e-4)
    assert s.manager.leaked_pages() == 0

    # bfloat16 (the matrix-core kernels take head size 32; rotation over half a head goes the
    # unfused way, no rotation the fused one).  Routing is discontinuous: a token whose two
    # best router probabilities lie within bfloat16's rounding may go to another expert than
    # in float32, and every later token attends to it.  So the comparison covers the tokens
    # before the first one whose routing is that close in any layer; up to there the bound is
    # the one the replay tests derive: the distance of the plain implementation's own
    # bfloat16 run from its float32 run, times the slack.
    from tests.test_gpu_replay import BF16_SLACK

    margins = []
    plain_routed_logits(w, cfg, tokens, margins)
    fragile = (torch.stack(margins).amin(0) < 0.2).nonzero().flatten()
    safe = int(fragile[0]) if fragile.numel() else len(tokens)
    assert safe >= 16, f"the seed makes token {safe} fragile; pick weights with a later one"
    w16 = {k: v.to(torch.bfloat16) for k, v in w.items()}
    want16 = plain_routed_logits({k: v.float() for k, v in w16.items()}, cfg, tokens)
    rounded = plain_routed_logits(w16, cfg, tokens).float()
    cost = float((rounded[:safe] - want16[:safe]).abs().max())
    b = ReplaySession(folder, "bfloat16", 256)
    got = b.step([{"id": "w", "tokens": tokens, "want": list(range(70))}], ["w"])
    assert torch.isfinite(got).all()
    error = (got[:safe] - want16[:safe]).abs().max()
    assert float(error) <= BF16_SLACK * cost, (float(error), cost, safe)


# ------------------------------------------------------- position encodings from outside


def register_position_toys():
    from mercury_amd.config import Qwen2Config, register_architecture
    from mercury_amd.parts import (Attention, DecoderModel, GatedMLP, PositionDescriptor,
                                   PositionEncoding, PreNormBlock, RMSNorm, TensorSpec,
                                   register_position)

    @register_position("test_interleaved_rotary")
    class InterleavedRotary(PositionEncoding):
        """Rotary encoding that pairs dims (2j, 2j + 1) of a head: it only describes itself
        (tables and layout); the kernels do the turning."""

        def __init__(self, head_dim, theta):
            self.head_dim, self.theta = head_dim, theta
            self.cos = self.sin = None

        def prepare(self, max_positions, device):
            inv = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim))
            angles = torch.outer(torch.arange(max_positions, dtype=torch.float32), inv)
            self.cos, self.sin = angles.cos().to(device), angles.sin().to(device)

        def describe(self):
            return PositionDescriptor(self.head_dim, self.cos, self.sin, interleaved=True)

    @register_position("test_added_positions")
    class AddedPositions(PositionEncoding):
        """A stored vector per position added to every query and key head: nothing the
        kernels know, so it describes nothing and applies itself."""

        def __init__(self, head_dim, positions):
            self.head_dim, self.positions = head_dim, positions
            self.table = None

        def param_specs(self):
            return {"table": TensorSpec((self.positions, self.head_dim))}

        def bind(self, params, dtype, device):
            self.table = params["table"]

        def describe(self):
            return None

        def apply(self, q, k, positions):
            rows = self.table[positions.long()][:, None, :]
            q += rows
            if k is not None:
                k += rows

    class PositionedAttention(Attention):
        """Attention whose position encoding brings tensors of its own."""

        def param_specs(self):
            specs = super().param_specs()
            specs.update({"position." + n: s for n, s in self.position.param_specs().items()})
            return specs

        def bind(self, params, dtype, device):
            super().bind(params, dtype, device)
            self.position.bind({n[len("position."):]: t for n, t in params.items()
                                if n.startswith("position.")}, dtype, device)

    names = {"mixer": "mixer.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2."}

    @register_architecture("TestPositionsLM", Qwen2Config)
    def build(cfg):
        h, eps, d = cfg.hidden_size, cfg.rms_norm_eps, cfg.head_dim
        positions = [InterleavedRotary(d, cfg.rope_theta), AddedPositions(d, 128)]
        layers = [PreNormBlock(PositionedAttention(h, cfg.num_attention_heads,
                                                   cfg.num_key_value_heads, d, pos, qkv_bias=True),
                               GatedMLP(h, cfg.intermediate_size), RMSNorm(h, eps), RMSNorm(h, eps),
                               names) for pos in positions]
        return DecoderModel(cfg.vocab_size, h, layers, RMSNorm(h, eps), tied_head=True,
                            layer_prefix="layers.{}.", embed_name="embed.weight",
                            norm_prefix="norm.", max_positions=128, config=cfg)

    return build


def plain_positions_logits(w, cfg, tokens):
    eps, d = cfg["rms_norm_eps"], cfg["head_dim"]
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    t = len(tokens)
    h = w["embed.weight"][torch.tensor(tokens)]
    inv = 1.0 / (cfg["rope_theta"] ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    angles = torch.outer(torch.arange(t, dtype=torch.float32), inv)[:, None, :]

    def interleaved(x):
        even, odd = x[..., 0::2], x[..., 1::2]
        out = torch.empty_like(x)
        out[..., 0::2] = even * angles.cos() - odd * angles.sin()
        out[..., 1::2] = odd * angles.cos() + even * angles.sin()
        return out

    for i in range(2):
        p = f"layers.{i}."
        x = plain.rms_norm(h, w[p + "norm1.weight"], eps)[0]
        q = (x @ w[p + "mixer.q_proj.weight"].T + w[p + "mixer.q_proj.bias"]).view(t, n_q, d)
        k = (x @ w[p + "mixer.k_proj.weight"].T + w[p + "mixer.k_proj.bias"]).view(t, n_kv, d)
        v = (x @ w[p + "mixer.v_proj.weight"].T + w[p + "mixer.v_proj.bias"]).view(t, n_kv, d)
        if i == 0:
            q, k = interleaved(q), interleaved(k)
        else:
            rows = w[p + "mixer.position.table"][:t, None, :]
            q, k = q + rows, k + rows
        h = h + plain.causal_attention(q, k, v, d ** -0.5).reshape(t, -1) @ w[p + "mixer.o_proj.weight"].T
        x = plain.rms_norm(h, w[p + "norm2.weight"], eps)[0]
        h = h + plain.gated_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                w[p + "mlp.down_proj.weight"])
    return plain.rms_norm(h, w["norm.weight"], eps)[0] @ w["embed.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_position_encodings_registered_from_outside(tmp_path, dtype):
    """Two position encodings the package does not have, defined here: a rotary in the
    interleaved pair layout, which only describes itself to the kernels (the host core runs
    its layer), and a stored vector per position added to queries and keys, which applies
    itself (its layer is run from Python between the host core's).  Whole, in portions and
    token by token."""
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import write_random_model
    from safetensors.torch import load_file
    from tests.test_gpu_replay import BF16_SLACK

    register_position_toys()
    config = {**helpers.TINY_A, "architectures": ["TestPositionsLM"], "hidden_size": 64,
              "head_dim": 32, "num_attention_heads": 4, "num_key_value_heads": 2,
              "intermediate_size": 96, "max_position_embeddings": 128}
    folder = write_random_model(tmp_path / "positions", config, seed=5, std=0.1, dtype=torch.bfloat16)
    w = {k: v.float() for k, v in load_file(str(folder / "model.safetensors")).items()}
    cfg = plain.read_config(folder)
    tokens = helpers.random_tokens(512, 75, 9)
    want = plain_positions_logits(w, cfg, tokens)
    # the encodings matter: with neither, the logits are others
    moved = plain_positions_logits(w, cfg, tokens[1:])
    assert (moved[:-1] - want[1:-1]).abs().max() > 1e-2

    s = ReplaySession(folder, dtype, 256)
    kinds = s.runner.program.kinds
    assert kinds.count("host") == 1 and kinds.count("attention") == 1
    if dtype == "float32":
        check = lambda got: torch.testing.assert_close(got, want, atol=2e-5, rtol=1e-4)
    else:
        w16 = {k: v.to(torch.bfloat16) for k, v in w.items()}
        cost = float((plain_positions_logits(w16, cfg, tokens).float() - want).abs().max())
        check = lambda got: float((got - want).abs().max()) <= BF16_SLACK * cost or pytest.fail(
            f"bfloat16 error {float((got - want).abs().max()):.3e} against a cost of {cost:.3e}")
    check(s.step([{"id": "w", "tokens": tokens, "want": list(range(75))}], ["w"]))
    parts, at = [], 0
    for size in (20, 2, 17, 1, 1, 30, 4):
        part = tokens[at:at + size]
        parts.append(s.step([{"id": "p", "tokens": part, "want": list(range(size))}],
                            ["p"] if at + size == 75 else []))
        at += size
    check(torch.cat(parts))
    assert s.manager.leaked_pages() == 0

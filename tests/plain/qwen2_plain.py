"""A plain, slow Qwen2 decoder: whole sequences, no cache, no batching, CPU tensors.

Every function is written from the formulas of the upstream reference implementation and
cites the file and lines it follows (paths relative to the reference tree).  Nothing here
imports from ``mercury_amd``: the engine under test and this file only share the model
folder on disk (``config.json`` + ``model.safetensors``, the latter read through the
``safetensors`` package, which the engine does not use).

All tensors have one floating-point type, the one the weights are read in: float32 by default
(float64 on request), where the reference's casts to the model dtype are the identity.  Read in
bfloat16, every function rounds where the reference rounds to the model dtype (after each
projection, sum, norm, rotation and activation), with the statistics of norms and softmax in
float32 as there; the distance of that run from the float32 run is what bfloat16 costs the
reference itself, which the tests use as the measure of the engine's bfloat16 error.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- configuration


def read_config(folder) -> dict:
    """The architecture numbers with the reference's defaults (mercury/config.py:45-71)."""
    raw = json.loads((Path(folder) / "config.json").read_text())
    heads = raw["num_attention_heads"]
    hidden = raw["hidden_size"]
    return {
        "hidden_size": hidden,
        "intermediate_size": raw["intermediate_size"],
        "num_hidden_layers": raw["num_hidden_layers"],
        "num_attention_heads": heads,
        "num_key_value_heads": raw.get("num_key_value_heads", heads),
        "head_dim": raw.get("head_dim") or hidden // heads,
        "vocab_size": raw["vocab_size"],
        "rms_norm_eps": raw.get("rms_norm_eps", 1e-6),
        "rope_theta": float(raw.get("rope_theta", 10000.0)),
        "tie_word_embeddings": bool(raw.get("tie_word_embeddings", False)),
    }


def read_weights(folder, dtype=torch.float32) -> dict:
    from safetensors.torch import load_file

    tensors = load_file(str(Path(folder) / "model.safetensors"))
    return {name: t.to(dtype) for name, t in tensors.items()}


# --------------------------------------------------------------------------- parts


def _wide(dtype):
    """The type statistics are computed in: float32, as the reference's `.float()`
    (mercury/model/qwen2.py:29-30), or the tensors' own when that is wider."""
    return torch.promote_types(dtype, torch.float32)


def rms_norm(x, weight, eps, residual=None):
    """(normalised * weight, x + residual).  mercury/model/qwen2.py:27-31.

    The sum with the residual happens first and is the second return value; the mean of
    squares is taken over the last axis and eps is added to that mean, inside the root.
    """
    if residual is not None:
        x = x + residual
    wide = x.to(_wide(x.dtype))
    variance = wide.pow(2).mean(-1, keepdim=True)
    normed = (wide * torch.rsqrt(variance + eps)).to(x.dtype)
    return normed * weight, x


def rotary_table(head_dim, positions, theta):
    """cos, sin of shape [len(positions), head_dim].  mercury/model/rope.py:37-47.

    inv_freq_j = 1 / theta^(2j/d) for j < d/2, all in float32 as upstream; the angle of
    (position, j) is their product; the half-table is repeated so that columns j and
    j + d/2 share one angle.
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    pos = torch.as_tensor(positions, dtype=torch.float32)
    freqs = torch.outer(pos, inv_freq)
    table = torch.cat((freqs, freqs), dim=-1)
    return table.cos(), table.sin()


def rotate_half(x):
    """cat(-second half, first half).  mercury/model/rope.py:6-8."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary(q, k, cos, sin):
    """q [T, n_q, d], k [T, n_kv, d], cos/sin [T, d].  mercury/model/rope.py:11-17."""
    cos = cos.unsqueeze(1).to(q.dtype)
    sin = sin.unsqueeze(1).to(q.dtype)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def causal_attention(q, k, v, scale, query_offset=0, window=None):
    """q [Tq, n_q, d]; k, v [S, n_kv, d] -> [Tq, n_q, d].

    Grouped heads: query head h reads key/value head h // (n_q / n_kv)
    (mercury/model/attention.py:26-29, repeat_interleave on the head axis).  Key j is
    visible to the query at absolute position p = query_offset + i iff j <= p
    (mercury/model/attention.py:96-100; tests/test_attention.py:25-35 is the same oracle).
    `window`, when given, additionally hides keys with j <= p - window; the reference has
    no window, the argument exists for the cache manager's window groups.
    """
    out_dtype = q.dtype
    q, k, v = (t.to(_wide(out_dtype)) for t in (q, k, v))     # scores and softmax in float32
    groups = q.shape[1] // k.shape[1]
    k = k.repeat_interleave(groups, dim=1)
    v = v.repeat_interleave(groups, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * scale
    key_pos = torch.arange(k.shape[0])
    query_pos = torch.arange(q.shape[0]) + query_offset
    hidden = key_pos[None, None, :] > query_pos[None, :, None]
    if window is not None:
        hidden = hidden | (key_pos[None, None, :] <= query_pos[None, :, None] - window)
    scores = scores.masked_fill(hidden, float("-inf"))
    weights = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", weights, v).to(out_dtype)


def silu(z):
    """z * sigmoid(z), the activation of the gated MLP (mercury/model/qwen2.py:42)."""
    wide = z.to(_wide(z.dtype))
    return (wide / (1.0 + torch.exp(-wide))).to(z.dtype)


def gated_mlp(x, gate_w, up_w, down_w):
    """down(silu(gate(x)) * up(x)), no biases.  mercury/model/qwen2.py:34-42."""
    return (silu(x @ gate_w.T) * (x @ up_w.T)) @ down_w.T


def attention_layer(x, w, prefix, cfg, cos, sin, window=None):
    """Biased q/k/v, rotary on q and k, attention, unbiased o.  mercury/model/qwen2.py:55-69."""
    n_q, n_kv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    tokens = x.shape[0]
    q = (x @ w[prefix + "q_proj.weight"].T + w[prefix + "q_proj.bias"]).view(tokens, n_q, d)
    k = (x @ w[prefix + "k_proj.weight"].T + w[prefix + "k_proj.bias"]).view(tokens, n_kv, d)
    v = (x @ w[prefix + "v_proj.weight"].T + w[prefix + "v_proj.bias"]).view(tokens, n_kv, d)
    q, k = apply_rotary(q, k, cos, sin)
    out = causal_attention(q, k, v, d**-0.5, 0, window)
    return out.reshape(tokens, n_q * d) @ w[prefix + "o_proj.weight"].T


def decoder_layer(x, residual, w, index, cfg, cos, sin):
    """norm -> attention -> norm -> mlp, the sum carried in `residual`.
    mercury/model/qwen2.py:82-94."""
    p = f"model.layers.{index}."
    eps = cfg["rms_norm_eps"]
    x, residual = rms_norm(x, w[p + "input_layernorm.weight"], eps, residual)
    x = attention_layer(x, w, p + "self_attn.", cfg, cos, sin)
    x, residual = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps, residual)
    x = gated_mlp(
        x,
        w[p + "mlp.gate_proj.weight"],
        w[p + "mlp.up_proj.weight"],
        w[p + "mlp.down_proj.weight"],
    )
    return x, residual


def forward_hidden(w, cfg, token_ids, first_position=0):
    """Final-norm hidden states [T, H] for one whole sequence.  mercury/model/qwen2.py:107-114.

    `first_position` shifts every absolute position; with only distances mattering to the
    rotary encoding, logits must not depend on it (an invariant the tests use).
    """
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    dtype = w["model.embed_tokens.weight"].dtype
    positions = torch.arange(first_position, first_position + len(ids))
    cos, sin = rotary_table(cfg["head_dim"], positions, cfg["rope_theta"])
    cos, sin = cos.to(dtype), sin.to(dtype)
    x = w["model.embed_tokens.weight"][ids]
    residual = None
    for index in range(cfg["num_hidden_layers"]):
        x, residual = decoder_layer(x, residual, w, index, cfg, cos, sin)
    x, _ = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"], residual)
    return x


def forward_logits(w, cfg, token_ids, first_position=0):
    """Logits [T, V]: hidden states times the output embedding, which is the input
    embedding when `tie_word_embeddings` is set.  mercury/model/qwen2.py:128-130, 145-150."""
    hidden = forward_hidden(w, cfg, token_ids, first_position)
    head = (
        w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    )
    return hidden @ head.T


def greedy_generate(w, cfg, prompt, steps):
    """Recompute the whole sequence for every new token; argmax of the last row."""
    tokens = list(prompt)
    out = []
    for _ in range(steps):
        logits = forward_logits(w, cfg, tokens)
        nxt = int(torch.argmax(logits[-1]))
        out.append(nxt)
        tokens.append(nxt)
    return out


# --------------------------------------------------------------------------- sampling


def nucleus_mask(probs, top_p):
    """Zero every probability after the token that crosses top_p in descending order
    (the crossing token stays).  mercury/sampling.py:6-14."""
    ordered, index = probs.sort(dim=-1, descending=True)
    cumulative = ordered.cumsum(dim=-1)
    drop = (cumulative - ordered) > top_p
    ordered = ordered.masked_fill(drop, 0.0)
    out = torch.zeros_like(probs)
    out.scatter_(-1, index, ordered)
    return out


def sampling_distribution(logits, temperature, top_p):
    """The distribution a non-greedy row is drawn from.  mercury/sampling.py:28-33:
    softmax(logits / max(temperature, 1e-5)) in float32, nucleus mask when top_p < 1,
    renormalised (uniform when everything was masked)."""
    scaled = logits.float() / max(temperature, 1e-5)
    probs = torch.softmax(scaled, dim=-1)
    if top_p < 1.0:
        probs = nucleus_mask(probs, top_p)
    total = probs.sum()
    if total > 0:
        return probs / total
    return torch.full_like(probs, 1.0 / probs.shape[-1])


def inverse_cdf_draw(probs, u):
    """The first index whose inclusive cumulative probability exceeds u * total.

    The reference draws with torch.multinomial from an engine-wide generator
    (mercury/sampling.py:34), which cannot be reproduced draw for draw; only the
    distribution is the reference's.  The engine draws by inverse CDF from a uniform
    number, and this is that rule written the slow way.
    """
    cumulative = probs.double().cumsum(-1)
    target = u * float(cumulative[-1])
    index = int(torch.searchsorted(cumulative, torch.tensor(target, dtype=torch.float64), right=True))
    return min(index, probs.shape[-1] - 1)


def slot_mapping(blocks, start, stop, block_size):
    """Physical slot of each position in [start, stop): table[p // bs] * bs + p % bs.
    mercury/runner.py:25-34."""
    return [blocks[p // block_size] * block_size + p % block_size for p in range(start, stop)]


def kv_bytes_per_token(cfg, elem_bytes):
    """2 * layers * kv heads * head_dim * element size.  mercury/config.py:73-81."""
    return 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * elem_bytes


def isclose(a, b, tol):
    return math.isclose(a, b, rel_tol=tol, abs_tol=tol)

"""Safetensors by name, the loader's one error, and the random-weights mode."""

from __future__ import annotations

import json

import pytest
import torch

from mercury_amd.config import build_model
from mercury_amd.weights import (DictSource, FolderSource, SafetensorsFile, WeightLoadError,
                                 check_source, random_state, save_file, write_random_model)
from mercury_amd.weights.loader import target_dtype
from tests.helpers import TINY_A, TINY_B


def test_file_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file as their_save

    tensors = {"a.weight": torch.randn(5, 7).to(torch.bfloat16), "b": torch.arange(6, dtype=torch.int32),
               "c.bias": torch.randn(3), "empty": torch.zeros(0, 4)}
    save_file(tensors, tmp_path / "ours.safetensors", metadata={"seed": 3})
    theirs = load_file(str(tmp_path / "ours.safetensors"))           # they read what we wrote
    assert set(theirs) == set(tensors)
    for name, t in tensors.items():
        assert torch.equal(theirs[name], t) and theirs[name].dtype == t.dtype
    their_save(tensors, str(tmp_path / "theirs.safetensors"))        # we read what they wrote
    with SafetensorsFile(tmp_path / "theirs.safetensors") as f:
        assert sorted(f.names()) == sorted(tensors)
        for name, t in tensors.items():
            assert f.shape(name) == tuple(t.shape) and f.dtype(name) == t.dtype
            assert torch.equal(f.tensor(name).clone(), t)


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    folder = write_random_model(tmp_path / "m", TINY_A, seed=11, std=0.02)
    assert json.loads((folder / "config.json").read_text()) == TINY_A
    source = FolderSource(folder)
    model = build_model(folder)
    check_source(model, source)
    assert source.tensor("model.embed_tokens.weight").dtype == torch.bfloat16
    norm = source.tensor("model.layers.0.input_layernorm.weight").float()
    proj = source.tensor("model.layers.1.mlp.gate_proj.weight").float()
    assert abs(norm.mean() - 1.0) < 0.02 and abs(proj.mean()) < 0.005
    assert abs(proj.std() - 0.02) < 0.002
    source.close()


def test_random_weights_depend_on_seed_and_name_only():
    model = build_model(TINY_A)
    a, b, c = random_state(model, 5), random_state(model, 5), random_state(model, 6)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.norm.weight"], c["model.norm.weight"])
    assert not torch.equal(a["model.layers.0.mlp.up_proj.weight"], a["model.layers.1.mlp.up_proj.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    model = build_model(TINY_B)
    state = random_state(model, 1, dtype=torch.float32)
    del state["model.layers.1.self_attn.q_proj.bias"]
    del state["lm_head.weight"]                       # untied: the head is required
    state["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(256)
    state["model.rotary.inv_freq"] = torch.zeros(16)
    state["model.layers.2.mlp.down_proj.weight"] = torch.zeros(704, 256)
    with pytest.raises(WeightLoadError) as info:
        check_source(model, DictSource(state))
    err = info.value
    assert err.missing == ["lm_head.weight", "model.layers.1.self_attn.q_proj.bias"]
    assert err.unexpected == ["model.layers.0.self_attn.o_proj.bias", "model.rotary.inv_freq"]
    assert [m[0] for m in err.mismatched] == ["model.layers.2.mlp.down_proj.weight"]
    text = str(err)
    for needle in ("missing (2)", "unexpected (2)", "wrong shape (1)", "(704, 256)", "(256, 704)"):
        assert needle in text


def test_a_stored_head_beside_a_tied_embedding_is_tolerated():
    """(reference: mercury/model/loader.py:88-89)"""
    model = build_model(TINY_A)
    state = random_state(model, 1)
    state["lm_head.weight"] = torch.zeros(512, 64)
    check_source(model, DictSource(state))


def test_dtype_policy():
    bf16, f32 = torch.bfloat16, torch.float32
    assert target_dtype("matrix", f32, bf16) == bf16        # cast to the compute dtype
    assert target_dtype("vector", f32, bf16) == f32         # a 32-bit vector stays 32-bit
    assert target_dtype("vector", bf16, bf16) == bf16
    assert target_dtype("matrix", bf16, f32) == f32         # the float32 path is all float32
    assert target_dtype("vector", bf16, f32) == f32
    assert target_dtype("table", torch.int64, bf16) == torch.int32


def test_no_weights_is_a_clear_error(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError, match="no safetensors"):
        FolderSource(tmp_path)


def test_random_weights_are_a_function_of_seed_name_and_index():
    """The engine's own generator: normal deviates from (seed, tensor name, element index)
    alone, so a tensor's values do not depend on what else is drawn, or where."""
    import torch

    from mercury_amd.weights.random_init import fill_normal, stream_key

    a = fill_normal(torch.empty(200_000), stream_key(3, "w"), 0.0, 1.0)
    assert torch.equal(a[:1000], fill_normal(torch.empty(1000), stream_key(3, "w"), 0.0, 1.0))
    assert not torch.equal(a[:1000], fill_normal(torch.empty(1000), stream_key(4, "w"), 0.0, 1.0))
    assert not torch.equal(a[:1000], fill_normal(torch.empty(1000), stream_key(3, "v"), 0.0, 1.0))
    # a standard normal: moments, tails, symmetry
    assert abs(float(a.mean())) < 0.01 and abs(float(a.std()) - 1.0) < 0.01
    assert abs(float((a.abs() > 1.959964).float().mean()) - 0.05) < 0.003
    assert abs(float((a > 0).float().mean()) - 0.5) < 0.005
    assert abs(float((a ** 4).mean()) - 3.0) < 0.1
    # scaled, shifted, and rounded to bfloat16 from the float32 value
    b = fill_normal(torch.empty(1000, dtype=torch.bfloat16), stream_key(3, "w"), 1.0, 0.02)
    assert torch.equal(b, (1.0 + 0.02 * a[:1000]).to(torch.bfloat16))

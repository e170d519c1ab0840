"""Random weights drawn on the GPU are, bit for bit, the ones the host draws (and a written
model folder holds), so the plain implementation can reproduce weights that only ever
existed on the device."""

from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_device_and_host_draw_the_same_numbers(dtype):
    from mercury_amd.weights.random_init import fill_normal, stream_key

    # a gate projection of the 0.5B model's size, and odd counts
    for count, name, mean, std in ((4864 * 896, "mlp.gate_proj.weight", 0.0, 0.02),
                                   (896, "input_layernorm.weight", 1.0, 0.02), (1, "x", 0.0, 1.0),
                                   (70_001, "y", 0.0, 1.0)):
        key = stream_key(11, name)
        host = fill_normal(torch.empty(count, dtype=dtype), key, mean, std)
        device = fill_normal(torch.empty(count, dtype=dtype, device="cuda:0"), key, mean, std)
        assert torch.equal(device.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                           host.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)), name


def test_an_engine_with_drawn_weights_equals_one_that_reads_the_written_folder(tmp_path):
    from mercury_amd import Engine, EngineConfig, SamplingParams
    from mercury_amd.weights import write_random_model
    from tests import helpers

    folder = write_random_model(tmp_path / "m", helpers.TINY_B, seed=21, std=0.05, dtype=torch.bfloat16)
    prompts = [helpers.random_tokens(1000, n, seed=n) for n in (3, 40)]
    common = dict(dtype="float32", num_blocks=64, max_model_len=256)
    read = Engine(EngineConfig(model=str(folder), **common))
    drawn = Engine(EngineConfig(model=str(folder / "config.json"), random_weights=True,
                                weight_seed=21, weight_std=0.05, **common))
    given = Engine(EngineConfig(model="", random_weights=True, weight_seed=21, weight_std=0.05,
                                **common), model_config=helpers.TINY_B)
    want = read.generate(prompts, SamplingParams(ignore_eos=True), 6)
    assert drawn.generate(prompts, SamplingParams(ignore_eos=True), 6) == want
    assert given.generate(prompts, SamplingParams(ignore_eos=True), 6) == want
    other = Engine(EngineConfig(model=str(folder), random_weights=True, weight_seed=22,
                                weight_std=0.05, **common))
    assert other.generate(prompts, SamplingParams(ignore_eos=True), 6) != want

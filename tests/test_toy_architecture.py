"""A second, made-up architecture is registered, written, loaded and stepped from the tests
alone (see toy_architecture.py): nothing under ``pagedserve_amd/`` knows it."""

import os

import pytest
import torch

import helpers
import toy_architecture as toy

CONFIG = {"architectures": [toy.NAME], "hidden": 96, "layers": 3, "heads": 6, "kv_heads": 2, "ffn": 200,
          "vocab": 301, "context": 160, "rms_eps": 1e-6, "embed_scale": 3.0, "window": 24}


def _folder(tmp_path, seed=4):
    from pagedserve_amd.model import write_random_model

    toy.register()
    folder = str(tmp_path / "toy")
    write_random_model(folder, dict(CONFIG), seed=seed)
    return folder


def test_registered_written_and_loaded_by_name(tmp_path):
    from pagedserve_amd.config import resolve_architecture
    from pagedserve_amd.model import load_model
    from pagedserve_amd.weights import SafetensorsFile

    folder = _folder(tmp_path)
    assert resolve_architecture(CONFIG).name == toy.NAME
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as handle:
        assert all(name.startswith("model.") for name in handle.names())
    model, config = load_model(folder, dtype="float32", device="cpu")
    assert isinstance(config, toy.ToyConfig) and config.head_dim == 16
    _, weights = toy.read_folder(folder, torch.float32)
    mixer = model.blocks[1].mixer
    # three stored matrices, one packed parameter: [q | k | v] rows
    assert mixer.qkv_weight.shape == (96 + 2 * 32, 96)
    assert torch.equal(mixer.qkv_weight[:96], weights["layers.1.q.weight"])
    assert torch.equal(mixer.qkv_weight[96:128], weights["layers.1.k.weight"])
    assert torch.equal(mixer.qkv_weight[128:], weights["layers.1.v.weight"])
    assert mixer.qkv_bias is None and mixer.window == 24 and model.blocks[0].mixer.window == 0
    assert model.head.weight is not model.embedding.table and model.head.bias_vector.shape == (301,)
    assert model.position.embedding_table() is None and model.embedding.scale == 3.0


def test_joined_tensors_are_checked_piece_by_piece(tmp_path):
    from safetensors.torch import load_file, save_file

    from pagedserve_amd.model import load_model
    from pagedserve_amd.weights import WeightError

    folder = _folder(tmp_path)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.0.k.weight"]
    tensors["model.layers.2.v.weight"] = torch.zeros(32, 95)
    tensors["model.layers.1.gate.weight"] = torch.zeros(3)
    save_file(tensors, path)
    with pytest.raises(WeightError) as caught:
        load_model(folder, dtype="float32", device="cpu")
    error = caught.value
    assert error.missing == ["layers.0.k.weight"]
    assert error.unexpected == ["model.layers.1.gate.weight"]
    assert [name for name, _, _ in error.wrong_shape] == ["layers.2.q.weight + layers.2.k.weight + layers.2.v.weight"]
    assert "[96, 96] + [32, 96] + [32, 95]" in str(error)


def test_a_slice_of_a_stored_tensor_feeds_a_parameter():
    from pagedserve_amd.weights import WeightSource

    stored = torch.arange(40.0).reshape(8, 5)
    source = WeightSource("packed", transpose=True, rows=(1, 4))
    assert source.result_shape([(8, 5)]) == (3, 8)
    assert torch.equal(source.assemble({"packed": stored}.__getitem__), stored.t()[1:4])
    assert WeightSource("packed", rows=(2, 9)).result_shape([(8, 5)]) is None
    assert WeightSource(("a", "b"), axis=1).result_shape([(3, 4), (3, 6)]) == (3, 10)
    assert WeightSource(("a", "b"), axis=1).result_shape([(3, 4), (2, 6)]) is None


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "mixed"])
def test_engine_matches_the_toy_formula(tmp_path, dtype, cut):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    folder = _folder(tmp_path)
    config, weights = toy.read_folder(folder)
    requests = {f"t{i}": helpers.random_tokens(n, CONFIG["vocab"], 700 + i)
                for i, n in enumerate([21, 33, 64, 150, 9, 88])}
    reference = {rid: toy.plain_logits(config, weights, tokens, bfloat16=dtype == "bfloat16")
                 for rid, tokens in requests.items()}
    steps = {"whole": helpers.trace_whole, "mixed": helpers.trace_mixed}[cut](requests)
    model, _ = load_model(folder, dtype=dtype, device="cuda")
    page_size = 8
    # the windowed layers form a cache group of their own and give pages back; the pool is
    # sized for the layers that keep everything
    pages = helpers.live_token_budget(steps, round_to=page_size) // page_size
    engine = Engine(model, num_pages=pages, page_size=page_size, max_requests=4, max_step_tokens=256)
    assert len(engine.cache.groups) == 2
    rows = helpers.replay_in_process(engine, steps)
    engine.cache.check_invariants()
    assert engine.cache.pools[1].peak_allocated < engine.cache.pools[0].peak_allocated or cut == "whole"
    error, scale, where = helpers.max_error(rows, reference)
    assert len(rows) == sum(len(tokens) for tokens in requests.values())
    assert error <= helpers.TOLERANCE[dtype] * scale, (error, scale, where)

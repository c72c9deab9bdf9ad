"""Configuration, registry, safetensors reading and the loader's error report (no GPU)."""

import json
import os

import pytest
import torch

import helpers
from pagedserve_amd.config import (ConfigError, GPT2Config, ModelSpec, LayerCall, PartSpec,
                                   BlockSpec, resolve_architecture)
from pagedserve_amd.model.decoder import DecoderModel
from pagedserve_amd.model.loading import load_model, write_random_model
from pagedserve_amd.weights import (SafetensorsError, SafetensorsFile, WeightError,
                                    write_safetensors)


def test_gpt2_config_reads_its_own_keys():
    config = GPT2Config.from_dict(helpers.TINY_B)
    assert (config.n_layer, config.n_embd, config.n_head, config.head_dim) == (3, 96, 2, 48)
    assert config.n_inner == 320 and config.vocab_size == 1000 and config.n_positions == 256
    assert config.layer_norm_epsilon == 1e-6 and config.activation_kind == "gelu_erf"
    assert config.scale_attn_by_inverse_layer_idx is True and config.tie_word_embeddings is True
    # defaults that config.json may leave out: n_inner = 4 n_embd (src/model/gpt2.py:38)
    minimal = GPT2Config.from_dict({"n_layer": 1, "n_embd": 32, "n_head": 2, "vocab_size": 10,
                                    "max_position_embeddings": 8})
    assert minimal.n_inner == 128 and minimal.n_positions == 8
    assert minimal.activation_kind == "gelu_tanh" and minimal.layer_norm_epsilon == 1e-5
    assert GPT2Config.from_dict(config.to_dict()) == config


@pytest.mark.parametrize("change,match", [
    ({"n_head": 5}, "divisible"),
    ({"add_cross_attention": True}, "cross-attention"),
    ({"activation_function": "relu"}, "activation_function"),
    ({"scale_attn_weights": False}, "scale_attn_weights"),
    ({"n_layer": 0}, "n_layer"),
    ({"n_inner": -3}, "n_inner"),
    ({"vocab_size": "many"}, "vocab_size"),
    ({"layer_norm_epsilon": 0}, "layer_norm_epsilon"),
])
def test_gpt2_config_rejects(change, match):
    with pytest.raises(ConfigError, match=match):
        GPT2Config.from_dict({**helpers.TINY_A, **change})


def test_registry_by_architecture_name():
    entry = resolve_architecture(helpers.TINY_A)
    assert entry.name == "GPT2LMHeadModel" and entry.config_class is GPT2Config
    assert resolve_architecture({"model_type": "gpt2"}).name == "GPT2LMHeadModel"
    with pytest.raises(ConfigError, match="LlamaForCausalLM.*known: GPT2LMHeadModel"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        resolve_architecture({})


def test_spec_is_layer_by_layer_data():
    entry = resolve_architecture(helpers.TINY_B)
    config = GPT2Config.from_dict(helpers.TINY_B)
    spec = entry.build_spec(config)
    assert len(spec.blocks) == 3 and [call.block for call in spec.schedule] == [0, 1, 2]
    scales = [block.mixer.as_dict()["scale"] for block in spec.blocks]
    assert scales == pytest.approx([48 ** -0.5, 48 ** -0.5 / 2, 48 ** -0.5 / 3])
    assert spec.blocks[0].feed_forward.as_dict() == {"inner": 320, "activation": "gelu_erf", "bias": True}
    assert spec.final_norm.as_dict()["eps"] == 1e-6
    off = entry.build_spec(GPT2Config.from_dict(helpers.TINY_A))
    assert {block.mixer.as_dict()["scale"] for block in off.blocks} == {16 ** -0.5}


def test_run_order_rules():
    norm = PartSpec.make("layernorm", eps=1e-5)
    block = BlockSpec.make("pre_norm", norm1=norm,
                           mixer=PartSpec.make("attention", heads=1, kv_heads=1, head_dim=16, scale=1.0),
                           norm2=norm, feed_forward=PartSpec.make("dense", inner=8, activation="gelu_erf"))
    assert block.mixer.kind == "attention" and block.with_part("mixer", norm).mixer is norm
    with pytest.raises(KeyError, match="no part 'gate'"):
        block.part("gate")

    def spec(schedule):
        return ModelSpec("toy", 10, 16, 8, PartSpec.make("none"), (block,), tuple(schedule), norm, True)

    # a block may run twice (own cache entry each time) and a call may read another's entry
    ok = spec([LayerCall(0, 0), LayerCall(0, 1), LayerCall(0, 0, writes_cache=False)])
    assert ok.num_cache_entries == 2
    with pytest.raises(ValueError, match="two writers"):
        spec([LayerCall(0, 0), LayerCall(0, 0)])
    with pytest.raises(ValueError, match="before any call has written"):
        spec([LayerCall(0, 0, writes_cache=False), LayerCall(0, 0)])
    with pytest.raises(ValueError, match="names block"):
        spec([LayerCall(1, 0)])
    with pytest.raises(ValueError, match="without gaps"):
        spec([LayerCall(0, 1)])


def test_safetensors_round_trip_and_library_agreement(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5), "b.c": torch.randn(7).to(torch.bfloat16),
               "ids": torch.arange(6, dtype=torch.int64).reshape(2, 3), "empty": torch.zeros(0, 4),
               "scalar": torch.tensor(3.5)}
    ours = tmp_path / "ours.safetensors"
    write_safetensors(str(ours), tensors, metadata={"k": "v"})
    theirs = load_file(str(ours))                       # the package reads what we write
    for name, tensor in tensors.items():
        assert torch.equal(theirs[name], tensor)
    lib = tmp_path / "lib.safetensors"
    save_file(tensors, str(lib))
    with SafetensorsFile(str(lib)) as handle:           # we read what the package writes
        assert sorted(handle.names()) == sorted(tensors)
        for name, tensor in tensors.items():
            assert handle.shape(name) == tuple(tensor.shape) and handle.dtype(name) == tensor.dtype
            assert torch.equal(handle.tensor(name), tensor)
    with SafetensorsFile(str(ours)) as handle:
        assert handle.metadata == {"k": "v"}
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes(b"\x05\x00\x00\x00\x00\x00\x00\x00{not")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(bad))
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(tmp_path / "absent.safetensors"))


def _load_cpu(folder, dtype):
    return load_model(folder, dtype=dtype, device="cpu")


def test_loader_places_tensors_and_keeps_precisions(tmp_path):
    folder, config, _ = helpers.tiny_folder(tmp_path, "B")      # names without prefix
    tensors = helpers.lively_tensors(config, 1)
    model, typed = _load_cpu(folder, "bfloat16")
    assert typed.n_inner == 320
    mixer = model.blocks[1].mixer
    # Conv1D [in, out] is transposed once at load (src/model/gpt2.py:14-17) ...
    expected = tensors["h.1.attn.c_attn.weight"].t().to(torch.bfloat16)
    assert mixer.qkv_weight.dtype == torch.bfloat16 and torch.equal(mixer.qkv_weight, expected)
    # ... vectors stay 32-bit, bit for bit
    assert mixer.qkv_bias.dtype == torch.float32
    assert torch.equal(mixer.qkv_bias, tensors["h.1.attn.c_attn.bias"])
    assert torch.equal(model.blocks[2].norm2.gamma, tensors["h.2.ln_2.weight"])
    # the tied head is the embedding table itself (src/model/paged_decoder.py:300-301)
    assert model.head.weight is model.embedding.table
    assert torch.equal(model.position.table, tensors["wpe.weight"].to(torch.bfloat16))
    model32, _ = _load_cpu(folder, "float32")
    assert torch.equal(model32.blocks[0].feed_forward.down_weight, tensors["h.0.mlp.c_proj.weight"].t())
    # with the prefix, and with a bfloat16 checkpoint
    folder_a, config_a, _ = helpers.tiny_folder(tmp_path, "A")
    model_a, _ = _load_cpu(folder_a, "float32")
    assert model_a.parameter_count == sum(t.numel() for t in helpers.lively_tensors(config_a, 0).values())
    half = {name: t.to(torch.bfloat16) for name, t in helpers.lively_tensors(config_a, 0).items()}
    helpers.write_folder(str(tmp_path / "half"), config_a, half)
    model_h, _ = _load_cpu(str(tmp_path / "half"), "bfloat16")
    assert model_h.final_norm.gamma.dtype == torch.float32
    assert torch.equal(model_h.final_norm.gamma, half["ln_f.weight"].float())


def test_loader_reports_everything_at_once(tmp_path):
    config = dict(helpers.TINY_A)
    tensors = helpers.lively_tensors(config, 0)
    del tensors["h.0.ln_1.bias"]
    del tensors["h.1.mlp.c_fc.weight"]
    tensors["h.1.attn.c_proj.weight"] = torch.zeros(64, 63)
    tensors["h.0.attn.c_attn.weight"] = torch.zeros(192, 64)       # Linear layout, not Conv1D
    tensors["h.0.attn.rotary.inv_freq"] = torch.zeros(4)
    tensors["wpe.weight"] = torch.zeros(128, 64, dtype=torch.int32)
    tensors["h.0.attn.bias"] = torch.ones(1, 1, 8, 8)              # mask buffers are ignored
    tensors["h.1.attn.masked_bias"] = torch.tensor(-1e4)
    tensors["lm_head.weight"] = tensors["wte.weight"].clone()      # ignored when tied
    folder = helpers.write_folder(str(tmp_path / "broken"), config, tensors)
    with pytest.raises(WeightError) as caught:
        _load_cpu(folder, "float32")
    error = caught.value
    assert error.missing == ["h.0.ln_1.bias", "h.1.mlp.c_fc.weight"]
    assert error.unexpected == ["transformer.h.0.attn.rotary.inv_freq"]
    assert {name for name, _, _ in error.wrong_shape} == {"transformer.h.1.attn.c_proj.weight",
                                                          "transformer.h.0.attn.c_attn.weight"}
    assert [name for name, _, _ in error.wrong_kind] == ["transformer.wpe.weight"]
    text = str(error)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "[192, 64], expected [64, 192]",
                   "wrong dtype"):
        assert needle in text
    # an untied model needs its head
    untied = dict(config, tie_word_embeddings=False)
    good = helpers.lively_tensors(config, 0)
    folder = helpers.write_folder(str(tmp_path / "untied"), untied, good)
    with pytest.raises(WeightError) as caught:
        _load_cpu(folder, "float32")
    assert caught.value.missing == ["lm_head.weight"]


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    import plain_gpt2

    folder = str(tmp_path / "random")
    config = write_random_model(folder, dict(helpers.TINY_A), seed=5)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    with open(os.path.join(folder, "config.json")) as handle:
        assert GPT2Config.from_dict(json.load(handle)) == config
    raw, weights = plain_gpt2.read_model_folder(folder)
    assert raw["architectures"] == ["GPT2LMHeadModel"]
    # N(0, 0.02); residual projections N(0, 0.02 / sqrt(2 L)); biases 0; norm scales 1
    assert abs(float(weights["wte.weight"].std()) - 0.02) < 2e-3
    assert abs(float(weights["h.1.mlp.c_proj.weight"].std()) - 0.02 / 2) < 1e-3
    assert float(weights["h.0.attn.c_attn.bias"].abs().max()) == 0
    assert torch.equal(weights["ln_f.weight"], torch.ones(64, dtype=torch.float64))
    again = str(tmp_path / "again")
    write_random_model(again, dict(helpers.TINY_A), seed=5)
    assert open(os.path.join(folder, "model.safetensors"), "rb").read() == \
        open(os.path.join(again, "model.safetensors"), "rb").read()
    other = str(tmp_path / "other")
    write_random_model(other, dict(helpers.TINY_A), seed=6)
    _, other_weights = plain_gpt2.read_model_folder(other)
    assert not torch.equal(other_weights["wte.weight"], weights["wte.weight"])
    model, _ = _load_cpu(folder, "float32")
    assert isinstance(model, DecoderModel)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_random_weights_in_memory_are_the_folder_loaders_tensors(tmp_path, which, dtype):
    """``random_model`` (what the benchmark and ``--random-weights`` use) binds bit for bit the
    tensors that ``write_random_model`` + ``load_model`` bind: the same draws, the same joined
    and transposed layouts, the same dtype per role, the tied head the table itself."""
    from pagedserve_amd.model.loading import random_model

    raw = dict(helpers.TINY[which][0])
    folder = str(tmp_path / "random")
    write_random_model(folder, raw, seed=11)
    from_folder, config_a = load_model(folder, dtype=dtype, device="cpu")
    in_memory, config_b = random_model(raw, seed=11, dtype=dtype, device="cpu")
    assert config_a == config_b
    assert sorted(from_folder.tensors) == sorted(in_memory.tensors) == sorted(from_folder.parameters())
    for name, tensor in from_folder.tensors.items():
        other = in_memory.tensors[name]
        assert tensor.dtype == other.dtype and tensor.shape == other.shape, name
        assert tensor.is_contiguous() and other.is_contiguous(), name
        assert torch.equal(tensor, other), name
    for model in (from_folder, in_memory):
        tied = model.spec.tie_head
        assert (model.head.weight is model.embedding.table) == tied
    other_seed, _ = random_model(raw, seed=12, dtype=dtype, device="cpu")
    assert not torch.equal(other_seed.tensors["embedding.table"], in_memory.tensors["embedding.table"])

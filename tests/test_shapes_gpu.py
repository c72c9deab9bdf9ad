"""The real layer sizes: GPT-2 small whole (12 layers, vocabulary 50257), and two-layer
models with the widths of medium and XL (1024 / 16 heads / 4096 and 1600 / 25 heads / 6400),
against the plain implementation, whole and cut, in both dtypes.  These sizes take code paths
that the tiny models do not (k > 1024 in the skinny product, 25 heads, a vocabulary that is
no multiple of anything)."""

import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu

SHAPES = {
    "small": dict(n_layer=12, n_embd=768, n_head=12, n_inner=3072, vocab_size=50257, n_positions=1024),
    "medium2": dict(n_layer=2, n_embd=1024, n_head=16, n_inner=4096, vocab_size=2003, n_positions=128),
    "xl2": dict(n_layer=2, n_embd=1600, n_head=25, n_inner=6400, vocab_size=1031, n_positions=128),
}


@pytest.fixture(scope="module")
def shape_folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("shapes")
    out = {}
    for index, (name, sizes) in enumerate(SHAPES.items()):
        config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "layer_norm_epsilon": 1e-5,
                  "activation_function": "gelu_new", "tie_word_embeddings": True, **sizes}
        folder = str(base / name)
        helpers.write_folder(folder, config, helpers.lively_tensors(config, 40 + index))
        out[name] = (folder, config)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_real_sizes_match_plain(shape_folders, name, dtype):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    folder, config = shape_folders[name]
    lengths = [37, 21, 50] if name == "small" else [45, 70, 33]
    requests = {f"s{i}": helpers.random_tokens(n, config["vocab_size"], 900 + i) for i, n in enumerate(lengths)}
    reference = {rid: helpers.plain_logits(folder, tokens, bfloat16=dtype == "bfloat16")
                 for rid, tokens in requests.items()}
    model, _ = load_model(folder, dtype=dtype)
    worst = {}
    for cut, builder in (("whole", helpers.trace_whole), ("mixed", helpers.trace_mixed),
                         ("tail", lambda r: helpers.trace_tail_decoded(r, tail=20))):
        steps = builder(requests)
        pages = -(-helpers.live_token_budget(steps) // 16)
        engine = Engine(model, num_pages=pages, page_size=16, max_requests=4, max_step_tokens=256)
        rows = helpers.replay_in_process(engine, steps)
        error, scale, where = helpers.max_error(rows, reference)
        worst[cut] = (error, scale, where)
        assert error <= helpers.TOLERANCE[dtype] * scale, (name, dtype, cut, error, scale, where)
        engine.cache.check_invariants()
    print(name, dtype, {cut: f"{e / s:.2e}" for cut, (e, s, _) in worst.items()})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_contexts_decode_in_ranges(tmp_path, dtype):
    """Contexts of more than 2,048 keys with 64 (token, head) pairs: the decode kernel runs two
    blocks of 16 waves per pair and merges them; the decoded tokens' logits match the plain
    implementation like any others."""
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "layer_norm_epsilon": 1e-5,
              "activation_function": "gelu_new", "tie_word_embeddings": True, "n_layer": 2, "n_embd": 512,
              "n_head": 16, "n_inner": 640, "vocab_size": 333, "n_positions": 2304}
    folder = str(tmp_path / "long")
    helpers.write_folder(folder, config, helpers.lively_tensors(config, 61))
    requests = {f"L{i}": helpers.random_tokens(2100 + 37 * i, config["vocab_size"], 950 + i) for i in range(4)}
    reference = {rid: helpers.plain_logits(folder, tokens, bfloat16=dtype == "bfloat16")
                 for rid, tokens in requests.items()}
    model, _ = load_model(folder, dtype=dtype)
    mixer = model.blocks[0].mixer if hasattr(model, "blocks") else None
    if mixer is not None:
        assert mixer._splits(4, 2304) == (2, 16)
    steps = helpers.trace_tail_decoded(requests, tail=3)
    pages = -(-helpers.live_token_budget(steps) // 16)
    engine = Engine(model, num_pages=pages, page_size=16, max_requests=4, max_step_tokens=2304)
    rows = helpers.replay_in_process(engine, steps)
    error, scale, where = helpers.max_error(rows, reference)
    assert error <= helpers.TOLERANCE[dtype] * scale, (dtype, error, scale, where)
    engine.cache.check_invariants()

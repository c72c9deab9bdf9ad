"""The real sizes whole: GPT-2 small, medium and XL (12 / 24 / 48 layers, widths 768 / 1024 /
1600, 12 / 16 / 25 heads, vocabulary 50257) against the plain implementation, whole and cut,
in both dtypes.  These sizes take code paths that the tiny models do not (k > 1024 in the
skinny product, 25 heads, a vocabulary that is no multiple of anything, decode steps replayed
from graphs of several hundred launches).  The plain implementation runs its float64 formulas
on the GPU here: on the CPU the XL model alone would take minutes."""

import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu

SHAPES = {
    "small": dict(n_layer=12, n_embd=768, n_head=12, n_inner=3072),
    "medium": dict(n_layer=24, n_embd=1024, n_head=16, n_inner=4096),
    "xl": dict(n_layer=48, n_embd=1600, n_head=25, n_inner=6400),
}
LENGTHS = [37, 21, 50]


@pytest.fixture(scope="module")
def shape_models(tmp_path_factory):
    """name -> (folder, config, requests, {bfloat16?: plain logits}); made when first asked for."""
    base = tmp_path_factory.mktemp("shapes")
    made = {}

    def get(name):
        if name not in made:
            config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "layer_norm_epsilon": 1e-5,
                      "activation_function": "gelu_new", "tie_word_embeddings": True, "vocab_size": 50257,
                      "n_positions": 1024, **SHAPES[name]}
            folder = str(base / name)
            helpers.write_folder(folder, config, helpers.lively_tensors(config, 40 + len(made)))
            requests = {f"s{i}": helpers.random_tokens(n, config["vocab_size"], 900 + i)
                        for i, n in enumerate(LENGTHS)}
            references = {bf16: helpers.plain_logits_of_many(folder, requests, bfloat16=bf16, device="cuda")
                          for bf16 in (False, True)}
            torch.cuda.empty_cache()
            made[name] = (folder, config, requests, references)
        return made[name]

    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))
def test_real_sizes_match_plain(shape_models, name, dtype):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    folder, config, requests, references = shape_models(name)
    reference = references[dtype == "bfloat16"]
    model, _ = load_model(folder, dtype=dtype)
    worst = {}
    cuts = [("whole", helpers.trace_whole), ("mixed", helpers.trace_mixed),
            ("tail", lambda r: helpers.trace_tail_decoded(r, tail=20))]
    if name == "small":
        cuts.append(("portions", helpers.trace_portions))
    for cut, builder in cuts:
        steps = builder(requests)
        pages = helpers.live_token_budget(steps, round_to=16) // 16
        engine = Engine(model, num_pages=pages, page_size=16, max_requests=4, max_step_tokens=256)
        rows = helpers.replay_in_process(engine, steps)
        error, scale, where = helpers.max_error(rows, reference)
        worst[cut] = (error, scale, where)
        assert error <= helpers.TOLERANCE[dtype] * scale, (name, dtype, cut, error, scale, where)
        engine.cache.check_invariants()
        if cut == "tail":
            # the decoded tokens came from replays of a recorded step
            summary = engine.graph_summary()
            assert summary["graph_replays"] >= 3 * 15 and not summary["capture_failures"], summary
            assert max(summary["graph_nodes"].values()) > 5 * config["n_layer"]
    print(name, dtype, {cut: f"{e / s:.2e}" for cut, (e, s, _) in worst.items()})
    del model
    torch.cuda.empty_cache()


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

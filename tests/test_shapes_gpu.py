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
            ("tail", lambda r: helpers.trace_tail_decoded(r, tail=20)),
            ("portions", helpers.trace_portions)]
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,heads,inner,live", [(1600, 25, 6400, 12), (1600, 25, 6400, 40), (1280, 20, 5120, 64),
                                                   (1536, 24, 7680, 33)])
def test_wide_layers_with_many_decoded_tokens_a_step(tmp_path, dtype, width, heads, inner, live):
    """Two layers of GPT-2 large and XL widths with 12 to 64 requests live at once: the decode
    steps take the products' paths for 9 to 16 and for 17 to 64 rows over a k beyond 1,024 (the
    norm inside the product with its columns dealt out evenly, tiles of 64 x 32, two column
    tiles with ranges of k chosen by the number of blocks), which the three-request traces of
    the real sizes above never reach."""
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "layer_norm_epsilon": 1e-5,
              "activation_function": "gelu_new", "tie_word_embeddings": True, "n_layer": 2, "n_embd": width,
              "n_head": heads, "n_inner": inner, "vocab_size": 1000, "n_positions": 128}
    folder = str(tmp_path / "wide")
    helpers.write_folder(folder, config, helpers.lively_tensors(config, 70 + live))
    requests = {f"w{i}": helpers.random_tokens(14 + (i * 7) % 23, config["vocab_size"], 1200 + i)
                for i in range(live + 6)}
    reference = helpers.plain_logits_of_many(folder, requests, bfloat16=dtype == "bfloat16", device="cuda")
    model, _ = load_model(folder, dtype=dtype)
    steps = helpers.trace_mixed(requests, max_live=live, portion=(9, 4, 17, 2), decode_tail=12, seed=live)
    most = max(sum(1 for entry in step["entries"] if len(entry["tokens"]) == 1) for step in steps)
    assert most >= min(live, 17) - 5, most      # steps of that many single tokens do occur
    pages = -(-helpers.live_token_budget(steps, round_to=16) // 16)
    engine = Engine(model, num_pages=pages, page_size=16, max_requests=live, max_step_tokens=1024)
    rows = helpers.replay_in_process(engine, steps)
    error, scale, where = helpers.max_error(rows, reference)
    assert error <= helpers.TOLERANCE[dtype] * scale, (dtype, width, live, error, scale, where)
    engine.cache.check_invariants()


def test_long_prompts_take_tiles_of_128_queries(tmp_path):
    """A step with so many (head, tile) pairs over so many keys that the attention part cuts
    the prompts' queries into tiles of 128 (32 heads of 16 dimensions, three portions of 1,840
    to 2,100 tokens, two of them behind cached prefixes that end inside a page and inside a
    tile): every position's logits against the plain implementation.  The step before it runs
    the tiles of 64 and of 32."""
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model
    from pagedserve_amd.ops import kernels

    length = 2100
    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "layer_norm_epsilon": 1e-5,
              "activation_function": "gelu_new", "tie_word_embeddings": True, "n_layer": 2, "n_embd": 512,
              "n_head": 32, "n_inner": 256, "vocab_size": 333, "n_positions": 2304}
    folder = str(tmp_path / "many_heads")
    helpers.write_folder(folder, config, helpers.lively_tensors(config, 83))
    requests = {name: helpers.random_tokens(length, config["vocab_size"], 1300 + i) for i, name in enumerate("abc")}
    reference = helpers.plain_logits_of_many(folder, requests, bfloat16=True, device="cuda")
    cuts = {"a": 100, "b": 260}
    first = [{"id": rid, "tokens": requests[rid][:cut], "want": list(range(cut))} for rid, cut in cuts.items()]
    second = [{"id": rid, "tokens": requests[rid][cuts.get(rid, 0):],
               "want": list(range(length - cuts.get(rid, 0)))} for rid in "abc"]
    steps = [{"step": 0, "entries": first, "end": []}, {"step": 1, "entries": second, "end": list("abc")}]
    large = sum(-(-len(entry["tokens"]) // kernels.PREFILL_LARGE_TILE) for entry in second)
    assert kernels.prefill_large_tile_pays(config["n_head"], 16, large, config["n_positions"])
    assert not kernels.prefill_large_tile_pays(config["n_head"], 16, 4, config["n_positions"])
    assert not kernels.prefill_large_tile_pays(config["n_head"], 16, large, 1024)
    model, _ = load_model(folder, dtype="bfloat16")
    engine = Engine(model, num_pages=3 * 132 + 2, page_size=16, max_requests=4, max_step_tokens=6144)
    rows = helpers.replay_in_process(engine, steps)
    assert len(rows) == 3 * length
    error, scale, where = helpers.max_error(rows, reference)
    assert error <= helpers.TOLERANCE["bfloat16"] * scale, (error, scale, where)
    engine.cache.check_invariants()


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_configurations_in_32_bit(tmp_path, seed):
    """Eight configurations drawn at random for each seed (1 to 25 heads of 4 to 256 dimensions,
    inner widths and vocabularies that are multiples of nothing, 1 to 3 layers, pages of 1 to 64
    tokens, both activations, tied and untied heads), each replayed as a mixed trace with
    portions of random sizes and pages that are used again, against the plain implementation
    in 32-bit, where the tolerance leaves no room for a wrong key, page, column or norm.  Every
    kernel meets sizes here that no fixed configuration of the other tests has."""
    import os
    import random

    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    rng = random.Random(seed)
    for trial in range(8):
        heads = rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 25])
        head_dim = rng.choice([4, 8, 12, 16, 20, 24, 32, 40, 48, 64, 72, 80, 96, 112, 128, 144, 192, 256]
                              if heads <= 4 else [4, 8, 16, 20, 24, 32, 48, 64, 80])
        width = heads * head_dim
        positions = rng.choice([96, 160, 256, 300])
        config = {
            "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": rng.choice([1, 1, 2, 3]),
            "n_embd": width, "n_head": heads,
            "n_inner": rng.choice([width, 2 * width, 4 * width, width + 8, 3 * width + 4, 100, 64, 320, 1000]),
            "vocab_size": rng.choice([5, 17, 41, 100, 257, 1000, 2049, 5000]), "n_positions": positions,
            "layer_norm_epsilon": rng.choice([1e-5, 1e-6, 3e-4]),
            "activation_function": rng.choice(["gelu_new", "gelu"]),
            "scale_attn_by_inverse_layer_idx": rng.choice([False, True]),
            "tie_word_embeddings": rng.choice([True, True, False]), "eos_token_id": None,
        }
        page = rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 32, 64])
        folder = helpers.write_folder(os.path.join(str(tmp_path), f"m{trial}"), config,
                                      helpers.lively_tensors(config, 7000 + 100 * seed + trial))
        requests = {f"r{i}": helpers.random_tokens(rng.randint(3, min(90, positions - 2)), config["vocab_size"],
                                                   1000 * seed + 10 * trial + i)
                    for i in range(rng.randint(3, 9))}
        reference = {name: helpers.plain_logits(folder, tokens) for name, tokens in requests.items()}
        model, _ = load_model(folder, dtype="float32")
        max_live = rng.randint(1, 6)
        steps = helpers.trace_mixed(requests, max_live=max_live, portion=tuple(rng.randint(1, 40) for _ in range(4)),
                                    decode_tail=rng.randint(1, 10), seed=trial)
        pages = -(-helpers.live_token_budget(steps, round_to=page) // page) + max_live + 1
        engine = Engine(model, num_pages=pages, page_size=page, max_requests=max_live, max_step_tokens=512)
        rows = helpers.replay_in_process(engine, steps)
        error, scale, where = helpers.max_error(rows, reference)
        assert error <= helpers.TOLERANCE["float32"] * scale, (config, page, error, scale, where)
        engine.cache.check_invariants()
        torch.cuda.synchronize()

"""Each part alone against the plain functions, a model whose run order names a block twice
and lets a call read another call's cache, and a toy mixer with state of its own that is
registered, built and stepped from here without touching the framework's files."""

import math
import os

import pytest
import torch

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    # bfloat16: five times what the parts measure (see tests/test_kernels_gpu.py: _tol)
    return 2e-5 if dtype == torch.float32 else 5e-3


def _ctx(engine_like, requests):
    """A StepContext for whole fresh requests of the given lengths, built by a real Engine's
    packer so that the part sees what it sees in production."""
    from pagedserve_amd.engine import StepEntry

    entries = [StepEntry(f"q{i}", [0] * n, []) for i, n in enumerate(requests)]
    for entry in entries:
        engine_like.cache.admit(entry.request_id)
        engine_like.cache.grow(entry.request_id, len(entry.tokens))
    ctx, _, _ = engine_like._pack(entries)
    return ctx


def _tiny_engine(tmp_path, which="A", dtype="float32", pages=32):
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import load_model

    folder, config, page_size = helpers.tiny_folder(tmp_path, which)
    model, typed = load_model(folder, dtype=dtype)
    return Engine(model, num_pages=pages, page_size=page_size, max_requests=8, max_step_tokens=128), folder, config


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_parts(dtype):
    from pagedserve_amd.parts import NORMS

    width = 80
    g = torch.Generator().manual_seed(0)
    h = torch.randn(9, width, generator=g).cuda()
    gamma, beta = torch.randn(width, generator=g).cuda(), torch.randn(width, generator=g).cuda()
    part = NORMS["layernorm"](width=width, dtype=dtype, eps=1e-6)
    assert set(part.parameters()) == {"gamma", "beta"}
    part.bind({"gamma": gamma, "beta": beta})
    out = torch.empty(9, width, dtype=dtype, device="cuda")
    part.forward(h, out)
    expected = P.layer_norm(h.double().cpu(), gamma.double().cpu(), beta.double().cpu(), 1e-6)
    torch.testing.assert_close(out.double().cpu(), expected, atol=_tol(dtype), rtol=_tol(dtype))
    rms = NORMS["rmsnorm"](width=width, dtype=dtype, eps=1e-6)
    rms.bind({"gamma": gamma})
    rms.forward(h, out)
    hd = h.double().cpu()
    expected = hd / torch.sqrt((hd * hd).mean(-1, keepdim=True) + 1e-6) * gamma.double().cpu()
    torch.testing.assert_close(out.double().cpu(), expected, atol=_tol(dtype), rtol=_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["gelu_tanh", "gelu_erf"])
def test_feed_forward_part(tmp_path, dtype, activation):
    from pagedserve_amd.parts import FEED_FORWARDS

    engine, _, _ = _tiny_engine(tmp_path, dtype="float32" if dtype == torch.float32 else "bfloat16")
    width, inner, tokens = 96, 200, 13
    g = torch.Generator().manual_seed(1)
    tensors = {"up.weight": (torch.randn(inner, width, generator=g) / math.sqrt(width)).to(dtype).cuda(),
               "up.bias": torch.randn(inner, generator=g).cuda(),
               "down.weight": (torch.randn(width, inner, generator=g) / math.sqrt(inner)).to(dtype).cuda(),
               "down.bias": torch.randn(width, generator=g).cuda()}
    part = FEED_FORWARDS["dense"](width=width, dtype=dtype, inner=inner, activation=activation)
    assert {name: spec.shape for name, spec in part.parameters().items()} == {
        "up.weight": (inner, width), "down.weight": (width, inner), "up.bias": (inner,), "down.bias": (width,)}
    part.bind(tensors)
    ctx = _ctx(engine, [tokens])
    x = torch.randn(tokens, width, generator=g).to(dtype).cuda()
    residual = torch.randn(tokens, width, generator=g).cuda()
    before = residual.double().cpu()
    part.forward(x, residual, ctx)
    weights = {"mlp.c_fc.weight": tensors["up.weight"].double().cpu().t(), "mlp.c_fc.bias": tensors["up.bias"].double().cpu(),
               "mlp.c_proj.weight": tensors["down.weight"].double().cpu().t(), "mlp.c_proj.bias": tensors["down.bias"].double().cpu()}
    expected = before + P.mlp_sublayer(x.double().cpu(), weights, "", "gelu_new" if activation == "gelu_tanh" else "gelu")
    torch.testing.assert_close(residual.double().cpu(), expected, atol=_tol(dtype) * 3, rtol=_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_whole_prompts(tmp_path, dtype):
    """The mixer alone on two fresh requests in one step equals the plain attention sub-layer
    on each request; a grouped-query variant (kv heads < heads) equals it with repeated heads."""
    from pagedserve_amd.parts import MIXERS, CacheView

    name = "float32" if dtype == torch.float32 else "bfloat16"
    engine, _, config = _tiny_engine(tmp_path, "A", name)
    width, heads, head_dim = config["n_embd"], config["n_head"], config["n_embd"] // config["n_head"]
    g = torch.Generator().manual_seed(2)
    lengths = [11, 20]
    ctx = _ctx(engine, lengths)
    k_pool, v_pool = engine.cache.entry_pools(0)
    for kv_heads in (heads, heads // 2):
        total = (heads + 2 * kv_heads) * head_dim
        tensors = {"qkv.weight": (torch.randn(total, width, generator=g) * 1.2 / math.sqrt(width)).to(dtype).cuda(),
                   "qkv.bias": (torch.randn(total, generator=g) * 0.1).cuda(),
                   "out.weight": (torch.randn(width, heads * head_dim, generator=g) / math.sqrt(width)).to(dtype).cuda(),
                   "out.bias": (torch.randn(width, generator=g) * 0.1).cuda()}
        part = MIXERS["attention"](width=width, dtype=dtype, heads=heads, kv_heads=kv_heads,
                                   head_dim=head_dim, scale=0.2)
        part.bind(tensors)
        view = CacheView(entry=0, writes=True, group=0,
                         k_pool=k_pool[:, :kv_heads].contiguous(), v_pool=v_pool[:, :kv_heads].contiguous())
        x = torch.randn(sum(lengths), width, generator=g).to(dtype).cuda()
        residual = torch.zeros(sum(lengths), width, device="cuda")
        part.forward(x, residual, ctx, view)
        w = tensors["qkv.weight"].double().cpu()
        b = tensors["qkv.bias"].double().cpu()
        q_rows, kv_rows = heads * head_dim, kv_heads * head_dim
        repeat = heads // kv_heads

        def expand(block):     # [kv_heads*hd, ...] -> [heads*hd, ...]: each kv head serves `repeat` heads
            shape = block.shape[1:]
            return block.reshape(kv_heads, head_dim, *shape).repeat_interleave(repeat, 0).reshape(q_rows, *shape)

        w_full = torch.cat([w[:q_rows], expand(w[q_rows:q_rows + kv_rows]), expand(w[q_rows + kv_rows:])])
        b_full = torch.cat([b[:q_rows], expand(b[q_rows:q_rows + kv_rows]), expand(b[q_rows + kv_rows:])])
        weights = {"attn.c_attn.weight": w_full.t(), "attn.c_attn.bias": b_full,
                   "attn.c_proj.weight": tensors["out.weight"].double().cpu().t(),
                   "attn.c_proj.bias": tensors["out.bias"].double().cpu()}
        start = 0
        for length in lengths:
            expected = P.attention_sublayer(x[start:start + length].double().cpu(), weights, "", heads, 0.2)
            torch.testing.assert_close(residual[start:start + length].double().cpu(), expected,
                                       atol=_tol(dtype) * 3, rtol=_tol(dtype))
            start += length


def test_block_part_is_pre_norm(tmp_path):
    from pagedserve_amd.engine import StepEntry

    engine, folder, config = _tiny_engine(tmp_path, "B", "float32")
    raw, weights = P.read_model_folder(folder)
    ctx = _ctx(engine, [17])
    g = torch.Generator().manual_seed(3)
    h = torch.randn(17, config["n_embd"], generator=g)
    stream = h.clone().cuda()
    engine.model.blocks[1].forward(stream, ctx, engine.views[1])
    expected = P.block(h.double(), weights, raw, 1)
    torch.testing.assert_close(stream.double().cpu(), expected, atol=2e-4, rtol=2e-5)


def _custom_model(tmp_path, schedule, dtype="float32"):
    """Tiny A's parts under another run order (the spec is data; no new model class)."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, resolve_architecture
    from pagedserve_amd.engine import Engine
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.weights import load_parameters

    folder, config, page_size = helpers.tiny_folder(tmp_path, "A")
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    spec = dataclasses.replace(arch.build_spec(typed), schedule=tuple(schedule))
    model = DecoderModel(spec, torch.float32 if dtype == "float32" else torch.bfloat16, "cuda")
    tensors = load_parameters(folder, model.parameters(), arch.weight_sources(typed, spec), model.dtype, "cuda",
                              strip_prefixes=arch.strip_prefixes)
    model.bind(tensors)
    engine = Engine(model, num_pages=24, page_size=page_size, max_requests=4, max_step_tokens=64)
    return engine, folder, config


def test_run_order_may_repeat_a_block_and_share_a_cache(tmp_path):
    from pagedserve_amd.config import LayerCall
    from pagedserve_amd.engine import StepEntry

    schedule = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 1, writes_cache=False)]
    engine, folder, config = _custom_model(tmp_path, schedule)
    assert len(engine.cache.groups) == 1 and engine.cache.groups[0].entries == (0, 1, 2)
    raw, weights = P.read_model_folder(folder)
    tokens = helpers.random_tokens(23, config["vocab_size"], 700)

    def plain(ids):
        ids_t = torch.tensor(ids)
        h = P.embed(weights["wte.weight"], weights["wpe.weight"], ids_t, torch.arange(len(ids)))
        h = P.block(h, weights, raw, 0)
        eps = raw["layer_norm_epsilon"]
        # block 1 writes cache entry 1 ...
        normed1 = P.layer_norm(h, weights["h.1.ln_1.weight"], weights["h.1.ln_1.bias"], eps)
        qkv1 = P.conv1d(normed1, weights["h.1.attn.c_attn.weight"], weights["h.1.attn.c_attn.bias"])
        h = P.block(h, weights, raw, 1)
        h = P.block(h, weights, raw, 0)          # block 0 again, with keys of its own (entry 2)
        # ... and its second call attends with new queries over the keys and values of its first call
        d, heads = raw["n_embd"], raw["n_head"]
        normed = P.layer_norm(h, weights["h.1.ln_1.weight"], weights["h.1.ln_1.bias"], eps)
        q = P.conv1d(normed, weights["h.1.attn.c_attn.weight"], weights["h.1.attn.c_attn.bias"])[:, :d]
        context = P.causal_attention(P.split_heads(q, heads), P.split_heads(qkv1[:, d:2 * d], heads),
                                     P.split_heads(qkv1[:, 2 * d:], heads), P.attention_scale(raw, 1))
        h = h + P.conv1d(P.merge_heads(context), weights["h.1.attn.c_proj.weight"], weights["h.1.attn.c_proj.bias"])
        normed = P.layer_norm(h, weights["h.1.ln_2.weight"], weights["h.1.ln_2.bias"], eps)
        h = h + P.mlp_sublayer(normed, weights, "h.1.", raw["activation_function"])
        return P.lm_head(h, weights, raw)

    expected = plain(tokens)
    whole = engine.step([StepEntry("w", tokens, list(range(23)))]).logits.double().cpu()
    assert float((whole - expected).abs().max()) <= 2e-5 * float(expected.abs().max())
    rows = []
    for start, size in ((0, 9), (9, 2), (11, 12)):
        rows.append(engine.step([StepEntry("c", tokens[start:start + size], list(range(size)))]).logits.double().cpu())
    cut = torch.cat(rows)
    assert float((cut - expected).abs().max()) <= 2e-5 * float(expected.abs().max())


def test_toy_mixer_with_state_of_its_own(tmp_path):
    """A running mean of the inputs of each request: state [width] per slot plus a count.
    Registered here; the framework's files know nothing of it."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, PartSpec, resolve_architecture
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.parts import MIXERS, Mixer, SlotStateSpec, register_mixer
    from pagedserve_amd.weights import MATRIX, ParamSpec, WeightSource, load_parameters

    if "toy_running_mean" not in MIXERS:
        @register_mixer("toy_running_mean")
        class RunningMean(Mixer):
            def __init__(self, width, dtype, gain):
                self.width, self.dtype, self.gain = width, dtype, gain

            def parameters(self):
                return {"mix.weight": ParamSpec((self.width, self.width), MATRIX)}

            def cache_spec(self):
                return SlotStateSpec((self.width + 1,), torch.float32)

            def forward(self, x, residual, ctx, cache):
                for item in ctx.items:                       # host loop: a toy, not a kernel
                    rows = slice(item.offset, item.offset + item.count)
                    state = cache.state[item.slot]
                    values = x[rows].float()
                    sums = state[:self.width] + values.cumsum(0)
                    counts = state[self.width] + torch.arange(1, item.count + 1, device=x.device)
                    mean = sums / counts.unsqueeze(1)
                    residual[rows] += self.gain * (mean @ self.mix_weight.float().t())
                    state[:self.width] = sums[-1]
                    state[self.width] = counts[-1]

    folder, config, page_size = helpers.tiny_folder(tmp_path, "A")
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    base = arch.build_spec(typed)
    toy_block = base.blocks[1].with_part("mixer", PartSpec.make("toy_running_mean", gain=0.5))
    spec = dataclasses.replace(base, blocks=(base.blocks[0], toy_block))
    model = DecoderModel(spec, torch.float32, "cuda")
    sources = arch.weight_sources(typed, base)
    sources = {k: v for k, v in sources.items() if not k.startswith("blocks.1.mixer.")}
    sources["blocks.1.mixer.mix.weight"] = WeightSource("h.1.attn.c_proj.weight", transpose=True)
    tensors = load_parameters(folder, model.parameters(), sources, torch.float32, "cuda",
                              strip_prefixes=arch.strip_prefixes,
                              ignorable=lambda name: name.startswith("h.1.attn."))
    model.bind(tensors)
    groups, states = model.cache_requirements()
    assert [g.entries for g in groups] == [(0,)] and [s.entry for s in states] == [1]
    engine = Engine(model, num_pages=16, page_size=page_size, max_requests=3, max_step_tokens=64)

    raw, weights = P.read_model_folder(folder)

    def plain(ids):
        h = P.embed(weights["wte.weight"], weights["wpe.weight"], torch.tensor(ids), torch.arange(len(ids)))
        h = P.block(h, weights, raw, 0)
        eps = raw["layer_norm_epsilon"]
        normed = P.layer_norm(h, weights["h.1.ln_1.weight"], weights["h.1.ln_1.bias"], eps)
        mean = normed.cumsum(0) / torch.arange(1, len(ids) + 1).unsqueeze(1)
        h = h + 0.5 * (mean @ weights["h.1.attn.c_proj.weight"])
        normed = P.layer_norm(h, weights["h.1.ln_2.weight"], weights["h.1.ln_2.bias"], eps)
        h = h + P.mlp_sublayer(normed, weights, "h.1.", raw["activation_function"])
        return P.lm_head(h, weights, raw)

    a = helpers.random_tokens(19, config["vocab_size"], 800)
    b = helpers.random_tokens(8, config["vocab_size"], 801)
    expected_a, expected_b = plain(a), plain(b)
    got_a, got_b = {}, {}
    plan = [[("a", 0, 7)], [("a", 7, 1), ("b", 0, 5)], [("b", 5, 1), ("a", 8, 9)], [("a", 17, 2), ("b", 6, 2)]]
    for step in plan:
        entries = [StepEntry(rid, (a if rid == "a" else b)[start:start + size], list(range(size)))
                   for rid, start, size in step]
        out = engine.step(entries).logits.double().cpu()
        row = 0
        for rid, start, size in step:
            for i in range(size):
                (got_a if rid == "a" else got_b)[start + i] = out[row]
                row += 1
    for got, expected in ((got_a, expected_a), (got_b, expected_b)):
        error = max(float((got[p] - expected[p]).abs().max()) for p in got)
        assert len(got) == len(expected) and error <= 2e-5 * float(expected.abs().max()), error
    # a new request in a used slot starts from zero state
    engine.finish("a")
    again = engine.step([StepEntry("c", a, list(range(len(a))))]).logits.double().cpu()
    assert float((again - expected_a).abs().max()) <= 2e-5 * float(expected_a.abs().max())


def test_toy_feed_forward_with_routing(tmp_path):
    """A routed feed-forward defined here: router logits in float, the best of four experts
    per token, its output scaled by the router's probability.  Layer 0 keeps the dense
    feed-forward, layer 1 gets the routed one: parts are chosen layer by layer, and the
    framework's files know nothing of this kind."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, PartSpec, resolve_architecture
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.parts import FEED_FORWARDS, FeedForward, register_feed_forward
    from pagedserve_amd.weights import MATRIX, ParamSpec, WeightSource, load_parameters

    experts = 4
    if "toy_routed" not in FEED_FORWARDS:
        @register_feed_forward("toy_routed")
        class Routed(FeedForward):
            def __init__(self, width, dtype, experts, inner):
                self.width, self.dtype, self.experts, self.inner = width, dtype, experts, inner

            def parameters(self):
                return {"router.weight": ParamSpec((self.experts, self.width), MATRIX),
                        "up.weight": ParamSpec((self.experts * self.inner, self.width), MATRIX),
                        "down.weight": ParamSpec((self.width, self.experts * self.inner), MATRIX)}

            def forward(self, x, residual, ctx):
                rows = x[:ctx.tokens].float()
                probabilities = torch.softmax(rows @ self.router_weight.float().t(), dim=-1)
                weight, choice = probabilities.max(dim=-1)
                for expert in range(self.experts):           # host loop: a toy, not a kernel
                    mine = (choice == expert).nonzero().flatten()
                    if mine.numel() == 0:
                        continue
                    cut = slice(expert * self.inner, (expert + 1) * self.inner)
                    hidden = torch.nn.functional.gelu(rows[mine] @ self.up_weight[cut].float().t(),
                                                      approximate="tanh")
                    residual[mine] += weight[mine, None] * (hidden @ self.down_weight[:, cut].float().t())

    config, page_size, seed, prefix = helpers.TINY["A"]
    tensors = helpers.lively_tensors(config, seed)
    generator = torch.Generator().manual_seed(77)
    tensors["h.1.mlp.router.weight"] = torch.randn(experts, config["n_embd"], generator=generator) * 0.5
    folder = helpers.write_folder(os.path.join(str(tmp_path), "routed"), config, tensors, prefix)
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    base = arch.build_spec(typed)
    inner = config["n_inner"] // experts
    routed = base.blocks[1].with_part("feed_forward", PartSpec.make("toy_routed", experts=experts, inner=inner))
    spec = dataclasses.replace(base, blocks=(base.blocks[0], routed))
    model = DecoderModel(spec, torch.float32, "cuda")
    sources = {k: v for k, v in arch.weight_sources(typed, base).items()
               if not k.startswith("blocks.1.feed_forward.")}
    sources["blocks.1.feed_forward.router.weight"] = WeightSource("h.1.mlp.router.weight")
    sources["blocks.1.feed_forward.up.weight"] = WeightSource("h.1.mlp.c_fc.weight", transpose=True)
    sources["blocks.1.feed_forward.down.weight"] = WeightSource("h.1.mlp.c_proj.weight", transpose=True)
    loaded = load_parameters(folder, model.parameters(), sources, torch.float32, "cuda",
                             strip_prefixes=arch.strip_prefixes,
                             ignorable=lambda name: name.startswith("h.1.mlp.c_") and name.endswith(".bias"))
    model.bind(loaded)
    engine = Engine(model, num_pages=16, page_size=page_size, max_requests=3, max_step_tokens=64)

    raw, weights = P.read_model_folder(folder)

    def plain(ids):
        h = P.embed(weights["wte.weight"], weights["wpe.weight"], torch.tensor(ids), torch.arange(len(ids)))
        h = P.block(h, weights, raw, 0)
        eps = raw["layer_norm_epsilon"]
        normed = P.layer_norm(h, weights["h.1.ln_1.weight"], weights["h.1.ln_1.bias"], eps)
        h = h + P.attention_sublayer(normed, weights, "h.1.", raw["n_head"], P.attention_scale(raw, 1))
        normed = P.layer_norm(h, weights["h.1.ln_2.weight"], weights["h.1.ln_2.bias"], eps)
        probabilities = torch.softmax(normed @ weights["h.1.mlp.router.weight"].t(), dim=-1)
        out = torch.zeros_like(h)
        for t in range(len(ids)):
            e = int(probabilities[t].argmax())
            cut = slice(e * inner, (e + 1) * inner)
            hidden = P.gelu_tanh(normed[t] @ weights["h.1.mlp.c_fc.weight"][:, cut])
            out[t] = probabilities[t, e] * (hidden @ weights["h.1.mlp.c_proj.weight"][cut])
        return P.lm_head(h + out, weights, raw), probabilities.argmax(-1)

    ids = helpers.random_tokens(40, config["vocab_size"], 810)
    expected, chosen = plain(ids)
    assert len(set(chosen.tolist())) >= 3            # the tokens really go to different experts
    rows = {}
    for start, size in ((0, 13), (13, 1), (14, 2), (16, 24)):
        out = engine.step([StepEntry("r", ids[start:start + size], list(range(size)))]).logits.double().cpu()
        for i in range(size):
            rows[start + i] = out[i]
    error = max(float((rows[p] - expected[p]).abs().max()) for p in rows)
    assert len(rows) == len(ids) and error <= 2e-5 * float(expected.abs().max()), error


def _rotate(values, positions, head_dim, base=100.0):
    """Pairs (2i, 2i+1) of every head turned by the angle position * base^(-2i/head_dim)."""
    heads = values.shape[-1] // head_dim
    shaped = values.reshape(values.shape[0], heads, head_dim // 2, 2).double()
    inverse = base ** (-torch.arange(0, head_dim, 2, dtype=torch.float64, device=values.device) / head_dim)
    angle = positions.double()[:, None, None] * inverse[None, None, :]
    cos, sin = torch.cos(angle), torch.sin(angle)
    first = shaped[..., 0] * cos - shaped[..., 1] * sin
    second = shaped[..., 0] * sin + shaped[..., 1] * cos
    return torch.stack((first, second), dim=-1).reshape(values.shape)


def test_toy_rotation_is_a_function_of_distances():
    """The toy rotation below is pinned by what a rotary encoding is for: scores of rotated
    queries and keys depend on the distance of their positions only."""
    generator = torch.Generator().manual_seed(5)
    q = torch.randn(6, 32, generator=generator, dtype=torch.float64)
    k = torch.randn(6, 32, generator=generator, dtype=torch.float64)
    positions = torch.tensor([0, 1, 2, 5, 9, 10])
    scores = _rotate(q, positions, 16) @ _rotate(k, positions, 16).t()
    shifted = _rotate(q, positions + 37, 16) @ _rotate(k, positions + 37, 16).t()
    torch.testing.assert_close(scores, shifted, atol=1e-10, rtol=0)
    assert float((scores - q @ k.t()).abs().max()) > 0.1      # and it does turn something


def test_toy_position_encoding_that_rotates_queries_and_keys(tmp_path):
    """Another position encoding, registered here: nothing is added to the embedding, queries
    and keys are rotated before the keys are cached (the hook that the attention part offers).
    Whole prompt, portions and decoded tokens against a plain computation."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, PartSpec, resolve_architecture
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.parts import POSITIONS, PositionEncoding, register_position
    from pagedserve_amd.weights import load_parameters

    if "toy_rotary" not in POSITIONS:
        @register_position("toy_rotary")
        class ToyRotary(PositionEncoding):
            transforms_qk = True

            def __init__(self, width, dtype, head_dim, max_positions=0):
                self.width, self.dtype, self.head_dim, self.max_positions = width, dtype, head_dim, max_positions

            def apply_to_qk(self, q, k, ctx):
                positions = ctx.positions[:q.shape[0]]
                q.copy_(_rotate(q, positions, self.head_dim).to(q.dtype))
                k.copy_(_rotate(k, positions, self.head_dim).to(k.dtype))

    folder, config, page_size = helpers.tiny_folder(tmp_path, "A")
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    base = arch.build_spec(typed)
    head_dim = config["n_embd"] // config["n_head"]
    spec = dataclasses.replace(base, position=PartSpec.make("toy_rotary", head_dim=head_dim,
                                                            max_positions=config["n_positions"]))
    model = DecoderModel(spec, torch.float32, "cuda")
    sources = {k: v for k, v in arch.weight_sources(typed, base).items() if not k.startswith("position.")}
    loaded = load_parameters(folder, model.parameters(), sources, torch.float32, "cuda",
                             strip_prefixes=arch.strip_prefixes,
                             ignorable=lambda name: name == "wpe.weight")
    model.bind(loaded)
    engine = Engine(model, num_pages=16, page_size=page_size, max_requests=3, max_step_tokens=64)

    raw, weights = P.read_model_folder(folder)
    heads = config["n_head"]

    def plain(ids):
        positions = torch.arange(len(ids))
        h = weights["wte.weight"][torch.tensor(ids)].double()
        eps = raw["layer_norm_epsilon"]
        for layer in range(config["n_layer"]):
            prefix = f"h.{layer}."
            normed = P.layer_norm(h, weights[prefix + "ln_1.weight"], weights[prefix + "ln_1.bias"], eps)
            qkv = P.conv1d(normed, weights[prefix + "attn.c_attn.weight"], weights[prefix + "attn.c_attn.bias"])
            q, k, v = qkv.split(config["n_embd"], dim=-1)
            q, k = _rotate(q, positions, head_dim), _rotate(k, positions, head_dim)
            context = P.merge_heads(P.causal_attention(P.split_heads(q, heads), P.split_heads(k, heads),
                                                       P.split_heads(v, heads), P.attention_scale(raw, layer)))
            h = h + P.conv1d(context, weights[prefix + "attn.c_proj.weight"], weights[prefix + "attn.c_proj.bias"])
            normed = P.layer_norm(h, weights[prefix + "ln_2.weight"], weights[prefix + "ln_2.bias"], eps)
            h = h + P.mlp_sublayer(normed, weights, prefix, raw["activation_function"])
        return P.lm_head(h, weights, raw)

    ids = helpers.random_tokens(45, config["vocab_size"], 820)
    expected = plain(ids)
    rows = {}
    for start, size in ((0, 11), (11, 1), (12, 1), (13, 2), (15, 30)):
        out = engine.step([StepEntry("r", ids[start:start + size], list(range(size)))]).logits.double().cpu()
        for i in range(size):
            rows[start + i] = out[i]
    error = max(float((rows[p] - expected[p]).abs().max()) for p in rows)
    assert len(rows) == len(ids) and error <= 2e-5 * float(expected.abs().max()), error


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_windowed_layer_has_pages_of_its_own_and_gives_them_back(tmp_path, dtype):
    """Layer 0 sees all keys, layer 1 the last 20 of them (the attention part's window): two
    cache groups with pools of their own.  Two requests advance in portions and single
    tokens far beyond the window, so pages of the windowed group go back and are used again
    while the requests run; logits against a plain computation with the same window."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, resolve_architecture
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.weights import load_parameters

    window = 20
    folder, config, page_size = helpers.tiny_folder(tmp_path, "A")
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    base = arch.build_spec(typed)
    mixer = base.blocks[1].mixer
    from pagedserve_amd.config import PartSpec
    windowed = base.blocks[1].with_part("mixer", PartSpec.make(mixer.kind, **{**mixer.as_dict(), "window": window}))
    spec = dataclasses.replace(base, blocks=(base.blocks[0], windowed))
    torch_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    model = DecoderModel(spec, torch_dtype, "cuda")
    model.bind(load_parameters(folder, model.parameters(), arch.weight_sources(typed, spec), torch_dtype, "cuda",
                               strip_prefixes=arch.strip_prefixes))
    groups, _ = model.cache_requirements()
    assert sorted(g.window for g in groups) == [0, window]
    # so few pages that the windowed group must reuse what it gave back: two requests of up to
    # 110 tokens need 28 pages of 8 in the full group, the windowed group gets by with far less
    engine = Engine(model, num_pages=30, page_size=page_size, max_requests=2, max_step_tokens=64)

    raw, weights = P.read_model_folder(folder)
    if dtype == "bfloat16":
        weights = P.round_weights_to_bfloat16(weights)
    heads = raw["n_head"]

    def plain(ids):
        h = P.embed(weights["wte.weight"], weights["wpe.weight"], torch.tensor(ids), torch.arange(len(ids)))
        h = P.block(h, weights, raw, 0)
        eps = raw["layer_norm_epsilon"]
        normed = P.layer_norm(h, weights["h.1.ln_1.weight"], weights["h.1.ln_1.bias"], eps)
        qkv = P.conv1d(normed, weights["h.1.attn.c_attn.weight"], weights["h.1.attn.c_attn.bias"])
        q, k, v = qkv.split(raw["n_embd"], dim=-1)
        context = P.causal_attention(P.split_heads(q, heads), P.split_heads(k, heads), P.split_heads(v, heads),
                                     P.attention_scale(raw, 1), window=window)
        h = h + P.conv1d(P.merge_heads(context), weights["h.1.attn.c_proj.weight"], weights["h.1.attn.c_proj.bias"])
        normed = P.layer_norm(h, weights["h.1.ln_2.weight"], weights["h.1.ln_2.bias"], eps)
        h = h + P.mlp_sublayer(normed, weights, "h.1.", raw["activation_function"])
        return P.lm_head(h, weights, raw)

    requests = {"a": helpers.random_tokens(110, config["vocab_size"], 830),
                "b": helpers.random_tokens(97, config["vocab_size"], 831)}
    expected = {rid: plain(ids) for rid, ids in requests.items()}
    # the window really matters for these weights
    unwindowed = helpers.plain_logits(folder, requests["a"], bfloat16=dtype == "bfloat16")
    assert float((unwindowed[-1] - expected["a"][-1]).abs().max()) > 1e-3 * float(expected["a"].abs().max())

    plan = [[("a", 33)], [("a", 1), ("b", 41)], [("a", 7), ("b", 1)], [("a", 1), ("b", 1)], [("a", 30), ("b", 2)],
            [("b", 37)], [("a", 1), ("b", 1)], [("a", 2), ("b", 13)], [("a", 35), ("b", 1)]]
    done = {"a": 0, "b": 0}
    got = {"a": {}, "b": {}}
    windowed_group = [g for g, spec_ in enumerate(engine.cache.groups) if spec_.window == window][0]
    most_pages = 0
    for step in plan:
        entries = []
        for rid, size in step:
            start = done[rid]
            entries.append(StepEntry(rid, requests[rid][start:start + size], list(range(size))))
        out = engine.step(entries).logits.double().cpu()
        row = 0
        for rid, size in step:
            for i in range(size):
                got[rid][done[rid] + i] = out[row]
                row += 1
            done[rid] += size
        engine.cache.check_invariants()
        most_pages = max(most_pages, engine.cache.pools[windowed_group].num_allocated)
    assert done == {"a": 110, "b": 97}
    # a request holds about window / page pages there, whatever its length
    assert most_pages <= 2 * (-(-window // page_size) + 9)
    tolerance = helpers.TOLERANCE[dtype]
    for rid in requests:
        scale = float(expected[rid].abs().max())
        error = max(float((got[rid][p] - expected[rid][p]).abs().max()) for p in got[rid])
        assert len(got[rid]) == len(requests[rid]) and error <= tolerance * scale, (rid, error, scale)


def test_mixers_may_ask_for_query_tiles_of_different_sizes(tmp_path):
    """Layer 1's mixer is a toy that wants the queries of a prompt portion in tiles of 24 and
    checks what it is handed; layer 0 keeps the attention part with the tiled kernel's 64.  The
    step lists the tiles once per size, each list starting with the tiles that see most keys."""
    import dataclasses

    from pagedserve_amd.config import GPT2Config, PartSpec, resolve_architecture
    from pagedserve_amd.engine import Engine, StepEntry
    from pagedserve_amd.model import DecoderModel
    from pagedserve_amd.ops import kernels
    from pagedserve_amd.parts import MIXERS, Mixer, register_mixer

    seen = []
    if "toy_tiles" not in MIXERS:
        @register_mixer("toy_tiles")
        class Tiles(Mixer):
            query_tile = 24

            def __init__(self, width, dtype):
                self.width, self.dtype = width, dtype

            def forward(self, x, residual, ctx, cache):
                item, q0 = ctx.query_tiles[self.query_tile]
                MIXERS["toy_tiles"].seen.append((item.tolist(), q0.tolist()))

    MIXERS["toy_tiles"].seen = seen
    config, page_size, seed, prefix = helpers.TINY["A"]
    folder = helpers.write_folder(os.path.join(str(tmp_path), "tiles"), config,
                                  helpers.lively_tensors(config, seed), prefix)
    arch = resolve_architecture(config)
    typed = GPT2Config.from_dict(config)
    base = arch.build_spec(typed)
    spec = dataclasses.replace(base, blocks=(base.blocks[0],
                                             base.blocks[1].with_part("mixer", PartSpec.make("toy_tiles"))))
    model = DecoderModel(spec, torch.bfloat16, "cuda")
    assert model.query_tiles == (24, kernels.PREFILL_SMALL_TILE, kernels.PREFILL_TILE, kernels.PREFILL_LARGE_TILE)
    from pagedserve_amd.weights import load_parameters

    sources = {k: v for k, v in arch.weight_sources(typed, base).items()
               if not k.startswith("blocks.1.mixer.")}
    loaded = load_parameters(folder, model.parameters(), sources, torch.bfloat16, "cuda",
                             strip_prefixes=arch.strip_prefixes,
                             ignorable=lambda name: name.startswith("h.1.attn."))
    model.bind(loaded)
    engine = Engine(model, num_pages=40, page_size=page_size, max_requests=4, max_step_tokens=128)
    ids = helpers.random_tokens(120, config["vocab_size"], 3)
    # "a" has 30 keys behind it when its portion of 50 comes; "b" is new and brings 70; "c" one token
    engine.step([StepEntry("a", ids[:30], [])])
    seen.clear()
    out = engine.step([StepEntry("a", ids[30:80], [49]), StepEntry("c", ids[:1], [0]),
                       StepEntry("b", ids[:70], [69])])
    assert out.logits.shape[0] == 3 and bool(torch.isfinite(out.logits).all())
    items, q0 = seen[0]
    # a: tiles at 0, 24, 48 (keys seen 30 + q0); b: 0, 24, 48 (keys seen q0): most keys first
    keys = [(30 if item == 0 else 0) + start for item, start in zip(items, q0)]
    assert sorted(zip(items, q0)) == [(0, 0), (0, 24), (0, 48), (2, 0), (2, 24), (2, 48)]
    assert keys == sorted(keys, reverse=True)
    # the other size's list is what the attention part of layer 0 read (64: one tile of a, two of b)
    assert sorted(zip(*[t.tolist() for t in engine._pack(
        [StepEntry("a", ids[80:90], [])])[0].query_tiles[64]])) == [(0, 0)]

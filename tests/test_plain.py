"""What fixes the plain implementation beside the reference's text: special cases that
reduce to a library routine, closed forms and invariants, each chosen so that a plausible
mistake (a wrong pairing of heads, a norm in the wrong place, a swapped activation, a mask
off by one) fails it.  Whole-model parity with the Hugging Face module, which the
reference's own test checks (testing/test_gpt2.py:12-68), is unpinned here: that test holds
no stored numbers, and library model code is not used as a source."""

import math

import pytest
import torch
from torch.nn import functional as F

import helpers
import plain_gpt2 as P

torch.set_default_dtype(torch.float32)


def _weights(config, seed=0):
    return {name: tensor.double() for name, tensor in helpers.lively_tensors(config, seed).items()}


def test_layer_norm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    # rows (1, 8, 32) x 768 as in testing/test_triton_residual_layernorm.py:7-35
    for rows in (1, 8, 32):
        x = torch.randn(rows, 768, generator=g, dtype=torch.float64)
        gamma = torch.randn(768, generator=g, dtype=torch.float64)
        beta = torch.randn(768, generator=g, dtype=torch.float64)
        for eps in (1e-5, 1e-6):
            torch.testing.assert_close(P.layer_norm(x, gamma, beta, eps),
                                       F.layer_norm(x, (768,), gamma, beta, eps), atol=1e-12, rtol=1e-12)


def test_layer_norm_invariants():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 50, generator=g, dtype=torch.float64)
    ones, zeros = torch.ones(50, dtype=torch.float64), torch.zeros(50, dtype=torch.float64)
    y = P.layer_norm(x, ones, zeros, 1e-5)
    assert y.mean(-1).abs().max() < 1e-12
    variance = x.var(-1, unbiased=False)
    torch.testing.assert_close(y.var(-1, unbiased=False), variance / (variance + 1e-5))
    torch.testing.assert_close(P.layer_norm(x + 7.0, ones, zeros, 1e-5), y, atol=1e-10, rtol=0)
    beta = torch.randn(50, generator=g, dtype=torch.float64)
    torch.testing.assert_close(P.layer_norm(torch.full((1, 50), 3.0, dtype=torch.float64), ones, beta, 1e-5),
                               beta.unsqueeze(0))


def test_gelu_forms():
    x = torch.linspace(-6, 6, 1001, dtype=torch.float64)
    torch.testing.assert_close(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-12, rtol=0)
    torch.testing.assert_close(P.gelu_erf(x), F.gelu(x), atol=1e-12, rtol=0)
    for form in (P.gelu_tanh, P.gelu_erf):
        torch.testing.assert_close(form(x) - form(-x), x, atol=1e-12, rtol=0)
        assert float(form(torch.zeros(1, dtype=torch.float64))) == 0.0
    # the two forms differ by more than the engine's tolerance, so a swapped option shows
    assert float((P.gelu_tanh(x) - P.gelu_erf(x)).abs().max()) > 1e-4
    assert P.ACTIVATIONS["gelu_new"] is P.gelu_tanh and P.ACTIVATIONS["gelu"] is P.gelu_erf


def test_conv1d_is_addmm():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 7, generator=g, dtype=torch.float64)
    w = torch.randn(7, 11, generator=g, dtype=torch.float64)
    b = torch.randn(11, generator=g, dtype=torch.float64)
    torch.testing.assert_close(P.conv1d(x, w, b), torch.addmm(b, x, w))
    # a one-hot row picks a row of the [in, out] matrix
    torch.testing.assert_close(P.conv1d(torch.eye(7, dtype=torch.float64)[3:4], w, torch.zeros(11, dtype=torch.float64)), w[3:4])


def test_causal_attention_is_sdpa():
    g = torch.Generator().manual_seed(3)
    for heads, tokens, head_dim in ((1, 1, 16), (2, 9, 48), (4, 33, 16)):
        q, k, v = (torch.randn(heads, tokens, head_dim, generator=g, dtype=torch.float64) for _ in range(3))
        expected = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        torch.testing.assert_close(P.causal_attention(q, k, v, head_dim ** -0.5), expected, atol=1e-12, rtol=1e-10)
    # first query sees one key: its output is that key's value; equal keys give the mean value
    torch.testing.assert_close(P.causal_attention(q, k, v, 0.25)[:, 0], v[:, 0])
    same = k[:, :1].expand_as(k)
    out = P.causal_attention(q, same, v, 0.25)
    torch.testing.assert_close(out[:, -1], v.mean(1), atol=1e-12, rtol=0)


def test_causal_attention_window():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(1, 12, 8, generator=g, dtype=torch.float64) for _ in range(3))
    out = P.causal_attention(q, k, v, 0.3, window=3)
    for t in range(12):
        lo = max(0, t - 2)
        expected = F.scaled_dot_product_attention(q[:, t:t + 1], k[:, lo:t + 1], v[:, lo:t + 1], scale=0.3)
        torch.testing.assert_close(out[:, t:t + 1], expected, atol=1e-12, rtol=1e-10)


def test_heads_are_contiguous_column_blocks():
    """q = k = v = x through an identity projection: the sub-layer must equal per-head
    attention on column blocks j*hd:(j+1)*hd, merged head-major."""
    g = torch.Generator().manual_seed(5)
    d, heads, tokens = 12, 3, 6
    hd = d // heads
    x = torch.randn(tokens, d, generator=g, dtype=torch.float64)
    eye = torch.eye(d, dtype=torch.float64)
    weights = {"attn.c_attn.weight": torch.cat([eye, 2 * eye, 3 * eye], dim=1),
               "attn.c_attn.bias": torch.zeros(3 * d, dtype=torch.float64),
               "attn.c_proj.weight": eye, "attn.c_proj.bias": torch.zeros(d, dtype=torch.float64)}
    out = P.attention_sublayer(x, weights, "", heads, hd ** -0.5)
    for j in range(heads):
        block = x[:, j * hd:(j + 1) * hd].unsqueeze(0)
        expected = F.scaled_dot_product_attention(block, 2 * block, 3 * block, is_causal=True)[0]
        torch.testing.assert_close(out[:, j * hd:(j + 1) * hd], expected, atol=1e-12, rtol=1e-10)


def test_closed_form_without_sublayers():
    """With both projections into the residual stream zeroed the blocks are identities:
    logits = LN_f(wte[id] + wpe[pos]) @ wte^T."""
    config = dict(helpers.TINY_A)
    weights = _weights(config)
    for name in list(weights):
        if name.endswith("c_proj.weight") or name.endswith("c_proj.bias"):
            weights[name] = torch.zeros_like(weights[name])
    ids = helpers.random_tokens(9, config["vocab_size"], 6)
    h = weights["wte.weight"][ids] + weights["wpe.weight"][torch.arange(9)]
    final = F.layer_norm(h, (config["n_embd"],), weights["ln_f.weight"], weights["ln_f.bias"],
                         config["layer_norm_epsilon"])
    torch.testing.assert_close(P.forward_logits(config, weights, ids), final @ weights["wte.weight"].t())


@pytest.mark.parametrize("which", ["A", "B"])
def test_causality_and_position_table(which):
    config = dict(helpers.TINY[which][0])
    weights = _weights(config, 7)
    ids = helpers.random_tokens(20, config["vocab_size"], 8)
    base = P.forward_logits(config, weights, ids)
    changed = list(ids)
    changed[13] = (changed[13] + 1) % config["vocab_size"]
    other = P.forward_logits(config, weights, changed)
    torch.testing.assert_close(other[:13], base[:13], atol=0, rtol=0)
    assert float((other[13:] - base[13:]).abs().max()) > 1e-3
    # positions enter through the table only: with equal rows a shift of all positions is invisible
    flat = dict(weights)
    flat["wpe.weight"] = weights["wpe.weight"][:1].expand_as(weights["wpe.weight"]).clone()
    torch.testing.assert_close(P.forward_logits(config, flat, ids, first_position=0),
                               P.forward_logits(config, flat, ids, first_position=17), atol=1e-12, rtol=0)
    assert float((P.forward_logits(config, weights, ids, first_position=17) - base).abs().max()) > 1e-3


def test_inverse_layer_scaling():
    """config.json's ``scale_attn_by_inverse_layer_idx`` divides the scores of layer i (from
    0) by i + 1: the key's documented meaning; the reference never reads it, so nothing in the
    reference pins it.  What can be pinned: the scale is one multiplication of the scores, so
    the option equals a model without it whose query weights of layer i are divided by i + 1."""
    config = dict(helpers.TINY_B)
    weights = _weights(config, 9)
    ids = helpers.random_tokens(12, config["vocab_size"], 10)
    folded = dict(weights)
    d = config["n_embd"]
    for layer in range(config["n_layer"]):
        w = weights[f"h.{layer}.attn.c_attn.weight"].clone()
        bias = weights[f"h.{layer}.attn.c_attn.bias"].clone()
        w[:, :d] /= layer + 1
        bias[:d] /= layer + 1
        folded[f"h.{layer}.attn.c_attn.weight"], folded[f"h.{layer}.attn.c_attn.bias"] = w, bias
    torch.testing.assert_close(P.forward_logits(config, weights, ids),
                               P.forward_logits(dict(config, scale_attn_by_inverse_layer_idx=False), folded, ids),
                               atol=1e-10, rtol=1e-10)
    assert P.attention_scale(config, 0) == pytest.approx(48 ** -0.5)
    assert P.attention_scale(config, 2) == pytest.approx(48 ** -0.5 / 3)
    one_layer = dict(config, n_layer=1)
    off = dict(one_layer, scale_attn_by_inverse_layer_idx=False)
    # layer 0 is divided by 1: the option changes nothing in a one-layer model ...
    torch.testing.assert_close(P.forward_logits(one_layer, weights, ids), P.forward_logits(off, weights, ids), atol=0, rtol=0)
    # ... and does in deeper ones
    deep_off = dict(config, scale_attn_by_inverse_layer_idx=False)
    assert float((P.forward_logits(config, weights, ids) - P.forward_logits(deep_off, weights, ids)).abs().max()) > 1e-3


def test_norms_stand_before_the_sublayers():
    """Pre-norm: a norm only feeds its sub-layer, the stream itself is never normed.  LayerNorm
    forgets a positive factor, so with the feed-forward's output projection zeroed
    block(3 h) - block(h) = 2 h (the attention term is the same for both), and likewise with
    the attention's output projection zeroed.  A block that norms after the sum, or norms the
    stream in place, gives a bounded difference instead."""
    config = dict(helpers.TINY_A, n_layer=1, layer_norm_epsilon=1e-12)
    g = torch.Generator().manual_seed(12)
    h = torch.randn(7, config["n_embd"], generator=g, dtype=torch.float64)
    for silenced in ("mlp.c_proj", "attn.c_proj"):
        weights = _weights(config, 11)
        for kind in ("weight", "bias"):
            weights[f"h.0.{silenced}.{kind}"] = torch.zeros_like(weights[f"h.0.{silenced}.{kind}"])
        difference = P.block(3.0 * h, weights, config, 0) - P.block(h, weights, config, 0)
        torch.testing.assert_close(difference, 2.0 * h, atol=1e-8, rtol=0)
        # the sub-layer that is left does contribute
        assert float((P.block(h, weights, config, 0) - h).abs().max()) > 1e-2


def test_second_norm_reads_the_stream_after_attention():
    """With the attention's output matrix zeroed its sub-layer adds its output bias b to every
    row, so the block is h + b + MLP(LN2(h + b)), written here with library routines.  A block
    whose second norm reads h, or whose feed-forward result replaces the stream, fails."""
    config = dict(helpers.TINY_B, n_layer=1)
    weights = _weights(config, 21)
    weights["h.0.attn.c_proj.weight"] = torch.zeros_like(weights["h.0.attn.c_proj.weight"])
    b = weights["h.0.attn.c_proj.bias"] * 20.0
    weights["h.0.attn.c_proj.bias"] = b
    g = torch.Generator().manual_seed(22)
    h = torch.randn(5, config["n_embd"], generator=g, dtype=torch.float64)
    stream = h + b
    normed = F.layer_norm(stream, (config["n_embd"],), weights["h.0.ln_2.weight"], weights["h.0.ln_2.bias"],
                          config["layer_norm_epsilon"])
    hidden = F.gelu(torch.addmm(weights["h.0.mlp.c_fc.bias"], normed, weights["h.0.mlp.c_fc.weight"]))
    expected = stream + torch.addmm(weights["h.0.mlp.c_proj.bias"], hidden, weights["h.0.mlp.c_proj.weight"])
    torch.testing.assert_close(P.block(h, weights, config, 0), expected, atol=1e-10, rtol=1e-10)
    wrong = F.layer_norm(h, (config["n_embd"],), weights["h.0.ln_2.weight"], weights["h.0.ln_2.bias"],
                         config["layer_norm_epsilon"])
    assert float((wrong - normed).abs().max()) > 1e-2


def test_untied_head_and_greedy():
    config = dict(helpers.TINY_A, tie_word_embeddings=False)
    weights = _weights(config, 13)
    ids = helpers.random_tokens(6, config["vocab_size"], 14)
    tied = P.forward_logits(dict(config, tie_word_embeddings=True), weights, ids)
    untied = P.forward_logits(config, weights, ids)
    assert float((tied - untied).abs().max()) > 1e-3
    generated = P.greedy_generate(config, weights, ids, 3)
    assert generated[0] == int(torch.argmax(untied[-1]))
    assert len(generated) == 3


def test_bfloat16_rounding_touches_matrices_only():
    weights = _weights(dict(helpers.TINY_A), 15)
    rounded = P.round_weights_to_bfloat16(weights)
    assert torch.equal(rounded["h.0.ln_1.bias"], weights["h.0.ln_1.bias"])
    assert not torch.equal(rounded["wte.weight"], weights["wte.weight"])
    assert torch.equal(rounded["wte.weight"], weights["wte.weight"].to(torch.bfloat16).double())


def test_rounded_stores_change_nothing_but_the_stored_activations():
    """``activations_stored_as(torch.bfloat16)`` rounds what a bfloat16 engine writes to memory
    between kernels and nothing else: switched off it is the identity; switched on the logits
    move by bfloat16 roundings (not more than a few parts in a thousand of the largest), and a
    stored value is a bfloat16 number."""
    import helpers

    config = dict(helpers.TINY_A)
    weights = {name: tensor.double() for name, tensor in helpers.lively_tensors(config, 3).items()}
    ids = helpers.random_tokens(20, config["vocab_size"], 4)
    exact = P.forward_logits(config, weights, ids)
    assert P.stored(exact) is exact
    with P.activations_stored_as(torch.bfloat16):
        rounded = P.forward_logits(config, weights, ids)
        value = P.stored(torch.tensor([1.0 + 2.0 ** -10], dtype=torch.float64))
        assert float(value) == 1.0
    assert P.ACTIVATION_STORAGE is None
    assert torch.equal(exact, P.forward_logits(config, weights, ids))
    change = float((rounded - exact).abs().max() / exact.abs().max())
    assert 1e-5 < change < 1e-2, change

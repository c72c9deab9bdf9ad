"""Shared fixtures of the tests: two tiny GPT-2 configurations that differ in every size
and option, model folders with lively random weights, and trace builders."""

import json
import math
import os

import torch

import plain_gpt2

# Every size and option differs between the two (head count, head size that is / is not a
# power of two, inner width = / != 4x, layers, vocabulary, positions, eps, activation,
# inverse-layer scaling, page size, tensor-name prefix).
TINY_A = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 2, "n_embd": 64, "n_head": 4, "n_inner": 256, "vocab_size": 512,
    "n_positions": 128, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
    "scale_attn_by_inverse_layer_idx": False, "tie_word_embeddings": True, "eos_token_id": 511,
}
TINY_B = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 3, "n_embd": 96, "n_head": 2, "n_inner": 320, "vocab_size": 1000,
    "n_positions": 256, "layer_norm_epsilon": 1e-6, "activation_function": "gelu",
    "scale_attn_by_inverse_layer_idx": True, "tie_word_embeddings": True, "eos_token_id": None,
}
# The sizes of the reference's own GPT-2 test (testing/test_gpt2.py:13-27: vocabulary 41, width
# 16, two heads of 8, inner width 32, tanh GELU) with more positions, so that the traces fit,
# and a head of its own instead of the tied one.
TINY_C = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 2, "n_embd": 16, "n_head": 2, "n_inner": 32, "vocab_size": 41,
    "n_positions": 96, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
    "scale_attn_by_inverse_layer_idx": False, "tie_word_embeddings": False, "eos_token_id": 1,
}
# A head size (20) that is no multiple of 8, widths that are no multiple of 8 either (every
# product takes the plain kernel), a page size that is no power of two.
TINY_D = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 2, "n_embd": 60, "n_head": 3, "n_inner": 100, "vocab_size": 333,
    "n_positions": 160, "layer_norm_epsilon": 3e-6, "activation_function": "gelu",
    "scale_attn_by_inverse_layer_idx": True, "tie_word_embeddings": True, "eos_token_id": None,
}
# configuration, page size, seed of the weights, prefix of the tensor names
TINY = {"A": (TINY_A, 8, 0, "transformer."), "B": (TINY_B, 16, 1, ""),
        "C": (TINY_C, 4, 2, "transformer."), "D": (TINY_D, 12, 3, "")}


def lively_tensors(config, seed):
    """Random checkpoint tensors whose every part matters: non-zero biases, norm scales
    away from 1, shifts away from 0, and query/key weights large enough that attention
    is far from uniform (score std about 1.5), so a wrong key, page or position shows."""
    g = torch.Generator().manual_seed(seed)
    d = config["n_embd"]
    inner = config.get("n_inner") or 4 * d

    def normal(shape, std):
        return torch.randn(shape, generator=g) * std

    tensors = {"wte.weight": normal((config["vocab_size"], d), 0.5),
               "wpe.weight": normal((config["n_positions"], d), 0.5)}
    for i in range(config["n_layer"]):
        h = f"h.{i}."
        tensors[h + "ln_1.weight"] = 1.0 + normal((d,), 0.1)
        tensors[h + "ln_1.bias"] = normal((d,), 0.1)
        qkv = normal((d, 3 * d), 1.0 / math.sqrt(d))
        qkv[:, :2 * d] *= 1.2
        tensors[h + "attn.c_attn.weight"] = qkv
        tensors[h + "attn.c_attn.bias"] = normal((3 * d,), 0.1)
        tensors[h + "attn.c_proj.weight"] = normal((d, d), 0.5 / math.sqrt(d))
        tensors[h + "attn.c_proj.bias"] = normal((d,), 0.1)
        tensors[h + "ln_2.weight"] = 1.0 + normal((d,), 0.1)
        tensors[h + "ln_2.bias"] = normal((d,), 0.1)
        tensors[h + "mlp.c_fc.weight"] = normal((d, inner), 1.0 / math.sqrt(d))
        tensors[h + "mlp.c_fc.bias"] = normal((inner,), 0.1)
        tensors[h + "mlp.c_proj.weight"] = normal((inner, d), 0.5 / math.sqrt(inner))
        tensors[h + "mlp.c_proj.bias"] = normal((d,), 0.1)
    tensors["ln_f.weight"] = 1.0 + normal((d,), 0.1)
    tensors["ln_f.bias"] = normal((d,), 0.1)
    if not config.get("tie_word_embeddings", True):
        tensors["lm_head.weight"] = normal((config["vocab_size"], d), 0.5)
    return tensors


def write_folder(folder, config, tensors, prefix="transformer."):
    """Model folder written with the safetensors package (not the engine's writer)."""
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    stored = {}
    for name, tensor in tensors.items():
        key = name if name.startswith("lm_head.") else prefix + name
        stored[key] = tensor.contiguous()
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config, handle)
    return folder


def tiny_folder(tmp_path, which):
    config, page_size, seed, prefix = TINY[which]
    folder = os.path.join(str(tmp_path), f"tiny_{which}")
    write_folder(folder, config, lively_tensors(config, seed), prefix)
    return folder, config, page_size


def plain_logits(folder, token_ids, bfloat16=False, stored_activations=False):
    """float64 logits [T, V] of the plain implementation; with ``bfloat16`` the matrices
    are first rounded as a bfloat16 engine stores them, and with ``stored_activations`` also
    the activations that such an engine writes to memory between two kernels."""
    config, weights = plain_gpt2.read_model_folder(folder, torch.float64)
    if bfloat16:
        weights = plain_gpt2.round_weights_to_bfloat16(weights)
    if stored_activations:
        with plain_gpt2.activations_stored_as(torch.bfloat16):
            return plain_gpt2.forward_logits(config, weights, token_ids)
    return plain_gpt2.forward_logits(config, weights, token_ids)


def plain_logits_of_many(folder, requests, bfloat16=False, device="cpu"):
    """{request: float64 logits} of the plain implementation with the weights read once; on
    ``device`` the same torch formulas run in float64 (large models take minutes on the CPU)."""
    config, weights = plain_gpt2.read_model_folder(folder, torch.float64)
    if bfloat16:
        weights = plain_gpt2.round_weights_to_bfloat16(weights)
    weights = {name: tensor.to(device) for name, tensor in weights.items()}
    return {rid: plain_gpt2.forward_logits(config, weights, tokens).cpu() for rid, tokens in requests.items()}


def random_tokens(count, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()


# ----------------------------------------------------------------------- traces
# A trace is a list of steps in the format that bin/trace_run reads.

def trace_whole(requests):
    """Each request alone, all tokens in one step, logits everywhere."""
    steps = []
    for rid, tokens in requests.items():
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": list(tokens), "want": list(range(len(tokens)))}], "end": [rid]})
    return steps


def trace_tail_decoded(requests, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, tokens in requests.items():
        tokens = list(tokens)
        head = max(1, len(tokens) - tail)
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": tokens[:head], "want": list(range(head))}], "end": []})
        for index in range(head, len(tokens)):
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": [tokens[index]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def trace_portions(requests, sizes=(7, 2, 13, 3, 2, 16, 5, 2, 9)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, tokens in requests.items():
        tokens = list(tokens)
        cursor, turn = 0, 0
        while cursor < len(tokens):
            size = min(sizes[turn % len(sizes)], len(tokens) - cursor)
            turn += 1
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": tokens[cursor:cursor + size], "want": list(range(size))}],
                "end": []})
            cursor += size
        steps[-1]["end"] = [rid]
    return steps


def trace_mixed(requests, max_live=4, portion=(5, 2, 11, 3), decode_tail=6, seed=0):
    """Up to ``max_live`` live requests: prompt portions of some beside single tokens of
    others in one step; requests end at different times so their pages are used again."""
    g = torch.Generator().manual_seed(seed)
    waiting = [(rid, list(tokens)) for rid, tokens in requests.items()]
    live = {}  # rid -> [tokens, cursor]
    steps = []
    turn = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, tokens = waiting.pop(0)
            live[rid] = [tokens, 0]
        entries, ended = [], []
        for rid in list(live):
            tokens, cursor = live[rid]
            remaining = len(tokens) - cursor
            # sometimes a live request sits a step out
            if len(live) > 1 and int(torch.randint(0, 5, (1,), generator=g)) == 0:
                continue
            if remaining <= decode_tail:
                size = 1
            else:
                size = min(portion[turn % len(portion)], remaining - decode_tail)
                turn += 1
            entries.append({"id": rid, "tokens": tokens[cursor:cursor + size],
                            "want": list(range(size))})
            live[rid][1] = cursor + size
            if cursor + size == len(tokens):
                ended.append(rid)
                del live[rid]
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def live_token_budget(steps, round_to=64):
    """Most tokens that live requests hold at any time, each rounded up to ``round_to``."""
    held, peak = {}, 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(-(-count // round_to) * round_to for count in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def replay_in_process(engine, steps, page_holders=None):
    """Run a trace through an Engine; returns {(request, position): float64 logits row}.
    ``page_holders`` (a dict) collects, per physical page of cache group 0, the requests that
    held it at some time."""
    from pagedserve_amd.engine import StepEntry

    rows = {}
    for step in steps:
        output = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in step["entries"]])
        values = output.logits.double().cpu()
        for index, key in enumerate(output.rows):
            rows[key] = values[index]
        if page_holders is not None:
            for rid, record in engine.cache.requests.items():
                for page in record.tables[0]:
                    if page >= 0:
                        page_holders.setdefault(page, set()).add(rid)
        for rid in step["end"]:
            engine.finish(rid)
    return rows


def max_error(rows, reference):
    """Largest |engine - plain| over all positions and the scale max|plain|."""
    worst, scale, where = 0.0, 0.0, None
    for (rid, position), row in rows.items():
        expected = reference[rid][position]
        error = float((row - expected).abs().max())
        if not math.isfinite(error):
            return float("inf"), 1.0, (rid, position)
        scale = max(scale, float(expected.abs().max()))
        if error > worst:
            worst, where = error, (rid, position)
    return worst, scale, where


# |engine - plain| <= TOLERANCE[dtype] * max|plain logits|.  Measured on MI355X: about 2e-6 in
# float32 and 2e-3 in bfloat16 at every size from the tiny models to GPT-2 small.
TOLERANCE = {"float32": 2e-5, "bfloat16": 4e-3}

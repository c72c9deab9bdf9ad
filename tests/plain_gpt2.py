"""Plain, slow GPT-2 forward over whole sequences: the oracle of the test suite.

One function per part, no cache, no batching, no kernels.  It shares no code with
``pagedserve_amd``: weights are read with the ``safetensors`` package (not the
engine's reader), the configuration is a raw ``config.json`` dict, and every
formula is written out from the reference's text (citations are ``file:line``
under the reference checkout).

Weights are addressed by their Hugging Face names without the ``transformer.``
prefix and stay in the checkpoint's Conv1D layout ``[in, out]`` (``y = x @ W + b``).
"""

import json
import math
import os

import torch


def read_model_folder(folder, dtype=torch.float64):
    """config.json as a dict and the tensors of model.safetensors (prefix stripped)."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
        for name in handle.keys():
            short = name[len("transformer."):] if name.startswith("transformer.") else name
            weights[short] = handle.get_tensor(name).to(dtype)
    return config, weights


def round_weights_to_bfloat16(weights):
    """What a bfloat16 engine stores: matrices rounded to bfloat16.

    Vectors (biases, norm scales) are left alone: the engine keeps a tensor that
    the file stores in 32-bit in 32-bit when it is only used in 32-bit arithmetic.
    """
    rounded = {}
    for name, tensor in weights.items():
        if tensor.ndim >= 2:
            rounded[name] = tensor.to(torch.bfloat16).to(tensor.dtype)
        else:
            rounded[name] = tensor
    return rounded


# None: activations keep the precision of the arithmetic.  torch.bfloat16: the activations that
# an engine writes to memory between two kernels (normed rows, queries / keys / values, the
# attention output, the activated hidden rows) are rounded to that type and back, as a bfloat16
# engine stores them; the residual stream, the statistics and the logits are not (they are
# 32-bit in such an engine).  The formulas are the same either way.
ACTIVATION_STORAGE = None


class activations_stored_as:
    """``with activations_stored_as(torch.bfloat16): forward_logits(...)``."""

    def __init__(self, dtype):
        self.dtype = dtype

    def __enter__(self):
        global ACTIVATION_STORAGE
        self.previous, ACTIVATION_STORAGE = ACTIVATION_STORAGE, self.dtype

    def __exit__(self, *exc):
        global ACTIVATION_STORAGE
        ACTIVATION_STORAGE = self.previous
        return False


def stored(x):
    if ACTIVATION_STORAGE is None:
        return x
    return x.to(ACTIVATION_STORAGE).to(x.dtype)


def embed(wte, wpe, token_ids, positions):
    """h0[t] = wte[id[t]] + wpe[pos[t]]   (src/model/paged_decoder.py:306-314)."""
    return wte[token_ids] + wpe[positions]


def layer_norm(x, gamma, beta, eps):
    """Biased-variance LayerNorm over the last axis.

    mean, centred values, variance of the centred values, rsqrt(var + eps), scale
    and shift (src/kernels/triton_residual_layernorm.py:25-39; the torch module
    with the same eps at src/model/paged_decoder.py:170-177).
    """
    mean = x.mean(dim=-1, keepdim=True)
    centred = x - mean
    variance = (centred * centred).mean(dim=-1, keepdim=True)
    return centred / torch.sqrt(variance + eps) * gamma + beta


def conv1d(x, weight, bias):
    """Checkpoint layout [in, out]: y = x @ W + b  (src/model/gpt2.py:14-17 is the
    transposed copy into a Linear, which computes the same product)."""
    return x @ weight + bias


def gelu_tanh(u):
    """0.5 u (1 + tanh(sqrt(2/pi) (u + 0.044715 u^3)))  ("gelu_tanh",
    src/model/paged_decoder.py:276-277)."""
    return 0.5 * u * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * u ** 3)))


def gelu_erf(u):
    """0.5 u (1 + erf(u / sqrt 2))  ("gelu", src/model/paged_decoder.py:274-275)."""
    return 0.5 * u * (1.0 + torch.erf(u / math.sqrt(2.0)))


ACTIVATIONS = {
    "gelu_new": gelu_tanh,
    "gelu_pytorch_tanh": gelu_tanh,
    "gelu": gelu_erf,
}


def split_heads(x, n_head):
    """[T, d] -> [H, T, hd]; head j is columns j*hd:(j+1)*hd
    (src/model/paged_decoder.py:55-57)."""
    tokens, width = x.shape
    return x.reshape(tokens, n_head, width // n_head).transpose(0, 1)


def merge_heads(x):
    """[H, T, hd] -> [T, d], head-major columns (src/model/paged_decoder.py:59-61)."""
    heads, tokens, head_dim = x.shape
    return x.transpose(0, 1).reshape(tokens, heads * head_dim)


def causal_attention(q, k, v, scale, window=0):
    """softmax(q k^T * scale + causal mask) v for [H, T, hd] tensors.

    Scores, upper-triangle mask with -inf, softmax over keys, weighted values
    (src/model/paged_decoder.py:83-91).  ``window`` > 0 additionally hides keys
    that lie ``window`` or more positions back (not part of GPT-2; used to test
    the attention kernels' window parameter).
    """
    tokens = q.shape[1]
    scores = q @ k.transpose(-1, -2) * scale
    query_pos = torch.arange(tokens, device=q.device).unsqueeze(1)
    key_pos = torch.arange(tokens, device=q.device).unsqueeze(0)
    hidden = key_pos > query_pos
    if window > 0:
        hidden = hidden | (query_pos - key_pos >= window)
    scores = scores.masked_fill(hidden, float("-inf"))
    return torch.softmax(scores, dim=-1) @ v


def attention_scale(config, layer_index):
    """hd^-0.5 (src/model/paged_attention.py:27), divided by (layer_index + 1)
    when config.json sets scale_attn_by_inverse_layer_idx (a GPT-2 config option
    that the reference never reads; 0-based layer index)."""
    head_dim = config["n_embd"] // config["n_head"]
    scale = head_dim ** -0.5
    if config.get("scale_attn_by_inverse_layer_idx", False):
        scale = scale / (layer_index + 1)
    return scale


def attention_sublayer(x, weights, prefix, n_head, scale):
    """Packed QKV projection, thirds, heads, attention, merge, output projection
    (src/model/paged_decoder.py:52-53,75-94)."""
    qkv = stored(conv1d(x, weights[prefix + "attn.c_attn.weight"], weights[prefix + "attn.c_attn.bias"]))
    width = x.shape[-1]
    q, k, v = qkv[:, :width], qkv[:, width:2 * width], qkv[:, 2 * width:]
    context = causal_attention(split_heads(q, n_head), split_heads(k, n_head),
                               split_heads(v, n_head), scale)
    return conv1d(stored(merge_heads(context)), weights[prefix + "attn.c_proj.weight"],
                  weights[prefix + "attn.c_proj.bias"])


def mlp_sublayer(x, weights, prefix, activation):
    """fc, activation, projection (src/model/paged_decoder.py:186-188)."""
    hidden = conv1d(x, weights[prefix + "mlp.c_fc.weight"], weights[prefix + "mlp.c_fc.bias"])
    hidden = stored(ACTIVATIONS[activation](hidden))
    return conv1d(hidden, weights[prefix + "mlp.c_proj.weight"], weights[prefix + "mlp.c_proj.bias"])


def block(h, weights, config, layer_index):
    """Pre-norm block: h + attn(LN1(h)), then + mlp(LN2(.))
    (src/model/paged_decoder.py:181-189)."""
    prefix = f"h.{layer_index}."
    eps = config.get("layer_norm_epsilon", 1e-5)
    normed = stored(layer_norm(h, weights[prefix + "ln_1.weight"], weights[prefix + "ln_1.bias"], eps))
    h = h + attention_sublayer(normed, weights, prefix, config["n_head"],
                               attention_scale(config, layer_index))
    normed = stored(layer_norm(h, weights[prefix + "ln_2.weight"], weights[prefix + "ln_2.bias"], eps))
    return h + mlp_sublayer(normed, weights, prefix, config.get("activation_function", "gelu_new"))


def lm_head(h, weights, config):
    """Final LayerNorm, then logits = f @ wte^T without bias when the head is tied,
    else f @ lm_head.weight^T (src/model/paged_decoder.py:291-301,330)."""
    eps = config.get("layer_norm_epsilon", 1e-5)
    final = stored(layer_norm(h, weights["ln_f.weight"], weights["ln_f.bias"], eps))
    if config.get("tie_word_embeddings", True):
        return final @ weights["wte.weight"].transpose(0, 1)
    return final @ weights["lm_head.weight"].transpose(0, 1)


def forward_logits(config, weights, token_ids, first_position=0):
    """Logits [T, V] at every position of one whole sequence
    (src/model/paged_decoder.py:316-331)."""
    device = weights["wte.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(first_position, first_position + ids.numel(), device=device)
    h = embed(weights["wte.weight"], weights["wpe.weight"], ids, positions)
    for layer_index in range(config["n_layer"]):
        h = block(h, weights, config, layer_index)
    return lm_head(h, weights, config)


def greedy_generate(config, weights, prompt_ids, max_new_tokens):
    """Greedy continuation by re-running the whole sequence for each new token
    (argmax as in src/scheduler/orca_scheduler.py:250; ties to the lowest id)."""
    sequence = list(prompt_ids)
    generated = []
    for _ in range(max_new_tokens):
        logits = forward_logits(config, weights, sequence)
        token = int(torch.argmax(logits[-1]))
        generated.append(token)
        sequence.append(token)
    return generated

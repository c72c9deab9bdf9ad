"""A made-up architecture that lives in the tests only: it shows that a second architecture is
a configuration class, a spec builder, a name map and one registry call, with no change under
``pagedserve_amd/``.  It differs from GPT-2 where a second architecture typically does: query,
key and value matrices are stored apart (and feed one packed product), key/value heads are
grouped, norms are RMS norms, nothing is added for positions, the token rows are scaled, the
head is a matrix of its own with a bias, matrices are stored ``[out, in]`` under the prefix
``model.``, and the second layer looks back over a window only.  It is no model of anyone's.

``plain_logits`` is its formula over a whole sequence in float64, written from this
docstring, sharing nothing with the package."""

import json
import math
import os
from dataclasses import asdict, dataclass

import torch

from pagedserve_amd.config import (Architecture, BlockSpec, ConfigError, LayerCall, ModelSpec,
                                   PartSpec, register_architecture)
from pagedserve_amd.config.registry import ARCHITECTURES
from pagedserve_amd.weights import WeightSource

NAME = "ToyGroupedDecoder"


@dataclass(frozen=True)
class ToyConfig:
    hidden: int
    layers: int
    heads: int
    kv_heads: int
    ffn: int
    vocab: int
    context: int
    rms_eps: float
    embed_scale: float
    window: int

    architecture = NAME

    @classmethod
    def from_dict(cls, raw):
        try:
            config = cls(**{name: raw[name] for name in cls.__dataclass_fields__})
        except KeyError as error:
            raise ConfigError(f"config.json lacks {error}") from None
        if config.hidden % config.heads or config.heads % config.kv_heads:
            raise ConfigError("hidden must divide into heads, heads into kv_heads")
        return config

    def to_dict(self):
        return {"architectures": [NAME], **asdict(self)}

    @property
    def head_dim(self):
        return self.hidden // self.heads


def build_spec(config):
    norm = PartSpec.make("rmsnorm", eps=config.rms_eps)
    blocks = []
    for layer in range(config.layers):
        blocks.append(BlockSpec.make(
            "pre_norm", norm1=norm,
            mixer=PartSpec.make("attention", heads=config.heads, kv_heads=config.kv_heads,
                                head_dim=config.head_dim, scale=config.head_dim ** -0.5,
                                window=config.window if layer % 2 else 0, bias=False),
            norm2=norm,
            feed_forward=PartSpec.make("dense", inner=config.ffn, activation="gelu_tanh", bias=False)))
    return ModelSpec(
        architecture=NAME, vocab_size=config.vocab, width=config.hidden, max_positions=config.context,
        position=PartSpec.make("none"), blocks=tuple(blocks),
        schedule=tuple(LayerCall(i, i) for i in range(config.layers)), final_norm=norm,
        tie_head=False, eos_token_id=None,
        embedding=PartSpec.make("lookup", scale=config.embed_scale),
        head=PartSpec.make("linear", bias=True))


def weight_sources(config, spec):
    sources = {"embedding.table": WeightSource("embed.weight"),
               "final_norm.gamma": WeightSource("final_norm.weight"),
               "head.weight": WeightSource("out.weight"), "head.bias": WeightSource("out.bias")}
    for i in range(config.layers):
        b, l = f"blocks.{i}.", f"layers.{i}."
        sources.update({
            b + "norm1.gamma": WeightSource(l + "attn_norm.weight"),
            # three tensors of the file feed the one packed product
            b + "mixer.qkv.weight": WeightSource((l + "q.weight", l + "k.weight", l + "v.weight"), axis=0),
            b + "mixer.out.weight": WeightSource(l + "o.weight"),
            b + "norm2.gamma": WeightSource(l + "ffn_norm.weight"),
            b + "feed_forward.up.weight": WeightSource(l + "up.weight"),
            b + "feed_forward.down.weight": WeightSource(l + "down.weight"),
        })
    return sources


def random_tensors(config, seed):
    g = torch.Generator().manual_seed(seed)
    d, hd = config.hidden, config.head_dim

    def normal(shape, std):
        return torch.randn(shape, generator=g) * std

    tensors = {"embed.weight": normal((config.vocab, d), 0.5),
               "final_norm.weight": 1.0 + normal((d,), 0.1),
               "out.weight": normal((config.vocab, d), 0.5), "out.bias": normal((config.vocab,), 0.3)}
    for i in range(config.layers):
        l = f"layers.{i}."
        tensors[l + "attn_norm.weight"] = 1.0 + normal((d,), 0.1)
        tensors[l + "q.weight"] = normal((config.heads * hd, d), 1.5 / math.sqrt(d))
        tensors[l + "k.weight"] = normal((config.kv_heads * hd, d), 1.5 / math.sqrt(d))
        tensors[l + "v.weight"] = normal((config.kv_heads * hd, d), 1.0 / math.sqrt(d))
        tensors[l + "o.weight"] = normal((d, config.heads * hd), 0.5 / math.sqrt(d))
        tensors[l + "ffn_norm.weight"] = 1.0 + normal((d,), 0.1)
        tensors[l + "up.weight"] = normal((config.ffn, d), 1.0 / math.sqrt(d))
        tensors[l + "down.weight"] = normal((d, config.ffn), 0.5 / math.sqrt(config.ffn))
    return tensors


def register():
    if NAME not in ARCHITECTURES:
        register_architecture(Architecture(
            name=NAME, config_class=ToyConfig, build_spec=build_spec, weight_sources=weight_sources,
            random_tensors=random_tensors, strip_prefixes=("model.",),
            stored_name=lambda config, name: "model." + name))
    return ARCHITECTURES[NAME]


# ------------------------------------------------------------------ the plain formula
def read_folder(folder, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
        for name in handle.keys():
            assert name.startswith("model.")
            weights[name[len("model."):]] = handle.get_tensor(name).to(dtype)
    return config, weights


def _rms(x, gamma, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gamma


def plain_logits(config, weights, token_ids, bfloat16=False):
    if bfloat16:
        weights = {name: (t.to(torch.bfloat16).to(t.dtype) if t.ndim >= 2 else t) for name, t in weights.items()}
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    tokens = ids.numel()
    d, heads, kv_heads = config["hidden"], config["heads"], config["kv_heads"]
    hd = d // heads
    h = weights["embed.weight"][ids] * config["embed_scale"]
    position = torch.arange(tokens)
    for i in range(config["layers"]):
        l = f"layers.{i}."
        x = _rms(h, weights[l + "attn_norm.weight"], config["rms_eps"])
        q = (x @ weights[l + "q.weight"].t()).reshape(tokens, heads, hd).transpose(0, 1)
        k = (x @ weights[l + "k.weight"].t()).reshape(tokens, kv_heads, hd).transpose(0, 1)
        v = (x @ weights[l + "v.weight"].t()).reshape(tokens, kv_heads, hd).transpose(0, 1)
        k = k.repeat_interleave(heads // kv_heads, 0)      # query head j reads key/value head j // group
        v = v.repeat_interleave(heads // kv_heads, 0)
        scores = q @ k.transpose(1, 2) * hd ** -0.5
        hidden = position[None, :] > position[:, None]
        if i % 2 and config["window"] > 0:
            hidden = hidden | (position[:, None] - position[None, :] >= config["window"])
        weights_ = torch.softmax(scores.masked_fill(hidden, float("-inf")), -1)
        h = h + (weights_ @ v).transpose(0, 1).reshape(tokens, d) @ weights[l + "o.weight"].t()
        x = _rms(h, weights[l + "ffn_norm.weight"], config["rms_eps"])
        u = x @ weights[l + "up.weight"].t()
        u = 0.5 * u * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * u ** 3)))
        h = h + u @ weights[l + "down.weight"].t()
    f = _rms(h, weights["final_norm.weight"], config["rms_eps"])
    return f @ weights["out.weight"].t() + weights["out.bias"]

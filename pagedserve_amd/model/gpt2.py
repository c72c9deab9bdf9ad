"""GPT-2 as data: which parts its layers have, in which order they run, and which
checkpoint tensor feeds each parameter.

The architecture of src/model/paged_decoder.py as src/model/gpt2.py:32-78 fills it:
learned absolute positions, pre-LayerNorm blocks of multi-head attention (key/value
heads = heads) and a GELU feed-forward of width ``n_inner``, a final LayerNorm and a
head tied to the token table.
"""

import math
import re

import torch

from ..config.gpt2 import GPT2Config
from ..config.registry import Architecture, register_architecture
from ..config.spec import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..weights.loader import WeightSource


def build_spec(config: GPT2Config) -> ModelSpec:
    blocks = []
    for layer in range(config.n_layer):
        # scores are scaled by head_dim**-0.5 (src/model/paged_attention.py:27) and, when
        # config.json sets scale_attn_by_inverse_layer_idx, also by 1 / (layer + 1).
        scale = config.head_dim ** -0.5
        if config.scale_attn_by_inverse_layer_idx:
            scale /= layer + 1
        norm = PartSpec.make("layernorm", eps=config.layer_norm_epsilon)
        blocks.append(BlockSpec.make(
            "pre_norm",
            norm1=norm,
            mixer=PartSpec.make("attention", heads=config.n_head, kv_heads=config.n_head,
                                head_dim=config.head_dim, scale=scale, window=0, bias=True),
            norm2=norm,
            feed_forward=PartSpec.make("dense", inner=config.n_inner,
                                       activation=config.activation_kind, bias=True),
        ))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab_size,
        width=config.n_embd,
        max_positions=config.n_positions,
        position=PartSpec.make("learned_absolute", max_positions=config.n_positions),
        blocks=tuple(blocks),
        schedule=tuple(LayerCall(block=i, cache=i) for i in range(config.n_layer)),
        final_norm=PartSpec.make("layernorm", eps=config.layer_norm_epsilon),
        tie_head=config.tie_word_embeddings,
        eos_token_id=config.eos_token_id,
        embedding=PartSpec.make("lookup", scale=1.0),
        head=PartSpec.make("linear", bias=False),
    )


def weight_sources(config: GPT2Config, spec: ModelSpec):
    """Parameter path -> checkpoint tensor.  Conv1D tensors are stored ``[in, out]``
    (src/model/gpt2.py:14-17) and are transposed into ``[out, in]``."""
    sources = {
        "embedding.table": WeightSource("wte.weight"),
        "position.table": WeightSource("wpe.weight"),
        "final_norm.gamma": WeightSource("ln_f.weight"),
        "final_norm.beta": WeightSource("ln_f.bias"),
    }
    if not config.tie_word_embeddings:
        sources["head.weight"] = WeightSource("lm_head.weight")
    for i in range(config.n_layer):
        b, h = f"blocks.{i}.", f"h.{i}."
        sources.update({
            b + "norm1.gamma": WeightSource(h + "ln_1.weight"),
            b + "norm1.beta": WeightSource(h + "ln_1.bias"),
            b + "mixer.qkv.weight": WeightSource(h + "attn.c_attn.weight", transpose=True),
            b + "mixer.qkv.bias": WeightSource(h + "attn.c_attn.bias"),
            b + "mixer.out.weight": WeightSource(h + "attn.c_proj.weight", transpose=True),
            b + "mixer.out.bias": WeightSource(h + "attn.c_proj.bias"),
            b + "norm2.gamma": WeightSource(h + "ln_2.weight"),
            b + "norm2.beta": WeightSource(h + "ln_2.bias"),
            b + "feed_forward.up.weight": WeightSource(h + "mlp.c_fc.weight", transpose=True),
            b + "feed_forward.up.bias": WeightSource(h + "mlp.c_fc.bias"),
            b + "feed_forward.down.weight": WeightSource(h + "mlp.c_proj.weight", transpose=True),
            b + "feed_forward.down.bias": WeightSource(h + "mlp.c_proj.bias"),
        })
    return sources


_MASK_BUFFER = re.compile(r"^h\.\d+\.attn\.(bias|masked_bias)$")


def ignorable(config: GPT2Config, name: str) -> bool:
    """Causal-mask buffers that older checkpoints carry, and the head of a tied model
    (it repeats wte)."""
    if _MASK_BUFFER.match(name):
        return True
    return config.tie_word_embeddings and name == "lm_head.weight"


def random_tensors(config: GPT2Config, seed: int, device="cpu"):
    """Checkpoint tensors of a random model: matrices and tables N(0, 0.02), the two
    projections into the residual stream N(0, 0.02 / sqrt(2 n_layer)), biases 0, norm
    scales 1.  Drawn from one seeded generator in a fixed order, on the CPU unless another
    device is named (a generator of another device draws other numbers: the CPU's are the ones
    that a written folder holds)."""
    generator = torch.Generator(device=device).manual_seed(int(seed))
    d, inner = config.n_embd, config.n_inner

    def normal(shape, std):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std

    residual_std = 0.02 / math.sqrt(2 * config.n_layer)
    tensors = {
        "wte.weight": normal((config.vocab_size, d), 0.02),
        "wpe.weight": normal((config.n_positions, d), 0.02),
    }
    for i in range(config.n_layer):
        h = f"h.{i}."
        tensors[h + "ln_1.weight"] = torch.ones(d, device=device)
        tensors[h + "ln_1.bias"] = torch.zeros(d, device=device)
        tensors[h + "attn.c_attn.weight"] = normal((d, 3 * d), 0.02)
        tensors[h + "attn.c_attn.bias"] = torch.zeros(3 * d, device=device)
        tensors[h + "attn.c_proj.weight"] = normal((d, d), residual_std)
        tensors[h + "attn.c_proj.bias"] = torch.zeros(d, device=device)
        tensors[h + "ln_2.weight"] = torch.ones(d, device=device)
        tensors[h + "ln_2.bias"] = torch.zeros(d, device=device)
        tensors[h + "mlp.c_fc.weight"] = normal((d, inner), 0.02)
        tensors[h + "mlp.c_fc.bias"] = torch.zeros(inner, device=device)
        tensors[h + "mlp.c_proj.weight"] = normal((inner, d), residual_std)
        tensors[h + "mlp.c_proj.bias"] = torch.zeros(d, device=device)
    tensors["ln_f.weight"] = torch.ones(d, device=device)
    tensors["ln_f.bias"] = torch.zeros(d, device=device)
    if not config.tie_word_embeddings:
        tensors["lm_head.weight"] = normal((config.vocab_size, d), 0.02)
    return tensors


# Sizes of the reference's built-in random model (main.py:104-115), as config.json keys.
REFERENCE_PRESET = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "vocab_size": 257,
    "n_embd": 64, "n_layer": 2, "n_head": 4, "n_inner": 256, "n_positions": 128,
    "activation_function": "gelu", "layer_norm_epsilon": 1e-5, "eos_token_id": 256,
}


GPT2 = register_architecture(Architecture(
    name="GPT2LMHeadModel",
    config_class=GPT2Config,
    build_spec=build_spec,
    weight_sources=weight_sources,
    random_tensors=random_tensors,
    ignorable=ignorable,
    model_type="gpt2",
    # tensors lie under "transformer." in GPT2LMHeadModel checkpoints and bare in GPT2Model ones;
    # the head of an untied model is never prefixed
    strip_prefixes=("transformer.",),
    stored_name=lambda config, name: name if name.startswith("lm_head.") else "transformer." + name,
    presets=(("reference", REFERENCE_PRESET),),
))

"""Load a model folder's tensors into the parameters that the parts declare.

The parts say which parameters they have (path, shape, role); the architecture says
which checkpoint tensor feeds each of them and whether it is stored transposed
(GPT-2's Conv1D keeps ``[in, out]``; src/model/gpt2.py:14-17 transposes it into a
Linear, and so does this loader, once, at load).  Everything that is wrong with a
folder is reported in ONE error: tensors that are missing, tensors that nobody
asked for, and tensors of the wrong shape or kind.

Precision: matrices and embedding tables are kept in the engine's dtype (bfloat16
or float32); integer tables become int32; vectors (biases, norm scales) are only
ever used in 32-bit arithmetic and are kept in float32, which holds a bfloat16 or
float16 checkpoint value exactly and leaves a tensor stored in 32-bit as it is.
"""

import os
from dataclasses import dataclass
from typing import Dict, Iterable, Tuple

import torch

from .safetensors_io import SafetensorsFile

MATRIX = "matrix"   # [out, in] operand of a matrix product -> engine dtype
TABLE = "table"     # rows looked up by index               -> engine dtype
VECTOR = "vector"   # bias / norm scale                     -> float32
INTEGER = "integer"  # integer table                         -> int32


@dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    role: str


@dataclass(frozen=True)
class WeightSource:
    """Checkpoint tensor ``name`` (without architecture prefix); ``transpose`` when
    the file stores the matrix as ``[in, out]``."""

    name: str
    transpose: bool = False


class WeightError(ValueError):
    """Everything that is wrong with a checkpoint, in one message."""

    def __init__(self, path, missing, unexpected, wrong_shape, wrong_kind):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_kind = list(wrong_kind)
        lines = [f"cannot load weights from {path}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, found, wanted in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(found)}, expected {list(wanted)}")
        for name, found, wanted in self.wrong_kind:
            lines.append(f"  wrong dtype: {name} is {found}, expected {wanted}")
        super().__init__("\n".join(lines))


_FLOATS = (torch.float64, torch.float32, torch.float16, torch.bfloat16)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def target_dtype(role: str, engine_dtype: torch.dtype) -> torch.dtype:
    if role in (MATRIX, TABLE):
        return engine_dtype
    if role == VECTOR:
        return torch.float32
    if role == INTEGER:
        return torch.int32
    raise ValueError(f"unknown parameter role {role!r}")


def canonical_names(file_names: Iterable[str], strip_prefixes: Tuple[str, ...]) -> Dict[str, str]:
    """Map canonical (prefix-free) names to the names in the file."""
    out = {}
    for name in file_names:
        short = name
        for prefix in strip_prefixes:
            if name.startswith(prefix):
                short = name[len(prefix):]
                break
        # A name that is present both with and without prefix keeps both spellings,
        # so that the second one is reported as unexpected.
        if short in out:
            out[name] = name
        else:
            out[short] = name
    return out


def load_parameters(folder, params: Dict[str, ParamSpec], sources: Dict[str, WeightSource],
                    engine_dtype: torch.dtype, device, strip_prefixes=("transformer.",),
                    ignorable=lambda name: False) -> Dict[str, torch.Tensor]:
    """Tensors for every path of ``params``, on ``device``; raises ``WeightError``."""
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as handle:
        available = canonical_names(handle.names(), strip_prefixes)
        missing, wrong_shape, wrong_kind = [], [], []
        used = set()
        plan = []
        for target, spec in params.items():
            if target not in sources:
                raise KeyError(f"architecture gives no checkpoint name for parameter {target!r}")
            source = sources[target]
            if source.name not in available:
                missing.append(source.name)
                continue
            file_name = available[source.name]
            used.add(source.name)
            found = handle.shape(file_name)
            wanted = tuple(reversed(spec.shape)) if source.transpose else tuple(spec.shape)
            if tuple(found) != wanted:
                wrong_shape.append((file_name, found, wanted))
                continue
            stored = handle.dtype(file_name)
            allowed = _INTS if spec.role == INTEGER else _FLOATS
            if stored not in allowed:
                wrong_kind.append((file_name, stored,
                                   "an integer type" if spec.role == INTEGER else "a float type"))
                continue
            plan.append((target, spec, source, file_name))
        unexpected = sorted(available[name] for name in available
                            if name not in used and not ignorable(name))
        if missing or unexpected or wrong_shape or wrong_kind:
            raise WeightError(path, sorted(set(missing)), unexpected, wrong_shape, wrong_kind)
        loaded = {}
        for target, spec, source, file_name in plan:
            tensor = handle.tensor(file_name)
            if source.transpose:
                tensor = tensor.transpose(0, 1)
            tensor = tensor.to(target_dtype(spec.role, engine_dtype)).contiguous()
            loaded[target] = tensor.to(device)
        return loaded

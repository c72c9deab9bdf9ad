"""Load a model folder's tensors into the parameters that the parts declare.

The parts say which parameters they have (path, shape, role); the architecture says
which checkpoint tensor feeds each of them and whether it is stored transposed
(GPT-2's Conv1D keeps ``[in, out]``; src/model/gpt2.py:14-17 transposes it into a
Linear, and so does this loader, once, at load), or which several tensors are joined into
one parameter, or which slice of a tensor it is.  Everything that is wrong with a
folder is reported in ONE error: tensors that are missing, tensors that nobody
asked for, and tensors of the wrong shape or kind.

Precision: matrices and embedding tables are kept in the engine's dtype (bfloat16
or float32); integer tables become int32; vectors (biases, norm scales) are only
ever used in 32-bit arithmetic and are kept in float32, which holds a bfloat16 or
float16 checkpoint value exactly and leaves a tensor stored in 32-bit as it is.
"""

import os
from dataclasses import dataclass
from typing import Dict, Iterable, Optional, Sequence, Tuple, Union

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
    """Where a parameter comes from in the checkpoint (names without architecture prefix).

    ``name`` is one tensor, or several that are joined along ``axis`` of the parameter (query,
    key and value matrices stored apart that feed one packed product).  ``transpose``: each
    stored tensor is ``[in, out]`` and is turned before joining.  ``rows``: only the slice
    ``[begin, end)`` along axis 0 of the (turned, joined) tensor is the parameter (a packed
    tensor in the file that feeds parameters stored apart)."""

    name: Union[str, Tuple[str, ...]]
    transpose: bool = False
    axis: int = 0
    rows: Optional[Tuple[int, int]] = None

    @property
    def names(self) -> Tuple[str, ...]:
        return (self.name,) if isinstance(self.name, str) else tuple(self.name)

    def label(self) -> str:
        return " + ".join(self.names) + (f" [{self.rows[0]}:{self.rows[1]}]" if self.rows else "")

    def result_shape(self, stored_shapes: Sequence[Tuple[int, ...]]):
        """Shape of the parameter that tensors of these stored shapes give, or ``None`` if
        they cannot be joined."""
        shapes = [tuple(reversed(shape)) if self.transpose else tuple(shape) for shape in stored_shapes]
        first = list(shapes[0])
        if not 0 <= self.axis < len(first):
            return None
        for shape in shapes[1:]:
            if len(shape) != len(first) or any(a != b for i, (a, b) in enumerate(zip(shape, first))
                                               if i != self.axis):
                return None
            first[self.axis] += shape[self.axis]
        if self.rows is not None:
            begin, end = self.rows
            if not 0 <= begin < end <= first[0]:
                return None
            first[0] = end - begin
        return tuple(first)

    def assemble(self, fetch):
        """The parameter's tensor from ``fetch(name) -> stored tensor``."""
        pieces = [fetch(name) for name in self.names]
        if self.transpose:
            pieces = [piece.transpose(0, 1) for piece in pieces]
        tensor = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=self.axis)
        if self.rows is not None:
            tensor = tensor[self.rows[0]:self.rows[1]]
        return tensor


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
            found = found if isinstance(found, str) else list(found)
            lines.append(f"  wrong shape: {name} is {found}, expected {list(wanted)}")
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
                    engine_dtype: torch.dtype, device, strip_prefixes: Tuple[str, ...] = (),
                    ignorable=lambda name: False) -> Dict[str, torch.Tensor]:
    """Tensors for every path of ``params``, on ``device``; raises ``WeightError``.
    ``strip_prefixes`` are the prefixes under which the architecture's checkpoints may store
    their tensors (the architecture's registry entry names them)."""
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
            absent = [name for name in source.names if name not in available]
            if absent:
                missing.extend(absent)
                used.update(name for name in source.names if name in available)
                continue
            used.update(source.names)
            file_names = [available[name] for name in source.names]
            found = source.result_shape([handle.shape(name) for name in file_names])
            if found != tuple(spec.shape):
                if len(file_names) == 1 and source.rows is None:
                    stored = tuple(handle.shape(file_names[0]))
                    wanted = tuple(reversed(spec.shape)) if source.transpose else tuple(spec.shape)
                    wrong_shape.append((file_names[0], stored, wanted))
                else:
                    shapes = " + ".join(str(list(handle.shape(name))) for name in file_names)
                    wrong_shape.append((source.label(), f"stored as {shapes}", spec.shape))
                continue
            allowed = _INTS if spec.role == INTEGER else _FLOATS
            bad = [(name, handle.dtype(name)) for name in file_names if handle.dtype(name) not in allowed]
            if bad:
                wrong_kind.extend((name, stored, "an integer type" if spec.role == INTEGER else "a float type")
                                  for name, stored in bad)
                continue
            plan.append((target, spec, source))
        unexpected = sorted(available[name] for name in available
                            if name not in used and not ignorable(name))
        if missing or unexpected or wrong_shape or wrong_kind:
            raise WeightError(path, sorted(set(missing)), unexpected, wrong_shape, wrong_kind)
        loaded = {}
        for target, spec, source in plan:
            tensor = source.assemble(lambda name: handle.tensor(available[name]))
            loaded[target] = tensor.to(target_dtype(spec.role, engine_dtype)).contiguous().to(device)
        return loaded

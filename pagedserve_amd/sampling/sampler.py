"""Token selection on the GPU from the step's float logits."""

from typing import List, Sequence

import torch

from ..ops import kernels
from .params import SamplingParams, uniform_for


class Sampler:
    """One kernel launch and one device-to-host copy per step.

    Rows with temperature 0 take the argmax (ties to the lowest id); the others are drawn
    by inverse CDF at a uniform number that the host makes from (seed, request, index)."""

    def __init__(self, device, max_rows: int):
        self.device = torch.device(device)
        self.max_rows = max_rows
        self._inv_temperature = torch.zeros(max_rows, dtype=torch.float32, device=self.device)
        self._uniform = torch.zeros(max_rows, dtype=torch.float32, device=self.device)
        self._tokens = torch.zeros(max_rows, dtype=torch.int32, device=self.device)
        self._host = torch.zeros((2, max_rows), dtype=torch.float32, pin_memory=True)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               request_keys: Sequence[int], indices: Sequence[int],
               seeds: Sequence[int]) -> List[int]:
        rows = logits.shape[0]
        if rows == 0:
            return []
        if rows > self.max_rows:
            raise ValueError(f"{rows} rows exceed the sampler's {self.max_rows}")
        if not (len(params) == len(request_keys) == len(indices) == len(seeds) == rows):
            raise ValueError("one parameter set, request key, index and seed per row are needed")
        tokens = self._tokens[:rows]
        if all(p.temperature == 0 for p in params):
            kernels.sample(logits, None, None, tokens)
        else:
            host = self._host[:, :rows]
            for row, (p, key, index, seed) in enumerate(zip(params, request_keys, indices, seeds)):
                host[0, row] = 0.0 if p.temperature == 0 else 1.0 / p.temperature
                host[1, row] = uniform_for(seed, key, index)
            self._inv_temperature[:rows].copy_(host[0], non_blocking=True)
            self._uniform[:rows].copy_(host[1], non_blocking=True)
            kernels.sample(logits, self._inv_temperature[:rows], self._uniform[:rows], tokens)
        return tokens.tolist()

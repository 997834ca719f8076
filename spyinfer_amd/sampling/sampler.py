"""Token choice.  The reference samples greedily on the host with ``std::max_element``
(src/engine/model_runner.cpp:131: the lowest id among equal maxima); temperature sampling is
added here.  Both run on the device; only token ids come back.

The uniform number of a draw is a function of (seed, draw index) alone, so what a request
samples does not depend on the batch it shares or on how its prompt was cut.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence

import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def uniform_for(seed: int, index: int) -> float:
    """Counter-based: splitmix64 of (seed, index) -> a multiple of 2^-24 in [0, 1)."""
    x = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & _MASK
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _MASK
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _MASK
    x ^= x >> 31
    return (x >> 40) / float(1 << 24)


@dataclasses.dataclass
class SamplingParams:
    #: 0 = greedy (first maximum); else softmax(logits / temperature)
    temperature: float = 0.0
    #: most tokens to generate; None = until max_model_len
    max_new_tokens: Optional[int] = None
    #: keep going after the end-of-sequence token (random weights emit it at random)
    ignore_eos: bool = False
    #: seed of this request's draws; None = engine seed + request id
    seed: Optional[int] = None

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.max_new_tokens is not None and self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def sample_device(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
                      indices: Sequence[int]) -> Optional[torch.Tensor]:
        """One token per row of ``logits [R, vocab]``, still on the device (int32 [R]); row r is draw ``indices[r]`` of
        seed ``seeds[r]``.  Nothing waits for the device here."""
        R = logits.shape[0]
        if R == 0:
            return None
        host = self._host_buffer(R)
        flat = host.numpy()
        flat[0] = temperatures
        flat[1] = [uniform_for(s, i) if t > 0 else 0.0 for s, i, t in zip(seeds, indices, temperatures)]
        dev = host.to(self.device, non_blocking=True)
        return ops.sample(logits, dev[0], dev[1])

    @staticmethod
    def _host_buffer(R: int) -> torch.Tensor:
        """Pinned host memory [2, R] for the rows' temperatures and uniform numbers (its copy to the device does not wait)."""
        return torch.empty((2, R), dtype=torch.float32, pin_memory=True)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               indices: Sequence[int]) -> List[int]:
        out = self.sample_device(logits, temperatures, seeds, indices)
        return [] if out is None else [int(x) for x in out.tolist()]

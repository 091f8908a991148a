"""Chooses the next token of each row of logits on the device."""
from __future__ import annotations

import torch

from ..kernels import ops as _ops
from .params import SamplingConfig

_M = (1 << 64) - 1


def uniform_at(seed: int, index: int) -> float:
    """A number in [0, 1) that depends only on (seed, index): a counter run
    through the splitmix64 finaliser, top 24 bits.  The reference seeds a
    thread-local mt19937 from the random device (src/core/runtime/InferRuntime.cu:240),
    which cannot be reproduced; this can, in any batch."""
    x = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & _M
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _M
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _M
    x ^= x >> 31
    return (x >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device, ops=_ops):
        self.device = device
        self.ops = ops

    def sample(self, logits: torch.Tensor, configs: list[SamplingConfig], indices: list[int],
               seen: list | None = None) -> list[int]:
        """One token per row.  ``indices[r]`` is the number of the output token
        row r decides (the counter of its random draw); ``seen[r]`` the tokens
        of its prompt and output so far (needed only with a repetition penalty).
        ``logits`` may be changed in place by the penalty."""
        if logits.shape[0] == 0:
            return []
        return self.sample_on_device(logits, configs, indices, seen).tolist()

    def sample_on_device(self, logits: torch.Tensor, configs: list[SamplingConfig], indices: list[int],
                         seen: list | None = None) -> torch.Tensor:
        """As ``sample``, but the tokens stay on the device (int32 [rows]) and
        nothing waits for them: the caller reads them when it needs them."""
        R = logits.shape[0]
        assert len(configs) == R and len(indices) == R
        if any(c.repetition_penalty != 1.0 for c in configs):
            flat, cu = [], [0]
            for r, c in enumerate(configs):
                if c.repetition_penalty != 1.0 and seen is not None:
                    flat.extend(sorted(set(int(t) for t in seen[r])))
                cu.append(len(flat))
            dev = self.device
            self.ops.repetition_penalty(
                logits, torch.tensor(flat or [0], dtype=torch.int32, device=dev),
                torch.tensor(cu, dtype=torch.int32, device=dev),
                torch.tensor([c.repetition_penalty for c in configs], dtype=torch.float32, device=dev))
        if all(c.greedy for c in configs):
            return self.ops.argmax(logits)
        eff = [c.effective() for c in configs]
        dev = self.device
        temperature = torch.tensor([e[0] for e in eff], dtype=torch.float32, device=dev)
        top_k = torch.tensor([e[1] for e in eff], dtype=torch.int32, device=dev)
        top_p = torch.tensor([e[2] for e in eff], dtype=torch.float32, device=dev)
        min_p = torch.tensor([e[3] for e in eff], dtype=torch.float32, device=dev)
        u = torch.tensor([uniform_at(c.seed, i) for c, i in zip(configs, indices)],
                         dtype=torch.float32, device=dev)
        return self.ops.sample(logits, temperature, u, top_k, top_p, min_p)

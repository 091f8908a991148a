"""Chooses the next token of each row of logits on the device."""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops as _ops
from ..kernels import staging as _staging
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


class SeenTokens:
    """The distinct tokens of a sequence that only grows (a request's prompt and output), kept up
    to date token by token: a repetition penalty needs them at every step, and to make a set of a
    few thousand tokens anew for every request and step costs more than the step itself."""

    def __init__(self):
        self._set: set = set()
        self._buf = np.empty(256, dtype=np.int32)
        self._n = 0
        self._consumed = 0

    def update(self, tokens) -> np.ndarray:
        """``tokens``: the sequence so far, longer than (or as long as) at the last call.
        Returns its distinct tokens, int32, in the order of their first appearance."""
        for t in tokens[self._consumed:]:
            t = int(t)
            if t not in self._set:
                self._set.add(t)
                if self._n == self._buf.size:
                    self._buf = np.concatenate([self._buf, np.empty(self._buf.size, dtype=np.int32)])
                self._buf[self._n] = t
                self._n += 1
        self._consumed = len(tokens)
        return self._buf[:self._n]


class Sampler:
    def __init__(self, device, ops=_ops):
        self.device = device
        self.ops = ops

    def _send(self, columns: list) -> list[torch.Tensor]:
        # (a copy from pageable memory would make the host wait for the step in flight, and a host that
        # waits cannot launch the next step ahead)
        return _staging.send(self.device, columns)

    def sample(self, logits: torch.Tensor, configs: list[SamplingConfig], indices: list[int],
               seen: list | None = None) -> list[int]:
        """One token per row.  ``indices[r]`` is the number of the output token
        row r decides (the counter of its random draw); ``seen[r]`` the tokens
        of its prompt and output so far (needed only with a repetition penalty):
        a sequence, or its distinct tokens as an int32 array (``SeenTokens``).
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
            parts, cu = [], [0]
            for r, c in enumerate(configs):
                if c.repetition_penalty != 1.0 and seen is not None:
                    row = seen[r]
                    if not isinstance(row, np.ndarray):      # a plain sequence: its distinct tokens
                        row = np.unique(np.asarray(row, dtype=np.int32))
                    parts.append(row)
                    cu.append(cu[-1] + row.size)
                else:
                    cu.append(cu[-1])
            flat = np.concatenate(parts) if parts and cu[-1] else np.zeros(1, dtype=np.int32)
            seen_d, cu_d, pen_d = self._send([
                flat.astype(np.int32, copy=False), np.asarray(cu, dtype=np.int32),
                np.asarray([c.repetition_penalty for c in configs], dtype=np.float32)])
            self.ops.repetition_penalty(logits, seen_d, cu_d, pen_d)
        if all(c.greedy for c in configs):
            return self.ops.argmax(logits)
        eff = [c.effective() for c in configs]
        temperature, top_k, top_p, min_p, u = self._send([
            np.asarray([e[0] for e in eff], dtype=np.float32), np.asarray([e[1] for e in eff], dtype=np.int32),
            np.asarray([e[2] for e in eff], dtype=np.float32), np.asarray([e[3] for e in eff], dtype=np.float32),
            np.asarray([uniform_at(c.seed, i) for c, i in zip(configs, indices)], dtype=np.float32)])
        return self.ops.sample(logits, temperature, u, top_k, top_p, min_p)

"""Small tables on their way to the device without making the host wait.

A copy from pageable host memory makes the host wait until the stream has reached it, that is
until everything queued before it has run; a host that waits cannot queue the kernels that
follow, and the device runs dry.  Tables that a step builds on the host (sampling parameters,
the attention's work lists) therefore go through pinned buffers and one asynchronous copy.
"""
from __future__ import annotations

import numpy as np
import torch


class PinnedRing:
    """Columns of 4-byte numbers packed into one pinned buffer and sent with one asynchronous
    copy.  The buffers go round a ring, so that one is written again only several sends after
    its copy was queued (and then waits for that copy, by an event)."""

    def __init__(self, device, ring: int = 8, ints: int = 4096):
        self.device = device
        self._bufs = [torch.empty(ints, dtype=torch.int32, pin_memory=True) for _ in range(ring)]
        self._events = [None] * ring
        self._next = 0

    def send(self, columns: list) -> list[torch.Tensor]:
        """``columns``: numpy arrays of int32 or float32 (any shape).  Returns them as device
        tensors of the same shapes, each starting at a multiple of 16 bytes."""
        offs, total = [], 0
        for c in columns:
            offs.append(total)
            total += (c.size + 3) & ~3
        i = self._next
        self._next = (i + 1) % len(self._bufs)
        if self._events[i] is not None:
            self._events[i].synchronize()
        if total > self._bufs[i].numel():
            self._bufs[i] = torch.empty(max(total, 2 * self._bufs[i].numel()), dtype=torch.int32, pin_memory=True)
        host = self._bufs[i][:max(total, 4)]
        flat = host.numpy()
        for c, o in zip(columns, offs):
            flat[o:o + c.size] = c.reshape(-1).view(np.int32)
        dev = host.to(self.device, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev
        out = []
        for c, o in zip(columns, offs):
            t = dev[o:o + c.size]
            out.append((t.view(torch.float32) if c.dtype == np.float32 else t).view(c.shape))
        return out


_rings: dict = {}


def send(device, columns: list) -> list[torch.Tensor]:
    """``columns`` through the ring of ``device`` (one ring a device, made at its first use)."""
    if torch.device(device).type != "cuda":      # (host tensors, for the work lists' tests: nothing to copy)
        return [torch.from_numpy(np.array(c, copy=True)).to(device) for c in columns]
    key = str(torch.device(device))
    ring = _rings.get(key)
    if ring is None:
        ring = _rings[key] = PinnedRing(torch.device(device))
    return ring.send(columns)

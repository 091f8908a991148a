"""Rotation tables on the host: what two encodings share and what they must not."""
import gc

import torch

from tffinfer_amd.parts.position import _TABLES, RotaryEmbedding


class ScaledRotary(RotaryEmbedding):
    """A law with a parameter of its own: positions divided by ``factor``."""

    def __init__(self, head_dim, theta, factor):
        super().__init__(head_dim, theta)
        self.factor = float(factor)

    def angles(self, max_positions):
        return super().angles(max_positions) / self.factor


def test_encodings_with_the_same_law_share_a_table_and_others_do_not():
    a, b, c = ScaledRotary(16, 1e4, 1.0), ScaledRotary(16, 1e4, 4.0), ScaledRotary(16, 1e4, 4.0)
    ta, tb, tc = (e.cached_table(32, "cpu") for e in (a, b, c))
    assert tb is tc and ta is not tb
    assert not torch.equal(ta, tb)
    assert torch.allclose(tb[4], ta[1])                 # position 4 scaled by 4 is position 1
    plain = RotaryEmbedding(16, 1e4).cached_table(32, "cpu")
    assert plain is not ta and torch.equal(plain, ta)   # another class: a table of its own


def test_a_table_goes_with_the_last_encoding_that_asked_for_it():
    e = ScaledRotary(8, 77.0, 3.0)
    t = e.cached_table(16, "cpu")
    key = [k for k, v in _TABLES.items() if v is t]
    assert len(key) == 1
    assert e.cached_table(16, "cpu") is t               # kept by the encoding itself
    del e, t
    gc.collect()
    assert key[0] not in _TABLES

"""Seeded synthetic encoder inputs for the benchmark configurations.

Each row gets a valid length drawn from a per-configuration distribution;
``input_ids`` are uniform in [1000, vocab) on valid positions and 0 on padding,
``segment_ids`` are 0 on the first half of the valid span and 1 on the rest,
``mask`` is 1 on valid positions.  Trailing all-padding columns are then
dropped to the batch maximum, which is what the reference's frontend does
before calling the engine (utils.py:3-13).
"""
from __future__ import annotations

import numpy as np


def make_inputs(batch: int, seq: int, lengths, vocab: int = 30522, seed: int = 20241,
                prune: bool = True):
    """lengths: array of per-row valid lengths (1..seq)."""
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, dtype=np.int64)
    assert lengths.shape == (batch,) and lengths.min() >= 1 and lengths.max() <= seq
    ids = np.zeros((batch, seq), np.int32)
    seg = np.zeros((batch, seq), np.int32)
    mask = np.zeros((batch, seq), np.int32)
    lo = min(1000, vocab - 1)
    for b in range(batch):
        n = int(lengths[b])
        ids[b, :n] = rng.integers(lo, vocab, size=n)
        seg[b, n // 2:n] = 1
        mask[b, :n] = 1
    if prune:
        m = int(lengths.max())
        ids, seg, mask = ids[:, :m], seg[:, :m], mask[:, :m]
    return (np.ascontiguousarray(ids), np.ascontiguousarray(seg),
            np.ascontiguousarray(mask))


def config_lengths(cfg: int, batch: int, seq: int, seed: int = 20241):
    """Valid-length distributions of the five benchmark configurations."""
    rng = np.random.default_rng(seed + 1000 + cfg)
    if cfg == 0:
        return rng.integers(32, 129, size=batch)
    if cfg == 1:
        return rng.integers(64, 129, size=batch)
    if cfg == 2:
        return rng.integers(100, 201, size=batch)
    if cfg == 3:
        return np.full(batch, seq)
    if cfg == 4:
        short = rng.integers(32, 129, size=batch)
        long_ = rng.integers(384, 513, size=batch)
        pick = rng.random(batch) < 0.7
        return np.where(pick, short, long_)
    raise ValueError(cfg)


# (cfg) -> (large?, batch, seq)
CONFIG_SHAPES = {0: (False, 8, 128), 1: (False, 128, 128), 2: (True, 128, 200),
                 3: (True, 8, 200), 4: (True, 64, 512)}


def config_inputs(cfg: int, batch: int | None = None, seed: int = 20241, vocab: int = 30522):
    large, b, s = CONFIG_SHAPES[cfg]
    if batch is not None:
        b = batch
    lens = config_lengths(cfg, b, s, seed)
    return make_inputs(b, s, lens, vocab=vocab, seed=seed + cfg)

"""Seeded synthetic tensors for the benchmark configurations.

Weights ~ N(0, 0.02) before quantisation, activations ~ N(0, 1), optionally
with 0.1 % of the entries replaced by +-20 (outliers at 20 sigma).  The
generator is numpy's counter-based Philox stream keyed by
seed = 0xC0FFEE ^ config_id (+ a per-tensor stream id), so any tensor can be
regenerated independently of the others.
"""
from __future__ import annotations

import numpy as np

BASE_SEED = 0xC0FFEE

# Llama-3-8B-shaped linears of one decoder layer: name -> (K, N)
LLAMA3_8B_LINEARS = {
    "q_proj": (4096, 4096),
    "k_proj": (4096, 1024),
    "v_proj": (4096, 1024),
    "o_proj": (4096, 4096),
    "gate_proj": (4096, 14336),
    "up_proj": (4096, 14336),
    "down_proj": (14336, 4096),
}


def rng(config_id: int, stream: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.Philox(key=[(BASE_SEED ^ config_id) & 0xFFFFFFFFFFFFFFFF, stream]))


def weights(config_id: int, N: int, K: int, stream: int = 0, std: float = 0.02) -> np.ndarray:
    g = rng(config_id, 2 * stream)
    return (g.standard_normal((N, K), dtype=np.float32) * np.float32(std)).astype(np.float32)


def activations(config_id: int, M: int, K: int, stream: int = 0, outliers: float = 0.0) -> np.ndarray:
    g = rng(config_id, 2 * stream + 1)
    x = g.standard_normal((M, K), dtype=np.float32)
    if outliers > 0.0:
        mask = g.random((M, K)) < outliers
        sign = np.where(g.random((M, K)) < 0.5, np.float32(-20.0), np.float32(20.0))
        x = np.where(mask, sign, x).astype(np.float32)
    return x

"""Seeded synthetic inputs for the five benchmark configurations of the int8
path (shapes and distributions as the benchmark definition states them).

The generator is numpy's PCG64 with seed 0xC0FFEE00 + 16*config + tensor index,
so every box sees the same bytes.
"""
from __future__ import annotations

import numpy as np


def _rng(config: int, tensor: int) -> np.random.Generator:
    return np.random.default_rng(0xC0FFEE00 + 16 * config + tensor)


def normal_f32(config: int, tensor: int, shape, sigma: float = 1.0) -> np.ndarray:
    x = _rng(config, tensor).standard_normal(shape, dtype=np.float32)
    if sigma != 1.0:
        x *= np.float32(sigma)
    return x


def uniform_i8(config: int, tensor: int, shape, lo=-127, hi=127) -> np.ndarray:
    return _rng(config, tensor).integers(lo, hi + 1, shape, dtype=np.int16).astype(np.int8)


def uniform_u8(config: int, tensor: int, shape) -> np.ndarray:
    return _rng(config, tensor).integers(0, 256, shape, dtype=np.uint8)


def uniform_f32(config: int, tensor: int, shape, lo: float, hi: float) -> np.ndarray:
    return _rng(config, tensor).uniform(lo, hi, shape).astype(np.float32)


def config1():
    """A f32[128,768] N(0,1); B i8[768,768] U{-127..127}, b_zp 0, b_scale 0.02."""
    return {"A": normal_f32(1, 0, (128, 768)), "B": uniform_i8(1, 1, (768, 768)),
            "b_zp": np.zeros((), np.int8), "b_scale": np.float32(0.02)}


def config2(rows=8192, cols=32768):
    """X f32[rows,cols] N(0, sigma=2); per-axis (axis=1) scales U[0.005,0.05], uint8 zps."""
    return {"X": normal_f32(2, 0, (rows, cols), 2.0),
            "scale": uniform_f32(2, 1, (cols,), 0.005, 0.05),
            "zp": uniform_u8(2, 2, (cols,))}


def config3(M=512, K=1024, N=4096):
    return {"A": uniform_u8(3, 0, (M, K)), "B": uniform_u8(3, 1, (K, N)),
            "a_scale": np.float32(0.01), "b_scale": np.float32(0.005), "y_scale": np.float32(0.5),
            "a_zp": np.array(128, np.uint8), "b_zp": np.array(120, np.uint8),
            "y_zp": np.array(0, np.uint8)}


CONFIG4_SHAPES = {"qkv": (768, 2304), "out": (768, 768), "ffn_up": (768, 3072),
                  "ffn_down": (3072, 768)}


def config4(name: str, M=4096):
    K, N = CONFIG4_SHAPES[name]
    i = list(CONFIG4_SHAPES).index(name)
    return {"X": normal_f32(4, 4 * i, (M, K)), "W": uniform_i8(4, 4 * i + 1, (K, N)),
            "w_scale": uniform_f32(4, 4 * i + 2, (N,), 1e-3, 1e-2)}


CONFIG5_SHAPES = {"up": (4096, 11008), "down": (11008, 4096)}


def config5(name: str, M=2048):
    K, N = CONFIG5_SHAPES[name]
    i = list(CONFIG5_SHAPES).index(name)
    return {"X": normal_f32(5, 4 * i + (0 if M == 2048 else M), (M, K)),
            "W": uniform_i8(5, 4 * i + 1, (K, N)),
            "w_scale": uniform_f32(5, 4 * i + 2, (N,), 1e-3, 5e-3)}

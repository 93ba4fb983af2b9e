"""Deterministic synthetic inputs for the benchmark/parity workloads (numpy, seed 0).

Generator: ``numpy.random.Generator(numpy.random.Philox(key=seed))``; every tensor
draws from its own child stream ``Philox(key=seed, counter=[tag,0,0,0])`` so a
tensor's bytes do not depend on which other tensors were generated before it.

Weights follow the reference's *symmetric* encode mode
(crates/inference/src/weights/q4_weights.rs:258-274): per block a scale
``s = |N(0, scale_std)| / 7`` (f32), replaced by 1.0 when f16(s) underflows to
zero (``degenerate_safe_scale``, q4_weights.rs:210-216), ``bias = -8*s``, both
stored as f16 bits, and 32 nibbles ``int4 + 8`` with int4 uniform in [-8, 7].
"""
from __future__ import annotations

import zlib

import numpy as np

from .q4_layout import BLOCK_WEIGHTS, pack_blocks

# benchmark workload shapes: name -> (N, K)
DECODE_LAYER_2B = {
    "qkv": (3072, 2048),
    "o": (2048, 2048),
    "gate": (6144, 2048),
    "up": (6144, 2048),
    "down": (2048, 6144),
}
CFG0 = {"gemv": (4096, 1024)}
PREFILL_27B = {"up": (17408, 5120), "down": (5120, 17408)}
LORA_2B = {"q": (2048, 2048), "v": (512, 2048)}
MOE_35B = {"experts": 64, "top_k": 8, "hidden": 2048, "inter": 512, "tokens": 16}


def rng_for(seed: int, tag: str) -> np.random.Generator:
    t = zlib.crc32(tag.encode())
    return np.random.Generator(np.random.Philox(key=seed, counter=[t, 0, 0, 0]))


def q4_weight(n: int, k: int, seed: int = 0, tag: str = "w", scale_std: float = 0.02,
              symmetric_bias: bool = True) -> np.ndarray:
    """Flat u8 array of ``n*(k/32)*20`` bytes in the native layout.

    ``symmetric_bias=False`` draws an independent bias ~ N(0, scale_std) instead of
    ``-8*s`` (exercises the asymmetric mode the layout also carries)."""
    if k % BLOCK_WEIGHTS:
        raise ValueError("K must be a multiple of 32")
    g = rng_for(seed, f"{tag}:{n}x{k}")
    nb = n * (k // BLOCK_WEIGHTS)
    s = (np.abs(g.normal(0.0, scale_std, size=nb)).astype(np.float32) / np.float32(7.0))
    with np.errstate(under="ignore"):
        s16 = s.astype(np.float16)
    dead = ~(s16 > 0)
    s = np.where(dead, np.float32(1.0), s)
    s16 = np.where(dead, np.float16(1.0), s16)
    if symmetric_bias:
        b16 = (np.float32(-8.0) * s).astype(np.float16)
    else:
        b16 = g.normal(0.0, scale_std, size=nb).astype(np.float32).astype(np.float16)
    nib = (g.integers(-8, 8, size=(nb, BLOCK_WEIGHTS), dtype=np.int8) + 8).astype(np.uint8)
    return pack_blocks(s16.view(np.uint16), b16.view(np.uint16), nib)


def activations(m: int, k: int, seed: int = 0, tag: str = "x", dtype=np.float32) -> np.ndarray:
    g = rng_for(seed, f"{tag}:{m}x{k}")
    return g.normal(0.0, 1.0, size=(m, k)).astype(np.float32).astype(dtype)


def lora_pair(rank: int, d_in: int, d_out: int, seed: int = 0, tag: str = "lora",
              std: float = 0.01, dtype=np.float16):
    """A [rank, d_in], B [d_out, rank], entries ~ N(0, std) stored as ``dtype``."""
    g = rng_for(seed, f"{tag}:{rank}:{d_in}:{d_out}")
    a = g.normal(0.0, std, size=(rank, d_in)).astype(np.float32).astype(dtype)
    b = g.normal(0.0, std, size=(d_out, rank)).astype(np.float32).astype(dtype)
    return a, b


def router_logits(tokens: int, experts: int, seed: int = 0, tag: str = "router") -> np.ndarray:
    g = rng_for(seed, f"{tag}:{tokens}x{experts}")
    return g.normal(0.0, 1.0, size=(tokens, experts)).astype(np.float32)

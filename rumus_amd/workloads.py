"""Seeded synthetic inputs for the benchmark configurations.

One generator, ``numpy.random.Generator(PCG64(seed))``, drawing in a fixed
order per configuration and casting to float32, so that tests, the smoke check
and the benchmark all see the same arrays for the same seed.
"""
from __future__ import annotations

import numpy as np


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def int8_linear(seed: int = 0, m: int = 32, k: int = 512, n: int = 512):
    """W [in=k,out=n] ~ N(0,0.02), X [m,k] ~ N(0,1), b [n] ~ N(0,0.01)."""
    r = _rng(seed)
    w = r.normal(0.0, 0.02, (k, n)).astype(np.float32)
    x = r.normal(0.0, 1.0, (m, k)).astype(np.float32)
    b = r.normal(0.0, 0.01, (n,)).astype(np.float32)
    return w, x, b


def w4_gemv(seed: int = 0, m: int = 1, k: int = 4096, n: int = 4096):
    """W [k,n] ~ N(0,0.02), x [m,k] ~ N(0,1); asymmetric g128 is applied by the caller."""
    r = _rng(seed)
    w = r.normal(0.0, 0.02, (k, n)).astype(np.float32)
    x = r.normal(0.0, 1.0, (m, k)).astype(np.float32)
    return w, x


def w4_gemm_actorder(seed: int = 0, m: int = 16, k: int = 4096, n: int = 11008,
                     group_size: int = 128):
    """W, then g_idx = perm(k)//group_size, then X, from one generator."""
    r = _rng(seed)
    w = r.normal(0.0, 0.02, (k, n)).astype(np.float32)
    perm = r.permutation(k)
    g_idx = (perm // group_size).astype(np.int32)
    x = r.normal(0.0, 1.0, (m, k)).astype(np.float32)
    return w, g_idx, x


def int8_gemm(seed: int = 0, m: int = 2048, k: int = 4096, n: int = 11008):
    """X [m,k] ~ N(0,1), W [k,n] ~ N(0,0.02)."""
    r = _rng(seed)
    x = r.normal(0.0, 1.0, (m, k)).astype(np.float32)
    w = r.normal(0.0, 0.02, (k, n)).astype(np.float32)
    return x, w


def decoder_block(dim: int = 4096, ffn: int = 11008, seed0: int = 0):
    """The seven projection matrices of a Llama-shaped block, [in, out] ~ N(0, 0.02), one seed
    each (seed0 .. seed0+6, in the order q, k, v, o, gate, up, down); RMSNorm weights are 1."""
    shapes = {"q": (dim, dim), "k": (dim, dim), "v": (dim, dim), "o": (dim, dim),
              "gate": (dim, ffn), "up": (dim, ffn), "down": (ffn, dim)}
    return {name: _rng(seed0 + i).normal(0.0, 0.02, shp).astype(np.float32)
            for i, (name, shp) in enumerate(shapes.items())}


def decoder_block_inputs(batch: int, n: int, dim: int = 4096, cache_len: int = 0, heads: int = 32,
                         seed: int = 7):
    """Hidden states [batch, n, dim] ~ N(0, 1) (the embedding lookup of random token ids is left
    out: it only selects rows) and, for decode, a K/V cache [batch, cache_len, heads, dim/heads] ~ N(0, 1)."""
    r = _rng(seed)
    x = r.normal(0.0, 1.0, (batch, n, dim)).astype(np.float32)
    if cache_len == 0:
        return x, None, None
    kc = r.normal(0.0, 1.0, (batch, cache_len, heads, dim // heads)).astype(np.float32)
    vc = r.normal(0.0, 1.0, (batch, cache_len, heads, dim // heads)).astype(np.float32)
    return x, kc, vc

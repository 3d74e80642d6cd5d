"""Synthetic workloads of the benchmark (the configurations bench.py and the tests run): shapes, seeded sequence
lengths, masks, inputs and weights, drawn the way the reference's benchmark draws them
(sample/tensorflow/benchmark.py:38-61: lengths `randint(lo, hi)`, mask = position < length, attention mask
[b,q,k] = mask[b,k], inputs N(0,1), dense kernels 0.02*N(0,1), biases 0, LayerNorm gamma 1 / beta 0).  numpy only.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np


def _np_dtype(dtype: str):
    if dtype == "fp32":
        return np.float32
    if dtype == "fp16":
        return np.float16
    raise ValueError("dtype must be 'fp32' or 'fp16'")


@dataclass
class Workload:
    name: str
    seed: int
    dtype: str
    layers: int
    B: int
    S: int
    heads: int
    d: int
    F: int
    lens_lo: int = 0
    lens_hi: int = 0
    bimodal: bool = False

    @property
    def H(self) -> int:
        return self.heads * self.d


WORKLOADS = {
    "cfg1": Workload("cfg1", 0, "fp32", 1, 8, 32, 12, 64, 3072, 8, 33),
    "cfg2": Workload("cfg2", 1, "fp16", 12, 100, 32, 12, 64, 3072, 8, 33),
    "cfg3": Workload("cfg3", 2, "fp16", 12, 1000, 64, 12, 64, 3072, 16, 65),
    "cfg4": Workload("cfg4", 3, "fp32", 12, 500, 64, 12, 64, 3072, 16, 65),
    "cfg5": Workload("cfg5", 4, "fp16", 24, 256, 128, 16, 64, 4096, bimodal=True),
}


def draw_lens(wl: Workload, rng: np.random.RandomState) -> np.ndarray:
    if wl.bimodal:
        short = rng.randint(8, 33, size=wl.B)
        long_ = rng.randint(96, 129, size=wl.B)
        return np.where(rng.random_sample(wl.B) < 0.7, short, long_).astype(np.int32)
    return rng.randint(wl.lens_lo, wl.lens_hi, size=wl.B).astype(np.int32)


def make_masks(wl: Workload, rng: np.random.RandomState):
    """lens, input mask [B,S] int32 and attr_mask[b,q,k] = mask[b,k]
    (sample/tensorflow/benchmark.py:38-61)."""
    lens = draw_lens(wl, rng)
    mask = (np.arange(wl.S)[None, :] < lens[:, None]).astype(np.int32)
    attr_mask = np.ascontiguousarray(np.broadcast_to(mask[:, None, :], (wl.B, wl.S, wl.S))).astype(_np_dtype(wl.dtype))
    return lens, mask, attr_mask


def make_layer_weights(wl: Workload, rng: np.random.RandomState, random_affine: bool = False) -> List[np.ndarray]:
    """One layer's 16 tensors in WEIGHT_SLOTS order: kernels 0.02*N(0,1) [in,out],
    biases 0, beta 0, gamma 1.  random_affine=True instead draws biases, beta and
    gamma at random so that tests can tell the slots apart."""
    H, F = wl.H, wl.F
    dt = _np_dtype(wl.dtype)

    def kern(i, o):
        return (0.02 * rng.randn(i, o)).astype(np.float32).astype(dt)

    def vec(n, base):
        if random_affine:
            return (base + 0.1 * rng.randn(n)).astype(np.float32).astype(dt)
        return np.full(n, base, dtype=dt)

    out = []
    for _ in range(3):                       # q, k, v
        out.append(kern(H, H)); out.append(vec(H, 0.0))
    out.append(kern(H, H)); out.append(vec(H, 0.0))            # attention output dense
    out.append(vec(H, 0.0)); out.append(vec(H, 1.0))            # LN beta, gamma
    out.append(kern(H, F)); out.append(vec(F, 0.0))            # intermediate
    out.append(kern(F, H)); out.append(vec(H, 0.0))            # output dense
    out.append(vec(H, 0.0)); out.append(vec(H, 1.0))            # LN beta, gamma
    return out


def make_workload(name: str, layers: Optional[int] = None, random_affine: bool = False,
                  with_inputs: bool = True):
    """Returns dict(wl, lens, mask, attr_mask, x, weights).  Draw order: lens, x, then
    per-layer weights."""
    wl = WORKLOADS[name]
    rng = np.random.RandomState(wl.seed)
    lens, mask, attr_mask = make_masks(wl, rng)
    x = None
    if with_inputs:
        x = rng.randn(wl.B, wl.S, wl.H).astype(np.float32).astype(_np_dtype(wl.dtype))
    L = wl.layers if layers is None else layers
    weights: List[np.ndarray] = []
    if with_inputs:
        for _ in range(L):
            weights.extend(make_layer_weights(wl, rng, random_affine))
    return dict(wl=wl, lens=lens, mask=mask, attr_mask=attr_mask, x=x, weights=weights)

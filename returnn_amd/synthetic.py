"""
Seeded synthetic inputs for the benchmark configurations of the NativeLstm2 forward op.

All arrays are generated on the host with ``numpy.random.default_rng(seed)`` in float32, in the op's
layout (X [T,B,4n] pre-projected gates, W [n,4n], y0/c0 [B,n], mask i [T,B] float 0/1, right padded).
Lower-precision runs round these same arrays, so every precision sees the identical seeded problem.
"""

from __future__ import annotations

import dataclasses
import math
from typing import Optional

import numpy


@dataclasses.dataclass
class Problem:
    """One op call: inputs of ``NativeLstm2(X, W, y0, c0, i, start, step)`` plus bookkeeping."""

    name: str
    X: numpy.ndarray
    W: numpy.ndarray
    y0: numpy.ndarray
    c0: numpy.ndarray
    i: numpy.ndarray
    start: int
    step: int
    dtype: str  # "f32" or "bf16": the precision the configuration is specified in
    lens: Optional[numpy.ndarray] = None

    @property
    def T(self) -> int:
        return self.i.shape[0]

    @property
    def B(self) -> int:
        return self.i.shape[1]

    @property
    def n(self) -> int:
        return self.y0.shape[1]

    def with_step(self, step: int) -> "Problem":
        """Same inputs, other direction (the bidirectional pair is two calls on the same X layout)."""
        return dataclasses.replace(self, step=step)


# name -> (T, B, n, dtype, ragged lens range or None, W limit, y0/c0 std)
_SPECS = {
    "cfg1": dict(T=32, B=4, n=64, dtype="f32", lens=None, w_lim=1.0 / 8.0, state_std=0.0),
    "cfg2": dict(T=500, B=64, n=512, dtype="f32", lens=(250, 500), w_lim=1.0 / math.sqrt(512.0), state_std=0.01),
    "cfg3": dict(T=1000, B=32, n=1024, dtype="bf16", lens=(500, 1000), w_lim=1.0 / 32.0, state_std=0.0),
    "cfg5": dict(T=4000, B=1, n=1024, dtype="bf16", lens=None, w_lim=1.0 / 32.0, state_std=0.0),
    # not one of the benchmark configurations: a layer whose W (134 MB) cannot stay on chip, read from memory every step
    "wide": dict(T=200, B=16, n=4096, dtype="bf16", lens=None, w_lim=1.0 / 64.0, state_std=0.0),
}


def config_names():
    return sorted(_SPECS)


def make_config(name: str, *, seed: int = 0, T: Optional[int] = None, B: Optional[int] = None, step: int = 1) -> Problem:
    """
    :param name: "cfg1" (T=32,B=4,n=64 fp32), "cfg2" (T=500,B=64,n=512 fp32 ragged),
        "cfg3" (T=1000,B=32,n=1024 bf16 ragged; the bidirectional pair is this with step=+1 and step=-1),
        "cfg5" (T=4000,B=1,n=1024 bf16), "wide" (T=200,B=16,n=4096 bf16: W does not fit on chip)
    :param T: override the number of frames (scaled-down variants for quick checks; lengths scale with it)
    :param B: override the batch size
    :param step: +1 or -1
    """
    spec = _SPECS[name]
    T_full = spec["T"]
    T = T_full if T is None else int(T)
    B = spec["B"] if B is None else int(B)
    n = spec["n"]
    rng = numpy.random.default_rng(seed)
    X = rng.standard_normal((T, B, 4 * n), dtype=numpy.float32)
    X *= numpy.float32(0.1)
    W = rng.uniform(-spec["w_lim"], spec["w_lim"], (n, 4 * n)).astype(numpy.float32)
    if spec["state_std"] > 0:
        y0 = (rng.standard_normal((B, n), dtype=numpy.float32) * numpy.float32(spec["state_std"])).astype(numpy.float32)
        c0 = (rng.standard_normal((B, n), dtype=numpy.float32) * numpy.float32(spec["state_std"])).astype(numpy.float32)
    else:
        y0 = numpy.zeros((B, n), dtype=numpy.float32)
        c0 = numpy.zeros((B, n), dtype=numpy.float32)
    lens = None
    if spec["lens"] is not None:
        lo, hi = spec["lens"]
        lo = max(1, (lo * T) // T_full)
        hi = max(lo, (hi * T) // T_full)
        lens = rng.integers(lo, hi + 1, size=(B,))
        lens[0] = T  # at least one sequence spans the whole batch
        i = (numpy.arange(T)[:, None] < lens[None, :]).astype(numpy.float32)
    else:
        i = numpy.ones((T, B), dtype=numpy.float32)
    return Problem(name=name, X=X, W=W, y0=y0, c0=c0, i=i, start=0, step=step, dtype=spec["dtype"], lens=lens)


def round_to_bf16(a: numpy.ndarray) -> numpy.ndarray:
    """float32 -> nearest-even bfloat16, returned as float32 (for feeding an fp32 checker the values a bf16 run sees)."""
    a = numpy.ascontiguousarray(a, dtype=numpy.float32)
    u = a.view(numpy.uint32)
    rounded = (u + numpy.uint32(0x7FFF) + ((u >> numpy.uint32(16)) & numpy.uint32(1))) & numpy.uint32(0xFFFF0000)
    out = rounded.view(numpy.float32).copy()
    nan = numpy.isnan(a)
    out[nan] = numpy.nan
    return out


@dataclasses.dataclass
class EncoderProblem:
    """A stack of bidirectional LSTM layers: features, lengths and per layer and direction the frontend parameters."""

    name: str
    features: numpy.ndarray  # [T,B,in]
    lens: numpy.ndarray  # [B]
    layers: list  # per layer {"fwd": params, "bwd": params}; params = {"ff_weight" [4n,in_l], "rec_weight" [4n,n], "bias" [4n]}
    n: int
    dtype: str

    @property
    def T(self) -> int:
        return self.features.shape[0]

    @property
    def B(self) -> int:
        return self.features.shape[1]

    @property
    def in_dim(self) -> int:
        return self.features.shape[2]

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def glorot_uniform(rng: numpy.random.Generator, shape) -> numpy.ndarray:
    """Uniform in +-sqrt(6/(d0+d1)): variance scaling with scale 1, mode fan_avg (returnn/frontend/init.py:172-197, 236-238)."""
    limit = math.sqrt(6.0 / (shape[0] + shape[1]))
    return rng.uniform(-limit, limit, shape).astype(numpy.float32)


def make_encoder_config(
    name: str = "cfg4",
    *,
    seed: int = 0,
    T: Optional[int] = None,
    B: Optional[int] = None,
    n: Optional[int] = None,
    num_layers: Optional[int] = None,
    in_dim: Optional[int] = None,
    bias_std: float = 0.0,
) -> EncoderProblem:
    """
    "cfg4": 6-layer bidirectional LSTM encoder, bf16: features [1000,32,80] ~ N(0,1), n=1024 per direction,
    layer inputs 80 then 2048, weights Glorot-uniform in the frontend layout (``ff_weight [4n,in]``,
    ``rec_weight [4n,n]``, gate order input, forget, cell-in, output), bias zero, lengths uniform in [500,1000]
    shared by all layers.  The overrides give scaled-down variants; ``bias_std`` > 0 draws a random bias instead.
    """
    assert name == "cfg4"
    T_full = 1000
    T = T_full if T is None else int(T)
    B = 32 if B is None else int(B)
    n = 1024 if n is None else int(n)
    num_layers = 6 if num_layers is None else int(num_layers)
    in_dim = 80 if in_dim is None else int(in_dim)
    rng = numpy.random.default_rng(seed)
    features = rng.standard_normal((T, B, in_dim), dtype=numpy.float32)
    lo = max(1, (500 * T) // T_full)
    lens = rng.integers(lo, T + 1, size=(B,))
    lens[0] = T
    layers = []
    for layer in range(num_layers):
        d_in = in_dim if layer == 0 else 2 * n
        entry = {}
        for direction in ("fwd", "bwd"):
            entry[direction] = {
                "ff_weight": glorot_uniform(rng, (4 * n, d_in)),
                "rec_weight": glorot_uniform(rng, (4 * n, n)),
                "bias": (rng.standard_normal((4 * n,)) * bias_std).astype(numpy.float32),
            }
        layers.append(entry)
    return EncoderProblem(name=name, features=features, lens=lens, layers=layers, n=n, dtype="bf16")

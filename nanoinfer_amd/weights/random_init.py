"""Random weights from a seed: a counter-based generator, so that every element of every tensor is
a function of (seed, tensor name, element index) alone.

The reference has no random-weights mode in its engine (tools/model.py:242-248 draws N(0, 0.02)
for training only).  Here a model folder can be written from a configuration and a seed, for tests
and measurements without a checkpoint.  Because an element depends on nothing but its own index,
tensors can be produced in any order, in pieces, on the CPU (numpy) or on the GPU (the
``ni_random_normal`` kernel) with the same bits: the large models of the measurements are
generated on the device and streamed into the file piece by piece, never held whole in host
memory.

Definition, all in IEEE float32 with every operation rounded on its own (no fused multiply-add):

* ``key`` = the first eight bytes of sha256("<seed>:<tensor name>"), little endian.
* ``z`` = splitmix64 finaliser of ``key + (index + 1) * 0x9E3779B97F4A7C15`` (mod 2^64).
* ``u1`` = ((z >> 40) + 1) / 2^24 in (0, 1];  ``u2`` = (z & 0xFFFFFF) / 2^24 in [0, 1).
* ``n`` = sqrt(-2 ln u1) * cos(2 pi u2)  (Box-Muller), with ``ln`` and ``cos`` evaluated by the
  fixed polynomials below, so that numpy and the kernel agree bit for bit;
* element = ``mean + std * n``, then rounded to the stored type (to nearest even for bfloat16).
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass
from typing import Iterator, Optional, Tuple

import numpy as np
import torch

GAMMA = 0x9E3779B97F4A7C15
MIX1 = 0xBF58476D1CE4E5B9
MIX2 = 0x94D049BB133111EB
LN2 = np.float32(0.6931471805599453)
HALF_PI = np.float32(1.5707963267948966)
SQRT_HALF = np.float32(0.7071067811865476)
# ln m = 2 (s + s^3/3 + s^5/5 + ...), s = (m - 1)/(m + 1), for m in [sqrt(1/2), sqrt(2)): |s| < 0.1716
def _ratio(a: float, b: float) -> np.float32:
    """a / b as ONE float32 division, which is what the kernel's `a.0f / b` is."""
    return np.float32(a) / np.float32(b)


LN_COEFFS = tuple(_ratio(2.0, k) for k in (1, 3, 5, 7, 9, 11))
# sin x and cos x for x in [0, pi/4], Taylor coefficients
SIN_COEFFS = (np.float32(1.0), _ratio(-1, 6), _ratio(1, 120), _ratio(-1, 5040), _ratio(1, 362880), _ratio(-1, 39916800))
COS_COEFFS = (np.float32(1.0), np.float32(-0.5), _ratio(1, 24), _ratio(-1, 720), _ratio(1, 40320), _ratio(-1, 3628800))


@dataclass(frozen=True)
class InitRule:
    """How the random weights of an architecture are drawn, as data: a tensor of one dimension (a
    norm's weight) is ``vector_mean + N(0, vector_std)``, every other one ``N(0, matrix_std)``;
    ``overrides`` holds (name suffix, mean, std) for tensors that want something else."""

    matrix_std: float = 0.02
    vector_mean: float = 1.0
    vector_std: float = 0.05
    overrides: Tuple[Tuple[str, float, float], ...] = ()

    def mean_std(self, name: str, shape: Tuple[int, ...]) -> Tuple[float, float]:
        for suffix, mean, std in self.overrides:
            if name.endswith(suffix):
                return float(mean), float(std)
        if len(shape) == 1:
            return float(self.vector_mean), float(self.vector_std)
        return 0.0, float(self.matrix_std)


def tensor_key(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little")


def _poly(x2: np.ndarray, coeffs) -> np.ndarray:
    """c0 + x2 (c1 + x2 (c2 + ...)) in float32, one rounding per operation."""
    acc = np.full_like(x2, coeffs[-1])
    for c in reversed(coeffs[:-1]):
        acc = acc * x2
        acc = acc + c
    return acc


def standard_normal(key: int, start: int, count: int) -> np.ndarray:
    """Elements ``start .. start + count - 1`` of the standard-normal stream of ``key``, float32."""
    block = 1 << 15                      # worked through in blocks that stay in the processor's cache
    if count > block:
        out = np.empty(count, dtype=np.float32)
        for at in range(0, count, block):
            n = min(block, count - at)
            out[at:at + n] = _standard_normal_block(key, start + at, n)
        return out
    return _standard_normal_block(key, start, count)


def _standard_normal_block(key: int, start: int, count: int) -> np.ndarray:
    f32 = np.float32
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        z = np.uint64(key) + idx * np.uint64(GAMMA)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(MIX1)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(MIX2)
        z = z ^ (z >> np.uint64(31))
    k1 = (z >> np.uint64(40)).astype(np.int64) + 1                  # 1 .. 2^24
    k2 = (z & np.uint64(0xFFFFFF)).astype(np.int64)                 # 0 .. 2^24 - 1
    # -2 ln u1, u1 = k1 / 2^24 = m * 2^e with m in [sqrt(1/2), sqrt(2))
    m, e = np.frexp(k1.astype(f32))                                 # m in [0.5, 1), exact
    low = m < SQRT_HALF
    m = np.where(low, m * f32(2.0), m).astype(f32)
    e = (e - low.astype(np.int32) - 24).astype(f32)
    s = (m - f32(1.0)) / (m + f32(1.0))
    ln_m = s * _poly(s * s, LN_COEFFS)
    ln_u = e * LN2 + ln_m
    radius = np.sqrt(f32(-2.0) * ln_u)
    # cos(2 pi u2), u2 = k2 / 2^24: quarter turns q and the rest f in [0, 1), folded to [0, 1/2]
    q = (k2 >> 22).astype(np.int32)
    f = (k2 & 0x3FFFFF).astype(f32) * f32(1.0 / (1 << 22))
    fold = f > f32(0.5)
    x = np.where(fold, f32(1.0) - f, f).astype(f32) * HALF_PI
    x2 = x * x
    sin_x = x * _poly(x2, SIN_COEFFS)
    cos_x = _poly(x2, COS_COEFFS)
    sin_f = np.where(fold, cos_x, sin_x)          # sin(pi/2 f) = cos(pi/2 (1 - f))
    cos_f = np.where(fold, sin_x, cos_x)
    c = np.select([q == 0, q == 1, q == 2], [cos_f, -sin_f, -cos_f], sin_f).astype(f32)
    return (radius * c).astype(f32)


def normal_cpu(key: int, start: int, count: int, mean: float, std: float, dtype: torch.dtype) -> torch.Tensor:
    n = standard_normal(key, start, count)
    t = torch.from_numpy(np.float32(std) * n + np.float32(mean))
    return t if dtype == torch.float32 else t.to(dtype)


def normal_gpu(key: int, start: int, count: int, mean: float, std: float, dtype: torch.dtype,
               device: torch.device) -> torch.Tensor:
    from .. import kernels as K
    out = torch.empty(count, dtype=dtype, device=device)
    return K.random_normal(out, key, start, mean, std)


GPU_WORTH_IT = 1 << 20        # elements from which a tensor is generated on the GPU when one is there
PIECE = 1 << 26               # elements generated, copied and written at a time


def pieces(seed: int, name: str, shape: Tuple[int, ...], mean: float, std: float, dtype: torch.dtype,
           device: Optional[torch.device] = None) -> Iterator[torch.Tensor]:
    """The tensor ``name`` as a run of flat CPU pieces of at most ``PIECE`` elements, in order.
    With a ``device`` large tensors are generated there (same values) and copied back piece by piece."""
    total = 1
    for s in shape:
        total *= int(s)
    key = tensor_key(seed, name)
    on_gpu = device is not None and total >= GPU_WORTH_IT
    for start in range(0, total, PIECE):
        count = min(PIECE, total - start)
        if on_gpu:
            yield normal_gpu(key, start, count, mean, std, dtype, device).cpu()
        else:
            yield normal_cpu(key, start, count, mean, std, dtype)


def random_tensor(seed: int, name: str, shape: Tuple[int, ...], mean: float, std: float,
                  dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """The whole tensor on the CPU (small models, tests)."""
    parts = list(pieces(seed, name, shape, mean, std, dtype))
    flat = parts[0] if len(parts) == 1 else torch.cat(parts)
    return flat.reshape(tuple(int(s) for s in shape))

"""Seeded random tensors as a function of (seed, tensor name, element index) alone.

The reference fills its synthetic benchmark weights from a seeded generator
(reference: benchmarks/SharpInference.Bench/ScoutHotPathBenchmarks.cs:54-84).  Here there is no
generator state: element i of a tensor is computed from a 64-bit key that stands for (seed, name)
and from i, with integer arithmetic and ONE float product, so that the host (this file, numpy)
and the device (csrc/random_fill.hip) give the same bits.  A model of hundreds of gigabytes is
filled straight into device memory, and the file that ``write_random_model`` writes from the same
seed on the host holds the same tensors.

    mix(z):  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9; z ^= z >> 27; z *= 0x94D049BB133111EB; z ^= z >> 31
    word(c) = mix(key + (c + 1) * 0x9E3779B97F4A7C15)                      (64-bit wrap-around)
    normal : S = sum of the twelve 16-bit fields of word(3i), word(3i+1), word(3i+2);
             value = float32(S - 393210) * float32(std / 65536)
             (twelve uniforms added: mean 0, deviation std, tails to +-6 std)
    uniform on [lo, hi): u = word(i) >> 40; m = round(lo * 2^24) + ((u * round((hi - lo) * 2^24)) >> 24);
             value = float32(m) * 2^-24
    integers: word(i) >> 49 (15 bits)
"""
from __future__ import annotations

import hashlib
from typing import Tuple

import numpy as np
import torch

FILL_NORMAL, FILL_UNIFORM, FILL_INT = 0, 1, 2
_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def name_key(seed: int, name: str) -> int:
    """The 64 bits that stand for (seed, tensor name)."""
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little")


def normal_scale(std: float) -> float:
    """std / 65536 as the float32 both sides multiply by."""
    return float(np.float32(std / 65536.0))


def uniform_fixed(lo: float, hi: float) -> Tuple[int, int]:
    return int(round(lo * (1 << 24))), int(round((hi - lo) * (1 << 24)))


def _mix(z: np.ndarray) -> np.ndarray:
    z = z ^ (z >> np.uint64(30))
    z = z * _M1
    z = z ^ (z >> np.uint64(27))
    z = z * _M2
    return z ^ (z >> np.uint64(31))


def _word(key: int, c: np.ndarray) -> np.ndarray:
    return _mix(np.uint64(key) + (c + np.uint64(1)) * _GOLDEN)


def _fields(w: np.ndarray) -> np.ndarray:
    m = np.uint64(0xFFFF)
    return ((w & m) + ((w >> np.uint64(16)) & m) + ((w >> np.uint64(32)) & m) + (w >> np.uint64(48))).astype(np.int64)


def host_fill(n: int, key: int, kind: int, std: float = 0.02, lo: float = 0.9, hi: float = 1.1,
              start: int = 0) -> np.ndarray:
    """Elements start .. start + n - 1 of the tensor with this key: float32 (or int32 for FILL_INT)."""
    out = np.empty(n, dtype=np.int32 if kind == FILL_INT else np.float32)
    with np.errstate(over="ignore"):
        for o in range(0, n, 1 << 22):                     # in pieces: the 64-bit temporaries stay small
            i = np.arange(start + o, start + min(n, o + (1 << 22)), dtype=np.uint64)
            if kind == FILL_NORMAL:
                three = np.uint64(3)
                s = _fields(_word(key, three * i)) + _fields(_word(key, three * i + np.uint64(1))) + \
                    _fields(_word(key, three * i + np.uint64(2)))
                out[o:o + len(i)] = (s - 393210).astype(np.float32) * np.float32(normal_scale(std))
            elif kind == FILL_UNIFORM:
                lo_f, span_f = uniform_fixed(lo, hi)
                u = _word(key, i) >> np.uint64(40)
                m = np.int64(lo_f) + ((u * np.uint64(span_f)) >> np.uint64(24)).astype(np.int64)
                out[o:o + len(i)] = m.astype(np.float32) * np.float32(2.0 ** -24)
            else:
                out[o:o + len(i)] = (_word(key, i) >> np.uint64(49)).astype(np.int32)
    return out


def host_tensor(shape, key: int, kind: int, dtype: torch.dtype, std: float = 0.02, lo: float = 0.9, hi: float = 1.1) -> torch.Tensor:
    n = 1
    for d in shape:
        n *= int(d)
    t = torch.from_numpy(host_fill(n, key, kind, std, lo, hi)).reshape(tuple(shape))
    return t if kind == FILL_INT else t.to(dtype)

"""Seeded synthetic inputs: a counter-based generator that is trivial to reproduce in any language.

Element i (linear index in storage order) of the stream with seed s is
``splitmix64_finalise(s XOR (0x9E3779B97F4A7C15 * (i + 1)))``; uniform variates take the top bits:
U[0,1) fp32 = top 24 bits / 2^24, U[-1,1) fp32 = top 24 bits / 2^23 - 1, U[-1,1) fp16 = top 11 bits
/ 1024 - 1 (every value exactly representable in fp16), N(0,1) by Box-Muller in fp64 on two
uniforms from the streams s and s + 0x5bd1e995, rounded to fp32.
"""
from __future__ import annotations

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def splitmix64(seed: int, n: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        i = np.arange(1, n + 1, dtype=np.uint64)
        z = np.uint64(seed) ^ (_GOLDEN * i)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform01_f32(seed: int, n: int) -> np.ndarray:
    return ((splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) / np.float32(1 << 24)).astype(np.float32)


def uniform_pm1_f32(seed: int, n: int) -> np.ndarray:
    return ((splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) / np.float32(1 << 23) - np.float32(1.0)).astype(np.float32)


def uniform_pm1_f16(seed: int, n: int) -> np.ndarray:
    return ((splitmix64(seed, n) >> np.uint64(53)).astype(np.float32) / np.float32(1024.0) - np.float32(1.0)).astype(np.float16)


def normal_f32(seed: int, n: int) -> np.ndarray:
    u1 = ((splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)     # (0, 1]
    u2 = (splitmix64(seed + 0x5bd1e995, n) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    return (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def matrix(kind: str, seed: int, shape) -> np.ndarray:
    """A column-major (Fortran-order) array of the given logical shape; element order of the stream
    is the storage order."""
    n = int(np.prod(shape))
    gen = {"u01_f32": uniform01_f32, "upm1_f32": uniform_pm1_f32, "upm1_f16": uniform_pm1_f16, "normal_f32": normal_f32}[kind]
    return gen(seed, n).reshape(tuple(shape), order="F")

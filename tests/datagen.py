"""Seeded synthetic inputs shared by the tests and the benchmark.

`pattern_bits` is the conformance suite's hash pattern
(test/backend/backend_conformance_common.hpp:119-142): raw leaf bits as a
function of the logical index and a salt, which covers NaNs, infinities,
subnormals and every exponent.  The other generators produce the value
distributions the benchmark configurations name.
"""
import numpy as np

M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.uint64)
    with np.errstate(over="ignore"):
        x = x + np.uint64(0x9E3779B97F4A7C15)
        x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return x ^ (x >> np.uint64(31))


def pattern_bits(bits: int, count: int, salt: int, start: int = 0) -> np.ndarray:
    idx = np.arange(start, start + count, dtype=np.uint64)
    with np.errstate(over="ignore"):
        raw = splitmix64(splitmix64(idx * np.uint64(0x9E3779B97F4A7C15)) ^ np.uint64(salt))
    if bits == 64:
        return raw
    kind = np.uint8 if bits <= 8 else (np.uint16 if bits == 16 else np.uint32)
    return (raw & np.uint64((1 << bits) - 1)).astype(kind)


def uniform01(count: int, salt: int) -> np.ndarray:
    """float64 uniform in [0,1) from the same hash."""
    idx = np.arange(count, dtype=np.uint64)
    with np.errstate(over="ignore"):
        raw = splitmix64(splitmix64(idx * np.uint64(0x9E3779B97F4A7C15)) ^ np.uint64(salt))
    return (raw >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def uniform_f32(count: int, lo: float, hi: float, salt: int) -> np.ndarray:
    return (lo + (hi - lo) * uniform01(count, salt)).astype(np.float32)


def uniform_i32(count: int, lo: int, hi: int, salt: int) -> np.ndarray:
    v = np.floor(lo + (hi - lo) * uniform01(count, salt)).astype(np.int64)
    return v.astype(np.int32).view(np.uint32)


def normal_f32(count: int, mean: float, std: float, salt: int) -> np.ndarray:
    """Box-Muller on the hash stream (deterministic, no global RNG state)."""
    u1 = uniform01(count, salt)
    u2 = uniform01(count, salt ^ 0x5DEECE66D)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    return (mean + std * r * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def bf16_rne(x: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (bits & np.uint64(0x7FFFFFFF)) > np.uint64(0x7F800000)
    r = ((bits + np.uint64(0x7FFF) + ((bits >> np.uint64(16)) & np.uint64(1))) >> np.uint64(16)).astype(np.uint16)
    r[nan] = 0x7FC0
    return r


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)

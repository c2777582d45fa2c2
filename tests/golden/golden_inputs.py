"""Deterministic inputs shared by make_golden.py and the tests that read its fixtures.

Values come from an integer hash of the element index (splitmix64 finaliser), mapped to the grid
k/64, k in [-128, 127]: exactly representable in fp16 and bf16, roughly unit variance, and
independent of any library's random generator, so the fixtures only need to hold outputs."""
import numpy as np


def golden_tensor(shape, stream):
    n = int(np.prod(shape))
    with np.errstate(over="ignore"):
        z = np.arange(n, dtype=np.uint64) + np.uint64(stream) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    k = (z >> np.uint64(56)).astype(np.int64) - 128
    return (k.astype(np.float32) / 64.0).reshape(shape)


def qkv(B, Sq, Skv, Hq, Hkv, D, DV, stream):
    return (golden_tensor((B, Sq, Hq, D), stream), golden_tensor((B, Skv, Hkv, D), stream + 1),
            golden_tensor((B, Skv, Hkv, DV), stream + 2))

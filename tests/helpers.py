"""Shared helpers of the parity tests."""
from __future__ import annotations

import ctypes
import json
import os

import numpy as np

FP_PQ = 25651
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_gqa_fixture():
    with open(os.path.join(GOLDEN, "gqa_spec_decode_69.json")) as f:
        return json.load(f)


def splitmix64(x: np.ndarray) -> np.ndarray:
    x = (x + np.uint64(0x9E3779B97F4A7C15)).astype(np.uint64)
    x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def uniform_fp(shape, seed: int) -> np.ndarray:
    """The generator of mi355_fp_fill_uniform: splitmix64(seed + i) % 25651."""
    n = int(np.prod(shape))
    with np.errstate(over="ignore"):
        v = splitmix64(np.arange(n, dtype=np.uint64) + np.uint64(seed))
    return (v % np.uint64(FP_PQ)).astype(np.uint16).reshape(shape)


def normal_f16(shape, std: float, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(size=shape, dtype=np.float32) * std).astype(np.float16)


class DeviceBuffer:
    """A raw slice of device memory for tests that call the C ABI directly."""

    def __init__(self, abi, arena_base: int, offset: int, nbytes: int):
        self.abi, self.ptr, self.nbytes = abi, arena_base + offset, nbytes

    def write(self, a: np.ndarray):
        a = np.ascontiguousarray(a)
        assert a.nbytes == self.nbytes
        rc = self.abi.mi355_memcpy_h2d(ctypes.c_void_p(self.ptr), a.ctypes.data_as(ctypes.c_void_p), a.nbytes)
        assert rc == 0

    def read(self, dtype, shape) -> np.ndarray:
        a = np.empty(shape, dtype)
        assert a.nbytes == self.nbytes
        rc = self.abi.mi355_memcpy_d2h(a.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(self.ptr), a.nbytes)
        assert rc == 0
        return a


def ulp16(x: np.ndarray) -> np.ndarray:
    """Spacing of fp16 numbers at magnitude |x| (normal range)."""
    a = np.maximum(np.abs(np.asarray(x, np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 10)


def assert_f16_close(got: np.ndarray, want: np.ndarray, rtol=1e-2, atol=1e-3, what="", peak=None,
                     strict_outliers=None):
    """The fp16 parity bar: |got - want| <= atol + rtol * |want| element-wise.

    `peak` (same shape, optional): the largest magnitude the element's fp16 for-loop
    accumulator passes through on the way to its final value.  Two evaluations that differ
    only in the order of the fp32 additions inside a tile product can round one iteration's
    tile, and then the accumulator, differently by one fp16 ulp OF THE ACCUMULATOR; where
    the partial sums cancel (|final| << peak) that ulp is larger than the bar above allows.
    With `peak` the bound becomes atol + rtol * |want| + 2 ulp16(peak), and
    `strict_outliers` caps the fraction of elements outside the plain bar.  Returns that
    count."""
    g = got.astype(np.float64)
    w = want.astype(np.float64)
    assert g.shape == w.shape, (g.shape, w.shape)
    finite = np.isfinite(w)
    assert np.array_equal(np.isfinite(g), finite), f"{what}: non-finite pattern differs"
    err = np.abs(g - w)[finite]
    tol = (atol + rtol * np.abs(w))[finite]
    strict_bad = int((err > tol).sum())
    if peak is not None:
        tol = tol + 2.0 * ulp16(np.asarray(peak, np.float64))[finite]
        if strict_outliers is not None:
            assert strict_bad <= strict_outliers * err.size, (
                f"{what}: {strict_bad} of {err.size} outside the plain tolerance")
    bad = err > tol
    assert not bad.any(), (
        f"{what}: {int(bad.sum())} of {bad.size} outside tolerance; worst abs err "
        f"{err.max():.3e}, worst ratio {(err / tol).max():.2f}")
    return strict_bad

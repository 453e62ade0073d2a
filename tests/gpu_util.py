"""Helpers shared by the GPU parity tests."""
import numpy as np

from deepj_amd import HipBackend, Tensor
from oracle import cpu_ref as ref


def tensor(a) -> Tensor:
    return Tensor.from2D(np.asarray(a, dtype=np.float32))


def rnd(rows, cols, seed) -> np.ndarray:
    """cpu.random(rows, cols, new Random(seed)) of the reference's GPU tests."""
    return ref.random_tensor(rows, cols, seed)


def assert_close(expected, actual, atol=1e-4, rtol=1e-4, what=""):
    """|e - a| <= atol + rtol*|e| (MetalBackendTest.java:452-466 in the reference)."""
    if isinstance(actual, Tensor):
        actual = actual.numpy()
    e = np.asarray(expected, dtype=np.float64)
    a = np.asarray(actual, dtype=np.float64)
    assert e.shape == a.shape, (what, e.shape, a.shape)
    bad = ~(np.abs(e - a) <= atol + rtol * np.abs(e))
    if bad.any():
        i = np.argwhere(bad)[0]
        raise AssertionError(f"{what}: mismatch at {tuple(i)} expected={e[tuple(i)]} actual={a[tuple(i)]} "
                             f"({bad.sum()} of {bad.size} elements)")


class backend:
    """with backend() as be: fresh HipBackend installed, released on exit."""

    def __enter__(self):
        self.be = HipBackend()
        Tensor.setBackend(self.be)
        return self.be

    def __exit__(self, *exc):
        self.be.releaseResources()
        return False

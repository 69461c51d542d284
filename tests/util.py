"""Shared helpers of the GPU parity tests."""
import numpy as np

from tessera_amd import KernelLaunch


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / max(|ref|, eps) with eps = 0.05 * rms(ref).

    The floor is there because the reference result is itself an fp32 sequential sum: its own
    rounding noise is about sqrt(k) * 2^-24 * rms(ref) (1e-5 * rms at k = 17408), so an output
    that cancels to less than a few percent of the rms cannot be reproduced to 1e-3 of its own
    size by any other summation order.  Such outputs are held to 1e-3 * 0.05 * rms instead."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    eps = 0.05 * np.sqrt(np.mean(ref * ref)) + 1e-30
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), eps)))


def strict_rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """The same figure with the floor the measurement plan names, eps = 1e-3 * rms(ref): reported next
    to rel_err by the full-size tests.  Near that floor it measures the reference's own summation
    noise as much as the device's (see rel_err), so it is printed, and asserted only loosely."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    eps = 1e-3 * np.sqrt(np.mean(ref * ref)) + 1e-30
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), eps)))


def rms_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / rms(ref): the absolute error in units of a typical output."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    return float(np.max(np.abs(got - ref)) / (np.sqrt(np.mean(ref * ref)) + 1e-30))


def norm_err(got: np.ndarray, ref: np.ndarray) -> float:
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    return float(np.linalg.norm(got - ref) / (np.linalg.norm(ref) + 1e-30))


def same_bits(a: np.ndarray, b: np.ndarray) -> bool:
    return np.array_equal(np.ascontiguousarray(a, np.float32).view(np.uint32),
                          np.ascontiguousarray(b, np.float32).view(np.uint32))


def same_bits_zero_sign_free(a: np.ndarray, b: np.ndarray) -> bool:
    """Bit equality except that -0 and +0 compare equal (a dot product starts from +0)."""
    return same_bits(np.asarray(a, np.float32) + np.float32(0), np.asarray(b, np.float32) + np.float32(0))


def run(backend, name, buffers, scalars, grid=(1, 1, 1), block=(256, 1, 1)):
    k = backend.LoadKernel(name)
    backend.LaunchKernel(k, KernelLaunch(grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                         list(buffers), list(scalars)))


def ref_grid_vec(m, n):
    """The reference's launch shape for the warp-per-output family
    (src/core/decode_internal.hpp:896-901): ceil(m*n/8) workgroups of 256."""
    return ((m * n + 7) // 8, 1, 1)

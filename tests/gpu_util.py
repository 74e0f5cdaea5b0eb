"""Shared helpers of the GPU parity tests: seeded inputs in the reference's
formats, parameter blocks, and the tolerance the path's contract states."""
import struct

import numpy as np

REL_L2_TOL = 1e-3        # relative L2 error of fp16 outputs vs the CPU oracle
MAX_ABS_RMS_TOL = 2e-2   # max-abs error <= 2e-2 x output RMS


def w4_case(rng, m, n, k, bias=False):
    """int4 ~ U{-8..7} packed 2/byte (low nibble = even K), scales ~ U[0.005,0.02] f16,
    activations ~ N(0,1) f16."""
    packed = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    scale = rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float16) if bias else None
    return x, packed, scale, b


def assert_close_to_oracle(actual_f16, expected_f32, what="", rel_l2_tol=REL_L2_TOL):
    actual = np.asarray(actual_f16, dtype=np.float32).reshape(-1)
    expected = np.asarray(expected_f32, dtype=np.float32).reshape(-1)
    assert actual.shape == expected.shape, (what, actual.shape, expected.shape)
    assert np.all(np.isfinite(actual)), f"{what}: non-finite output"
    difference = actual.astype(np.float64) - expected.astype(np.float64)
    norm = float(np.sqrt(np.sum(expected.astype(np.float64) ** 2)))
    rel_l2 = float(np.sqrt(np.sum(difference ** 2))) / max(norm, 1e-30)
    rms = norm / np.sqrt(max(1, expected.size))
    max_abs = float(np.max(np.abs(difference))) if difference.size else 0.0
    assert rel_l2 <= rel_l2_tol, f"{what}: rel-L2 {rel_l2:.3e} > {rel_l2_tol}"
    assert max_abs <= MAX_ABS_RMS_TOL * rms + 1e-6, \
        f"{what}: max-abs {max_abs:.3e} > {MAX_ABS_RMS_TOL} x RMS {rms:.3e}"
    return rel_l2, max_abs


def u32s(*values):
    """Metal_parameters.u32s (lib/metal_parameters.ml:14-22)."""
    return struct.pack("<%dI" % len(values), *values)


def linear_grid(columns):
    """linear_f16_grid (lib/metal_dispatch_common.ml:64-70): thread count the reference passes."""
    return ((columns + 7) // 8) * 8 * 32

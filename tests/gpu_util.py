"""Helpers shared by the GPU parity tests."""
import math

import numpy as np


def int4_tolerances(y, ref, k, x):
    """Parity bar for the float int4 paths: max-abs-err <= 1e-3*sqrt(K)*max|x| and relative error
    <= 1e-2, relative error being max|delta| / max|ref| as the reference's own kernel_bench
    computes it (apps/llm-bench/src/bin/kernel_bench.rs:99-106).  Returns (abs_err, rel_err)."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    assert y.shape == ref.shape
    d = float(np.abs(y - ref).max()) if y.size else 0.0
    rel = d / max(float(np.abs(ref).max()), 1e-6) if y.size else 0.0
    abs_tol = 1e-3 * math.sqrt(k) * float(np.abs(np.asarray(x, np.float64)).max())
    assert d <= abs_tol, f"max abs err {d} > {abs_tol}"
    assert rel <= 1e-2, f"relative err {rel} > 1e-2"
    return d, rel


def pack_zero_points(zq):
    """[n][groups] uint4 values -> MatMulNBits packing, group 2j in the low nibble."""
    n, groups = zq.shape
    out = np.zeros((n, (groups + 1) // 2), np.uint8)
    for j in range(groups):
        out[:, j // 2] |= (zq[:, j].astype(np.uint8) << (4 * (j & 1))).astype(np.uint8)
    return out


def bf16_round(x):
    """f32 -> bf16 (round to nearest even) -> f32, in numpy."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32)

"""Pins the int8 GEMM part of the CPU checker against the reference's unit-test vectors
(crates/yscv-kernels/src/ops/int8_matmul.rs:2437-2666, crates/yscv-onnx/src/tests/qlinear.rs,
tests/coverage.rs) and against numpy int64 matmul.  No GPU."""
import numpy as np
import pytest

REF_DISPATCH_SHAPES = [(1, 1, 1), (2, 3, 4), (4, 16, 8), (5, 17, 6), (8, 64, 8)]  # int8_matmul.rs:2468-2477
REF_PREPACKED_SHAPES = [(1, 1, 1), (1, 17, 5), (3, 31, 7), (4, 64, 16), (8, 127, 33), (16, 128, 64)]  # :2480-2500
BLOCKED_SHAPES = [(4, 64, 16), (8, 67, 32), (12, 130, 48), (4, 4, 16), (16, 256, 64)]  # MR4xNR16 gate with K tails


def np_ref(a, b, m, k, n):
    return (a.reshape(m, k).astype(np.int64) @ b.reshape(k, n).astype(np.int64)).astype(np.int32)


def test_scalar_goldens(oracle):
    # int8_matmul.rs:2459-2465
    assert oracle.int8_matmul_scalar([1, 2, 3, 4], [5, 6, 7, 8], 2, 2, 2).ravel().tolist() == [19, 22, 43, 50]
    # :2449-2456
    assert (oracle.int8_matmul_scalar(np.zeros(12), np.zeros(12), 3, 4, 3) == 0).all()
    # :2503-2509
    a = np.full(128, -128, np.int8)
    assert oracle.int8_matmul_scalar(a, a, 1, 128, 1).tolist() == [[128 * 128 * 128]]


@pytest.mark.parametrize("m,k,n", REF_DISPATCH_SHAPES + REF_PREPACKED_SHAPES + BLOCKED_SHAPES)
def test_scalar_prepacked_simd_agree_with_int64(oracle, m, k, n):
    a = oracle.lcg_i8(0xDEAD ^ (m * k), m * k)
    b = oracle.lcg_i8(0xBEEF ^ (k * n), k * n)
    exp = np_ref(a, b, m, k, n)
    assert np.array_equal(oracle.int8_matmul_scalar(a, b, m, k, n), exp)
    bt = oracle.transpose_b(b, k, n)
    assert np.array_equal(bt.reshape(n, k), b.reshape(k, n).T)
    assert np.array_equal(oracle.int8_matmul_prepacked_scalar(a, bt, m, k, n), exp)
    assert np.array_equal(oracle.simd_int8_matmul_dispatch(a, b, m, k, n), exp)
    pk = oracle.SimdPackedI8B(b, k, n)
    assert np.array_equal(pk.matmul(a, m), exp)
    assert np.array_equal(pk.matmul(a, m, threads=3), exp)


def test_lcg_matches_reference_formula(oracle):
    # kernel_bench.rs:28-50
    s, exp_i8, exp_f = 0xAA, [], []
    for _ in range(6):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        exp_i8.append((s >> 33) % 256 - 128)
        exp_f.append(np.float32((s >> 33) % 2001 - 1000) * np.float32(0.001))
    assert oracle.lcg_i8(0xAA, 6).tolist() == exp_i8
    assert oracle.lcg_f32(0xAA, 6).tolist() == [float(v) for v in exp_f]


def test_zero_point_algebra(oracle):
    # sum (a - z) b == sum a b - z * colsum(b)   (conv/quantized.rs:119-147)
    rng = np.random.default_rng(2)
    m, k, n = 7, 96, 10
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    for zp in (128, 0, 3, 255):
        got = oracle.u8i8_matmul_zp(a, zp, b, m, k, n)
        exp = ((a.astype(np.int64) - zp) @ b.astype(np.int64)).astype(np.int32)
        assert np.array_equal(got, exp)
        raw = (a.astype(np.int64) @ b.astype(np.int64))
        cs = oracle.i8_col_sums(b, k, n).astype(np.int64)
        assert np.array_equal((raw - zp * cs).astype(np.int32), got)
    # a_zp = 128 is exactly the signed kernel on (a ^ 0x80) as i8  (int8_matmul.rs:1866-1868)
    a_s = (a ^ 0x80).view(np.int8)
    assert np.array_equal(oracle.u8i8_matmul_zp(a, 128, b, m, k, n), oracle.int8_matmul_scalar(a_s, b, m, k, n))


def test_matmul_integer_reference_examples(oracle):
    # qlinear.rs:667-705 symmetric fast path
    a = np.arange(24) - 12
    b = (np.arange(24) * 5) % 23 - 11
    out, fast = oracle.exec_matmul_integer(a, b, 0.0, 0.0, 3, 8, 3)
    assert fast and np.array_equal(out, (a.reshape(3, 8) @ b.reshape(8, 3)).astype(np.float32))
    # coverage.rs:359-390 asymmetric: a_zp = 10, B = I -> [0,1,2,3]
    out, fast = oracle.exec_matmul_integer([10, 11, 12, 13], [1, 0, 0, 1], 10.0, 0.0, 2, 2, 2)
    assert not fast and out.ravel().tolist() == [0.0, 1.0, 2.0, 3.0]
    # gemm_matmul.rs:73-87
    out, _ = oracle.exec_matmul_integer([1, 2, 3, 4], [5, 6, 7, 8], 0.0, 0.0, 2, 2, 2)
    assert out[0, 0] == 19.0


def test_qlinear_matmul_reference_examples(oracle):
    # qlinear.rs:150-194: composite (0.05*0.1)/0.25, round half away, clamp
    a = np.arange(32) - 16
    b = (np.arange(32) * 7) % 31 - 15
    out, fast = oracle.exec_qlinear_matmul(a, 0.05, 0.0, b, 0.1, 0.0, 0.25, 0.0, 4, 8, 4)
    assert fast
    comp = np.float32(np.float32(0.05) * np.float32(0.1)) / np.float32(0.25)
    acc = (a.reshape(4, 8) @ b.reshape(8, 4)).astype(np.float32)
    v = acc * comp
    exp = np.clip(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)), -128, 127)
    assert np.array_equal(out, exp.astype(np.float32))
    # coverage.rs:303-357: unit scales -> plain matmul rounded half away and clamped
    a2 = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    b2 = [0.5, -0.5, 1.0, -1.0, 0.0, 2.0]
    out, fast = oracle.exec_qlinear_matmul(a2, 1.0, 0.0, b2, 1.0, 0.0, 1.0, 0.0, 2, 3, 2)
    # fast path casts b to i8 by truncation: 0.5 -> 0, -0.5 -> 0
    bi = np.trunc(np.array(b2)).reshape(3, 2)
    assert fast and np.array_equal(out, (np.array(a2).reshape(2, 3) @ bi).astype(np.float32))
    # asymmetric input takes the f32 fallback (linear.rs:494-537)
    out, fast = oracle.exec_qlinear_matmul([3, 4, 5, 6], 0.5, 3.0, [1, 0, 0, 1], 1.0, 0.0, 0.5, 0.0, 2, 2, 2)
    assert not fast and out.ravel().tolist() == [0.0, 1.0, 2.0, 3.0]


def test_prepack_gates(oracle):
    # runner/layout.rs:6-11, plan/build.rs:1371-1377
    assert oracle.should_use_prepacked_i8_b(512, 4096, 4096)
    assert oracle.should_use_prepacked_i8_b(1, 512, 1024)
    assert not oracle.should_use_prepacked_i8_b(1, 4, 32)
    assert not oracle.should_use_prepacked_i8_b(4, 4, 33)
    assert oracle.should_prepack_i8_b(4, 16) and not oracle.should_prepack_i8_b(3, 16)
    assert oracle.should_prepack_i8_b(512, 1025) and not oracle.should_prepack_i8_b(511, 1025)

"""Pins the int4 part of the CPU checker against the reference's own unit-test
vectors (crates/yscv-kernels/src/ops/int4_matmul.rs:648-945, ops/quantize.rs:669-833)
and against closed forms / brute force.  No GPU."""
import numpy as np
import pytest


def test_nibble_goldens(oracle):
    o = oracle.orc()
    # int4_matmul.rs:665-676
    assert (o.orc_unpack_low(0x78), o.orc_unpack_high(0x78)) == (-8, 7)
    assert (o.orc_unpack_low(0x00), o.orc_unpack_high(0x00)) == (0, 0)
    assert (o.orc_unpack_low(0xFF), o.orc_unpack_high(0xFF)) == (-1, -1)


def test_nibble_brute_force_closed_form(oracle):
    o = oracle.orc()
    for b in range(256):
        lo, hi = b & 15, b >> 4
        assert o.orc_unpack_low(b) == ((lo ^ 8) - 8)
        assert o.orc_unpack_high(b) == ((hi ^ 8) - 8)
        # quantize.rs:201-213 spells the same decode differently
        assert o.orc_nibble_lo(b) == o.orc_unpack_low(b)
        assert o.orc_nibble_hi(b) == o.orc_unpack_high(b)


def test_gemv_hand_kat(oracle):
    # nibbles (1,2),(-8,-1); groups of 2; 0.5*(1*1+2*2) + 0.25*(-8*3 + -1*4) = 2.5 - 7.0
    y = oracle.packed_int4_gemv_scalar([0x21, 0xF8], [0.5, 0.25], [1, 2, 3, 4], 1, 4, 2)
    assert y.tolist() == [-4.5]


def test_pack_then_gemv_close_to_fp32_dot(oracle):
    # int4_matmul.rs:679-717
    m_w, k, g = 2, 32, 16
    w = oracle.lcg_f32(0xDEADBEEF, m_w * k)
    packed, scales = oracle.pack_int4_symmetric_per_group(w, m_w, k, g)
    got = oracle.packed_int4_gemv_scalar(packed, scales, np.ones(k, np.float32), m_w, k, g)
    exp = w.reshape(m_w, k).astype(np.float64).sum(1)
    rel = np.abs(got - exp) / np.maximum(np.abs(exp), 1e-6)
    assert (rel < 0.12).all()


def test_zero_weights(oracle):
    # int4_matmul.rs:761-773; scale is 1.0 when abs-max <= EPSILON (:629-633)
    packed, scales = oracle.pack_int4_symmetric_per_group(np.zeros(96, np.float32), 3, 32, 16)
    assert (scales == 1.0).all() and (packed == 0).all()
    y = oracle.packed_int4_gemv_scalar(packed, scales, np.full(32, 1.5, np.float32), 3, 32, 16)
    assert (y == 0).all()


def test_gemm_m1_is_gemv_bitwise(oracle):
    # int4_matmul.rs:776-813 asks <=1e-5; the two scalar loops use the same order, so it is exact.
    n, k, g = 4, 64, 32
    packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(0xAA, n * k), n, k, g)
    x = oracle.lcg_f32(0xBB, k)
    gv = oracle.packed_int4_gemv_scalar(packed, scales, x, n, k, g)
    gm = oracle.packed_int4_gemm_scalar(packed, scales, x, 1, n, k, g)
    assert np.array_equal(gv, gm[0])


def test_gemm_rows_are_gemvs(oracle):
    n, k, g, m = 8, 64, 32, 5
    packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(0x100, n * k), n, k, g)
    x = oracle.lcg_f32(0x205, m * k).reshape(m, k)
    gm = oracle.packed_int4_gemm_scalar(packed, scales, x, m, n, k, g)
    for i in range(m):
        assert np.array_equal(gm[i], oracle.packed_int4_gemv_scalar(packed, scales, x[i], n, k, g))


def test_all_ones_activation_closed_form(oracle):
    # with x = 1 every group sum is a small integer, exact in f32: y = sum_g s_g * sum(q)
    rng = np.random.default_rng(7)
    n, k, g = 6, 128, 32
    packed = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.choice(np.array([0.5, 0.25, 2.0, 0.125], np.float32), n * (k // g))
    y = oracle.packed_int4_gemv_scalar(packed, scales, np.ones(k, np.float32), n, k, g)
    lo = ((packed & 15).astype(np.int32) ^ 8) - 8
    hi = ((packed >> 4).astype(np.int32) ^ 8) - 8
    qsum = (lo + hi).reshape(n, k // g, g // 2).sum(2)
    exp = (scales.reshape(n, -1).astype(np.float64) * qsum).sum(1)  # power-of-two scales: exact
    assert np.array_equal(y.astype(np.float64), exp)


def test_gemv_against_f64_dequant_matmul(oracle):
    rng = np.random.default_rng(11)
    n, k, g = 16, 512, 32
    packed = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    y = oracle.packed_int4_gemv_scalar(packed, scales, x, n, k, g)
    q = np.empty((n, k), np.float64)
    pb = packed.reshape(n, k // 2)
    q[:, 0::2] = ((pb & 15).astype(np.int32) ^ 8) - 8
    q[:, 1::2] = ((pb >> 4).astype(np.int32) ^ 8) - 8
    wd = q * np.repeat(scales.reshape(n, -1).astype(np.float64), g, axis=1)
    exp = wd @ x.astype(np.float64)
    bound = k * 2.0 ** -23 * (np.abs(wd) @ np.abs(x.astype(np.float64)))
    assert (np.abs(y - exp) <= bound).all()
    # a transposed/shifted operand would be off by O(1), far above the bound
    assert np.abs(y - np.roll(exp, 1)).max() > 100 * bound.max()


def test_pack_error_bound_and_layout(oracle):
    rng = np.random.default_rng(3)
    m_w, k, g = 4, 64, 16
    w = rng.standard_normal(m_w * k).astype(np.float32)
    packed, scales = oracle.pack_int4_symmetric_per_group(w, m_w, k, g)
    assert packed.size == m_w * k // 2 and scales.size == m_w * k // g
    absmax = np.abs(w.reshape(m_w, k // g, g)).max(2)
    assert np.array_equal(scales.reshape(m_w, -1), (absmax / np.float32(7.0)).astype(np.float32))
    lo = ((packed & 15).astype(np.int32) ^ 8) - 8
    hi = ((packed >> 4).astype(np.int32) ^ 8) - 8
    q = np.stack([lo, hi], 1).reshape(m_w, k)  # low nibble = even element
    err = np.abs(w.reshape(m_w, k) - q * np.repeat(scales.reshape(m_w, -1), g, axis=1))
    assert (err <= np.repeat(scales.reshape(m_w, -1), g, axis=1) * 0.5 + 1e-6).all()
    assert q.min() >= -7 and q.max() <= 7  # abs-max maps to +-7


def test_dequant_goldens(oracle):
    # quantize.rs:681-698
    out = oracle.dequantize_int4_to_f32([0xE3], 0.5, 0)
    assert np.allclose(out, [1.5, -1.0], atol=1e-6)
    out = oracle.dequantize_int4_to_f32([0x05], 0.1, 2)
    assert np.allclose(out, [0.3, -0.2], atol=1e-6)


def test_quantize_int4_round_and_clamp_golden(oracle):
    # quantize.rs:760-772 -> [7,-8,0,4]; odd length (:775-787)
    packed = oracle.quantize_f32_to_int4([100.0, -100.0, 0.0, 3.5], 1.0, 0)
    assert oracle.dequantize_int4_to_f32(packed, 1.0, 0).tolist() == [7.0, -8.0, 0.0, 4.0]
    packed = oracle.quantize_f32_to_int4([1.0, 2.0, 3.0], 1.0, 0)
    assert oracle.dequantize_int4_to_f32(packed, 1.0, 0).tolist() == [1.0, 2.0, 3.0, 0.0]
    # ties to even: 0.5 -> 0, 1.5 -> 2, 2.5 -> 2
    packed = oracle.quantize_f32_to_int4([0.5, 1.5, 2.5, -2.5], 1.0, 0)
    assert oracle.dequantize_int4_to_f32(packed, 1.0, 0).tolist() == [0.0, 2.0, 2.0, -2.0]


def test_quant_dequant_property(oracle):
    # crates/yscv-kernels/src/proptest_tests.rs:147-174: error <= scale/2 inside the range
    rng = np.random.default_rng(5)
    scale = 0.37
    x = rng.uniform(-8 * scale, 7 * scale, 101).astype(np.float32)
    rec = oracle.dequantize_int4_to_f32(oracle.quantize_f32_to_int4(x, scale, 0), scale, 0)[: x.size]
    assert (np.abs(rec - x) <= scale / 2 + 1e-6).all()


def test_simd_gemv_matches_scalar(oracle):
    # int4_matmul.rs:720-758 (<=1e-4) and :857-900
    for (m_w, k, g, sw, sx) in [(4, 128, 32, 0xCAFEBABE, 0xF00DBA12), (8, 256, 32, 0x12345678, 0x9ABCDEF0),
                                (8, 256, 16, 0x12345678, 0x9ABCDEF0), (3, 96, 6, 1, 2)]:
        packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(sw, m_w * k), m_w, k, g)
        x = oracle.lcg_f32(sx, k)
        s = oracle.packed_int4_gemv_scalar(packed, scales, x, m_w, k, g)
        d = oracle.simd_packed_int4_gemv_dispatch(packed, scales, x, m_w, k, g)
        assert np.abs(s - d).max() <= 1e-4
        d2 = oracle.simd_packed_int4_gemv_dispatch(packed, scales, x, m_w, k, g, threads=3)
        assert np.array_equal(d, d2)


def test_simd_gemm_matches_scalar(oracle):
    # int4_matmul.rs:816-855 (<=1e-3)
    n, k, g = 8, 64, 32
    packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(0x100, n * k), n, k, g)
    for m in (1, 4, 16, 32):
        x = oracle.lcg_f32(0x200 + m, m * k)
        s = oracle.packed_int4_gemm_scalar(packed, scales, x, m, n, k, g)
        d = oracle.simd_packed_int4_gemm_dispatch(packed, scales, x, m, n, k, g)
        assert np.abs(s - d).max() <= 1e-3
        d2 = oracle.simd_packed_int4_gemm_dispatch(packed, scales, x, m, n, k, g, threads=4)
        assert np.array_equal(d, d2)


def test_matmul_nbits_bridge(oracle):
    rng = np.random.default_rng(21)
    m, n, k, g = 3, 5, 64, 16
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    groups = k // g
    zq = rng.integers(6, 11, (n, groups))
    zp_bytes = np.zeros((n, (groups + 1) // 2), np.uint8)
    for j in range(groups):
        zp_bytes[:, j // 2] |= (zq[:, j] << (4 * (j & 1))).astype(np.uint8)
    y = oracle.matmul_nbits(b, scales, zp_bytes, x, m, n, k, g)
    # brute force in f64 from the ONNX definition (q - zp) * scale
    q = np.empty((n, k), np.float64)
    pb = b.reshape(n, k // 2)
    q[:, 0::2] = pb & 15
    q[:, 1::2] = pb >> 4
    wd = (q - np.repeat(zq, g, axis=1)) * np.repeat(scales.reshape(n, groups).astype(np.float64), g, axis=1)
    exp = x.astype(np.float64) @ wd.T
    assert np.abs(y - exp).max() <= 1e-5
    # zp omitted == 8 == the reference's symmetric format after byte ^ 0x88
    y8 = oracle.matmul_nbits(b, scales, None, x, m, n, k, g)
    ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales, x, m, n, k, g)
    assert np.abs(y8 - ref).max() <= 1e-5 * np.abs(ref).max() + 1e-6


def test_fp16_bf16_bit_goldens(oracle):
    # crates/yscv-tensor/src/tests/fp16.rs:43-59
    assert oracle.fp16_bits_to_f32([0x3C00, 0x4000, 0x3800]).tolist() == [1.0, 2.0, 0.5]
    assert oracle.bf16_bits_to_f32([0x3F80, 0x4000, 0x3F00]).tolist() == [1.0, 2.0, 0.5]
    # widening agrees with IEEE (numpy) for every normal fp16 pattern, both signs
    bits = np.arange(0x0400, 0x7C00, dtype=np.uint16)
    assert np.array_equal(oracle.fp16_bits_to_f32(bits), bits.view(np.float16).astype(np.float32))
    assert np.array_equal(oracle.fp16_bits_to_f32(bits | 0x8000), (bits | 0x8000).view(np.float16).astype(np.float32))
    # reference quirk, restated faithfully: the subnormal branch (tensor.rs:743-753) uses
    # exponent 127-15-e and so yields HALF the IEEE value for fp16 subnormals (|v| < 6.1e-5).
    sub = np.arange(1, 0x0400, dtype=np.uint16)
    assert np.array_equal(oracle.fp16_bits_to_f32(sub) * 2, sub.view(np.float16).astype(np.float32))
    # f32 -> fp16 truncates (tensor.rs:733), so 1 + 2^-11 + 2^-12 stays 1.0 where RNE would round up
    v = np.float32(1.0 + 2.0 ** -11 + 2.0 ** -12)
    assert oracle.f32_to_fp16_bits_trunc([v]).tolist() == [0x3C00]
    assert np.float16(v).view(np.uint16) == 0x3C01
    # f32 -> bf16 is RNE (tensor.rs:764-769): 1 + 2^-8 is a tie -> even (1.0); 1 + 3*2^-8 -> 1 + 2^-6
    assert oracle.f32_to_bf16_bits([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8]).tolist() == [0x3F80, 0x3F82]


def test_matmul_nbits_bridge_hand_vectors_and_default_zero_point(oracle):
    """The MatMulNBits definition the checker composes from dequantize_int4_to_f32 (quantize.rs:215-222) and an f32 dot:
    unsigned nibbles, value (q - zp) * scale, zero point 8 when none is given, group 2j in the low nibble of a
    zero-point byte."""
    # bytes [0xA9, 0x70]: nibbles 9, 10 | 0, 7; K = 4, block 2, scales 0.5 / 0.25, x = 1 2 3 4
    b = np.array([0xA9, 0x70], np.uint8)
    s = np.array([0.5, 0.25], np.float32)
    x = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    assert oracle.matmul_nbits(b, s, None, x, 1, 1, 4, 2).tolist() == [[-4.5]]        # zp 8: (1*1 + 2*2)/2 + (-8*3 - 1*4)/4
    zps = np.array([0x79], np.uint8)                                                   # block 0: zp 9, block 1: zp 7
    assert oracle.matmul_nbits(b, s, zps, x, 1, 1, 4, 2).tolist() == [[-4.25]]         # (0*1 + 1*2)/2 + (-7*3 + 0*4)/4
    # zero point 8 everywhere = the reference kernel on byte ^ 0x88, up to the order of the scale multiplication
    rng = np.random.default_rng(11)
    m, n, k, g = 3, 10, 128, 32
    bb = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    xx = rng.standard_normal((m, k)).astype(np.float32)
    ref = oracle.packed_int4_gemm_scalar(bb ^ 0x88, sc, xx, m, n, k, g).reshape(m, n)
    got = oracle.matmul_nbits(bb, sc, None, xx, m, n, k, g)
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    explicit = np.full((n, (k // g + 1) // 2), 0x88, np.uint8)
    assert np.array_equal(oracle.matmul_nbits(bb, sc, explicit, xx, m, n, k, g), got)
    # float64 definition with random zero points
    zq = rng.integers(0, 16, (n, k // g))
    zp = np.zeros((n, (k // g + 1) // 2), np.uint8)
    for j in range(k // g):
        zp[:, j // 2] |= (zq[:, j] << (4 * (j & 1))).astype(np.uint8)
    q = np.empty((n, k))
    pb = bb.reshape(n, k // 2)
    q[:, 0::2], q[:, 1::2] = pb & 15, pb >> 4
    w = (q - np.repeat(zq, g, axis=1)) * np.repeat(sc.reshape(n, k // g).astype(np.float64), g, axis=1)
    want = xx.astype(np.float64) @ w.T
    got = oracle.matmul_nbits(bb, sc, zp, xx, m, n, k, g)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()

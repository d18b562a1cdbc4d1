"""GPU parity (bit-exact) of the int8 MFMA GEMM and its fused epilogues against the CPU restatement
of the reference, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REF_DISPATCH_SHAPES = [(1, 1, 1), (2, 3, 4), (4, 16, 8), (5, 17, 6), (8, 64, 8)]  # int8_matmul.rs:2468-2477
REF_PREPACKED_SHAPES = [(1, 1, 1), (1, 17, 5), (3, 31, 7), (4, 64, 16), (8, 127, 33), (16, 128, 64)]  # :2480-2500
EXTRA_SHAPES = [(65, 256, 129), (64, 512, 128), (130, 300, 260), (4, 4, 16), (12, 130, 48)]


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available()
    return torch


@pytest.fixture(scope="module")
def K():
    from yscv_amd import kernels

    return kernels


def test_goldens(oracle, K):
    out = np.zeros(4, np.int32)
    K.int8_matmul_dispatch([1, 2, 3, 4], [5, 6, 7, 8], 2, 2, 2, out)  # int8_matmul.rs:2459-2465
    assert out.tolist() == [19, 22, 43, 50]
    a = np.full(128, -128, np.int8)
    out = np.zeros(1, np.int32)
    K.int8_matmul_dispatch(a, a, 1, 128, 1, out)  # :2503-2509
    assert out[0] == 128 * 128 * 128
    out = np.ones(9, np.int32)
    K.int8_matmul_dispatch(np.zeros(12, np.int8), np.zeros(12, np.int8), 3, 4, 3, out)  # :2449-2456
    assert (out == 0).all()


@pytest.mark.parametrize("m,k,n", REF_DISPATCH_SHAPES + REF_PREPACKED_SHAPES + EXTRA_SHAPES)
def test_dispatch_and_prepacked_match_scalar(oracle, K, m, k, n):
    a = oracle.lcg_i8(0xDEAD ^ (m * k), m * k)
    b = oracle.lcg_i8(0xBEEF ^ (k * n), k * n)
    exp = oracle.int8_matmul_scalar(a, b, m, k, n)
    got = np.full((m, n), np.iinfo(np.int32).min, np.int32)
    K.int8_matmul_dispatch(a, b, m, k, n, got)
    assert np.array_equal(got, exp)
    packed = K.pack_i8_b_for_matmul(b, k, n)
    assert packed.k() == k and packed.n() == n
    got2 = np.full((m, n), np.iinfo(np.int32).min, np.int32)
    K.int8_matmul_prepacked_dispatch(a, packed, m, got2)
    assert np.array_equal(got2, exp)


def test_config2_full_size_bit_exact(oracle, K, torch_cuda):
    """BASELINE config 2: A u8 [512][4096] zero point 128, B i8 [4096][4096] in -127..127; int32 result
    bit-exact, then requantised to u8 with composite 1/4096 and zero point 128."""
    torch = torch_cuda
    rng = np.random.default_rng(2000)
    m, k, n = 512, 4096, 4096
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-127, 128, (k, n), dtype=np.int8)
    exp = ((a.astype(np.int64) - 128) @ b.astype(np.int64)).astype(np.int64)
    assert np.abs(exp).max() < 2**31
    exp = exp.astype(np.int32)
    # spot-check the int64 formula against the restated scalar kernel on a few rows
    rows = [0, 255, 511]
    sub = oracle.u8i8_matmul_zp(a[rows], 128, b, len(rows), k, n)
    assert np.array_equal(sub, exp[rows])
    packed = K.pack_i8_b_for_matmul(b, k, n)
    a_dev = torch.from_numpy(a).cuda()
    got = packed.matmul(a_dev, a_zp=128).cpu().numpy()
    assert np.array_equal(got, exp)
    for mode in (K.ROUND_HALF_AWAY, K.ROUND_TIES_EVEN):
        q = packed.matmul_requant(a_dev, 128, 1.0 / 4096, 128.0, mode, 0, 255).cpu().numpy()
        q_exp = oracle.requant_general(exp, n, None, 1.0 / 4096, 128.0, mode, 0, 255)
        assert q.dtype == np.uint8 and np.array_equal(q.astype(np.int32), q_exp)
    # reference clamp range [-128,127] (linear.rs:484) with int8 activations and zero point 0
    a_s = (a ^ 0x80).view(np.int8)
    q = packed.matmul_requant(torch.from_numpy(a_s).cuda(), 0, 1.0 / 4096, 0.0, K.ROUND_HALF_AWAY, -128, 127).cpu().numpy()
    q_exp = oracle.requant_general(exp, n, None, 1.0 / 4096, 0.0, K.ROUND_HALF_AWAY, -128, 127)
    assert q.dtype == np.int8 and np.array_equal(q.astype(np.int32), q_exp)


# k a multiple of 64: the LDS-ring kernel.  Row / column tails, column counts that are not multiples of 4 or 16,
# several ring revolutions, and sizes on both sides of the 64x128 / 128x128 tile switch (256 big tiles).
RING_SHAPES = [(1, 64, 1), (65, 256, 129), (70, 2048, 250), (130, 1024, 260), (257, 4096, 515), (33, 192, 1030),
               (2048, 512, 2048), (2100, 320, 2050), (1999, 1088, 2500)]


@pytest.mark.parametrize("m,k,n", RING_SHAPES)
@pytest.mark.parametrize("signed", [False, True])
def test_ring_kernel_shapes_bit_exact(oracle, K, torch_cuda, m, k, n, signed):
    torch = torch_cuda
    rng = np.random.default_rng(m * 31 + k * 7 + n + int(signed))
    a = rng.integers(-128, 128, (m, k)).astype(np.int8) if signed else rng.integers(0, 256, (m, k)).astype(np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    zp = 0 if signed else int(rng.integers(0, 256))
    # float64 holds these sums exactly (|sum| < 2^31 << 2^53), so BLAS gives the integer reference quickly
    exp = ((a.astype(np.float64) - zp) @ b.astype(np.float64)).astype(np.int64)
    rows = [0, m // 2, m - 1]
    sub = (a[rows].astype(np.int64) - zp) @ b.astype(np.int64)  # the same rows in integer arithmetic
    assert np.array_equal(exp[rows], sub)
    packed = K.pack_i8_b_for_matmul(b, k, n)
    a_dev = torch.from_numpy(a).cuda()
    got = packed.matmul(a_dev, a_zp=zp).cpu().numpy()
    assert np.array_equal(got, exp.astype(np.int32))
    corr = rng.integers(-3000, 3000, n, dtype=np.int32)
    comp = rng.uniform(2e-5, 4e-4, n).astype(np.float32)
    lo, hi = (-128, 127) if signed else (0, 255)
    q = packed.matmul_requant(a_dev, zp, torch.from_numpy(comp).cuda(), 7.0, K.ROUND_HALF_AWAY, lo, hi,
                              corr=torch.from_numpy(corr).cuda()).cpu().numpy()
    q_exp = oracle.requant_general(exp.astype(np.int32), n, corr, comp, 7.0, K.ROUND_HALF_AWAY, lo, hi)
    assert np.array_equal(q.astype(np.int32), np.asarray(q_exp).reshape(m, n))


@pytest.mark.parametrize("zp", [0, 3, 128, 255])
def test_u8_zero_points(oracle, K, torch_cuda, zp):
    torch = torch_cuda
    rng = np.random.default_rng(zp)
    m, k, n = 70, 200, 150
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    exp = oracle.u8i8_matmul_zp(a, zp, b, m, k, n)
    got = K.pack_i8_b_for_matmul(b, k, n).matmul(torch.from_numpy(a).cuda(), a_zp=zp).cpu().numpy()
    assert np.array_equal(got, exp)


def test_fused_per_channel_requant(oracle, K, torch_cuda):
    """GEMM + per-column corr/composite epilogue == requant_i8_per_channel on the exact accumulators."""
    torch = torch_cuda
    rng = np.random.default_rng(5)
    m, k, n = 96, 320, 144
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    acc = oracle.int8_matmul_scalar(a, b, m, k, n)
    corr = rng.integers(-5000, 5000, n, dtype=np.int32)
    comp = rng.uniform(1e-4, 3e-3, n).astype(np.float32)
    exp = oracle.requant_i8_per_channel(acc.ravel(), corr, comp, 3.0, n).reshape(m, n)
    packed = K.pack_i8_b_for_matmul(b, k, n)
    got = packed.matmul_requant(torch.from_numpy(a).cuda(), 0, torch.from_numpy(comp).cuda(), 3.0, K.ROUND_TIES_EVEN,
                                -128, 127, corr=torch.from_numpy(corr).cuda()).cpu().numpy()
    assert np.array_equal(got, exp)


def test_qlinear_matmul_reference_example(oracle, K, torch_cuda):
    """crates/yscv-onnx/src/tests/qlinear.rs:150-194 through the fused kernel."""
    torch = torch_cuda
    a = (np.arange(32) - 16).astype(np.int8).reshape(4, 8)
    b = ((np.arange(32) * 7) % 31 - 15).astype(np.int8).reshape(8, 4)
    exp, fast = oracle.exec_qlinear_matmul(a.astype(np.float32), 0.05, 0.0, b.astype(np.float32), 0.1, 0.0, 0.25, 0.0, 4, 8, 4)
    assert fast
    comp = float(np.float32(np.float32(0.05) * np.float32(0.1)) / np.float32(0.25))
    got = K.pack_i8_b_for_matmul(b, 8, 4).matmul_requant(torch.from_numpy(a).cuda(), 0, comp, 0.0, K.ROUND_HALF_AWAY,
                                                         -128, 127).cpu().numpy()
    assert np.array_equal(got.astype(np.float32), exp)


def test_linearity_at_full_size(K, torch_cuda):
    """Size-independent property at the config-2 size: (A1 + A2) B == A1 B + A2 B in exact int32."""
    torch = torch_cuda
    g = torch.Generator(device="cuda").manual_seed(11)
    m, k, n = 512, 4096, 4096
    a1 = torch.randint(-60, 60, (m, k), device="cuda", generator=g, dtype=torch.int8)
    a2 = torch.randint(-60, 60, (m, k), device="cuda", generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (k, n), generator=torch.Generator().manual_seed(12), dtype=torch.int8)
    packed = K.pack_i8_b_for_matmul(b.numpy(), k, n)
    y1, y2, y12 = packed.matmul(a1), packed.matmul(a2), packed.matmul(a1 + a2)
    assert torch.equal(y12, y1 + y2)
    # and against torch's own integer matmul on a row sample (int64 on the CPU)
    rows = [0, 100, 511]
    ref = a1[rows].cpu().long() @ b.long()
    assert torch.equal(y1[rows].cpu().long(), ref)

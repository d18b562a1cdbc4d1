"""GPU parity of the packed-int4 matmul kernels against the CPU restatement of the reference,
through the C ABI.  Float parity bar: see gpu_util.int4_tolerances."""
import numpy as np
import pytest

from gpu_util import bf16_round, int4_tolerances, pack_zero_points

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch


@pytest.fixture(scope="module")
def K():
    from yscv_amd import kernels

    return kernels


def _rand_packed(rng, n, k):
    return rng.integers(0, 256, n * k // 2, dtype=np.uint8)


# ---- the reference's own unit-test shapes, through the exact-signature entry points -----------

@pytest.mark.parametrize("m_w,k,g,sw,sx", [(4, 128, 32, 0xCAFEBABE, 0xF00DBA12), (8, 256, 32, 0x12345678, 0x9ABCDEF0),
                                           (2, 32, 16, 0xDEADBEEF, 7), (3, 96, 6, 1, 2), (4, 64, 32, 0xAA, 0xBB)])
def test_gemv_dispatch_reference_shapes(oracle, K, m_w, k, g, sw, sx):
    # int4_matmul.rs:720-758, :857-900 (reference tolerance between its own kernels: 1e-4)
    packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(sw, m_w * k), m_w, k, g)
    x = oracle.lcg_f32(sx, k)
    ref = oracle.packed_int4_gemv_scalar(packed, scales, x, m_w, k, g)
    out = np.full(m_w, 999.0, np.float32)
    K.packed_int4_gemv_dispatch(packed, scales, x, out, m_w, k, g)
    assert np.abs(out - ref).max() <= 1e-4
    int4_tolerances(out, ref, k, x)


def test_gemv_zero_weights_emit_exact_zeros(oracle, K):
    # int4_matmul.rs:761-773
    m_w, k, g = 3, 32, 16
    packed, scales = oracle.pack_int4_symmetric_per_group(np.zeros(m_w * k, np.float32), m_w, k, g)
    out = np.full(m_w, 999.0, np.float32)
    K.packed_int4_gemv_dispatch(packed, scales, np.full(k, 1.5, np.float32), out, m_w, k, g)
    assert (out == 0).all()
    m_w, k, g = 20, 256, 32  # tiled path
    packed, scales = oracle.pack_int4_symmetric_per_group(np.zeros(m_w * k, np.float32), m_w, k, g)
    out = np.full(m_w, 999.0, np.float32)
    K.packed_int4_gemv_dispatch(packed, scales, np.full(k, 1.5, np.float32), out, m_w, k, g)
    assert (out == 0).all()


@pytest.mark.parametrize("m", [1, 4, 16, 32])
def test_gemm_dispatch_reference_shapes(oracle, K, m):
    # int4_matmul.rs:816-855 (reference tolerance 1e-3)
    n, k, g = 8, 64, 32
    packed, scales = oracle.pack_int4_symmetric_per_group(oracle.lcg_f32(0x100, n * k), n, k, g)
    x = oracle.lcg_f32(0x200 + m, m * k)
    ref = oracle.packed_int4_gemm_scalar(packed, scales, x, m, n, k, g)
    out = np.full((m, n), 999.0, np.float32)
    K.packed_int4_gemm_dispatch(packed, scales, x, out, m, n, k, g)
    assert np.abs(out - ref).max() <= 1e-3
    int4_tolerances(out, ref, k, x)


def test_hand_kat(K):
    # nibbles (1,2),(-8,-1), groups of 2, scales .5/.25, x = 1..4 -> -4.5 (generic kernel, g = 2)
    out = np.zeros(1, np.float32)
    K.packed_int4_gemv_dispatch(np.array([0x21, 0xF8], np.uint8), np.array([0.5, 0.25], np.float32),
                                np.array([1, 2, 3, 4], np.float32), out, 1, 4, 2)
    assert out.tolist() == [-4.5]


def test_pack_int4_bit_exact(oracle, K):
    rng = np.random.default_rng(31)
    for (m_w, k, g) in [(4, 64, 16), (7, 256, 32), (3, 384, 128), (2, 12, 6)]:
        w = rng.standard_normal(m_w * k).astype(np.float32)
        w[: g] = 0  # an all-zero group -> scale 1.0
        w[g] = np.float32(0.5) * np.float32(1e-3)
        p_ref, s_ref = oracle.pack_int4_symmetric_per_group(w, m_w, k, g)
        p, s = K.pack_int4_symmetric_per_group(w, m_w, k, g)
        assert np.array_equal(s, s_ref) and np.array_equal(p, p_ref)


def test_dequantize_int4_bit_exact(oracle, K):
    rng = np.random.default_rng(32)
    packed = rng.integers(0, 256, 777, dtype=np.uint8)
    for scale, zp in [(0.5, 0), (0.1, 2), (0.25, 1), (0.1, -3)]:
        out = np.empty(2 * packed.size, np.float32)
        K.dequantize_int4_to_f32(packed, scale, zp, out)
        assert np.array_equal(out, oracle.dequantize_int4_to_f32(packed, scale, zp))
    out = np.empty(2, np.float32)
    K.dequantize_int4_to_f32(np.array([0xE3], np.uint8), 0.5, 0, out)  # quantize.rs:681-688
    assert out.tolist() == [1.5, -1.0]


# ---- device handles: BASELINE config shapes -----------------------------------------------------

def test_config1_gemv_4096(oracle, K, torch_cuda):
    """BASELINE config 1: M=1 K=4096 N=4096, uint4 weights (zero point 8), g=32, f32 scales
    U(0.005,0.02), f32 activations N(0,1)."""
    torch = torch_cuda
    rng = np.random.default_rng(1000)
    n = k = 4096
    g = 32
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    ref = oracle.packed_int4_gemv_scalar(b ^ 0x88, scales, x, n, k, g)
    w = K.PackedInt4Weight(b, scales, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    y = w.matmul(torch.from_numpy(x).cuda().reshape(1, k)).cpu().numpy().ravel()
    d, rel = int4_tolerances(y, ref, k, x)
    assert rel < 2e-5, rel  # what hi+lo fp16 activations and fp32 group accumulation deliver
    # the same weight given in the reference's signed format is the same numbers
    w2 = K.PackedInt4Weight(b ^ 0x88, scales, g, n, k)
    y2 = w2.matmul(torch.from_numpy(x).cuda().reshape(1, k)).cpu().numpy().ravel()
    assert np.array_equal(y, y2)
    # explicit zero points that are all 8 take the same path
    zp8 = np.full((n, (k // g + 1) // 2), 0x88, np.uint8)
    w3 = K.PackedInt4Weight(b, scales, g, n, k, zero_points=zp8, nibble_format=K.NIBBLE_UNSIGNED)
    y3 = w3.matmul(torch.from_numpy(x).cuda().reshape(1, k)).cpu().numpy().ravel()
    assert np.array_equal(y, y3)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 11, 16])
@pytest.mark.parametrize("xdt", ["f32", "f16", "bf16"])
def test_skinny_all_m_and_dtypes(oracle, K, torch_cuda, m, xdt):
    torch = torch_cuda
    rng = np.random.default_rng(2000 + m)
    n, k, g = 528, 1024, 32
    b = _rand_packed(rng, n, k)
    scales16 = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[xdt]
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(tdt)
    x = xt.float().numpy()  # exact widening of what the kernel sees
    ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales16.astype(np.float32), x, m, n, k, g)
    w = K.PackedInt4Weight(b, scales16, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    y = w.matmul(xt.cuda(), out_dtype=torch.float32, mode="gemv").cpu().numpy()
    d, rel = int4_tolerances(y, ref, k, x)
    # f32 input: hi + lo activations against exact weights.  fp16 / bf16 input with symmetric weights: the 1024-offsets
    # stay in the weights and are cancelled per group in fp32, which costs a few units of 1e-5.
    assert rel < (2e-5 if xdt == "f32" else 5e-5), rel
    # GEMM kernel on the same data agrees with the skinny kernel to fp32 rounding
    y2 = w.matmul(xt.cuda(), out_dtype=torch.float32, mode="gemm").cpu().numpy()
    int4_tolerances(y2, ref, k, x)
    assert np.abs(y2 - y).max() <= 1e-4 * np.abs(ref).max()


@pytest.mark.parametrize("m", [1, 16])
def test_skinny_long_k_grid_split(oracle, K, torch_cuda, m):
    """K = 14336 (Llama down projection) needs the grid-level K split + fixed-order reduction."""
    torch = torch_cuda
    rng = np.random.default_rng(2100 + m)
    n, k, g = 272, 14336, 32
    b = _rand_packed(rng, n, k)
    scales16 = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).half()
    x = xt.float().numpy()
    ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales16.astype(np.float32), x, m, n, k, g)
    w = K.PackedInt4Weight(b, scales16, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    y = w.matmul(xt.cuda(), out_dtype=torch.float32).cpu().numpy()
    d, rel = int4_tolerances(y, ref, k, x)
    assert rel < 5e-5, rel
    y_again = w.matmul(xt.cuda(), out_dtype=torch.float32).cpu().numpy()
    assert np.array_equal(y, y_again)  # no atomics: bitwise reproducible


@pytest.mark.parametrize("g", [64, 128, 256])
@pytest.mark.parametrize("m", [3, 40])
def test_group_sizes_and_zero_points(oracle, K, torch_cuda, g, m):
    """Config-3 style weights: uint4 with zero points 6..10, fp16 scales, bf16 in / bf16 out."""
    torch = torch_cuda
    rng = np.random.default_rng(3000 + g + m)
    n, k = 200, 1024
    groups = k // g
    b = _rand_packed(rng, n, k)
    scales16 = rng.uniform(0.005, 0.02, n * groups).astype(np.float16)
    zq = rng.integers(6, 11, (n, groups))
    zps = pack_zero_points(zq)
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16()
    x = xt.float().numpy()
    ref = oracle.matmul_nbits(b, scales16.astype(np.float32), zps, x, m, n, k, g)
    w = K.PackedInt4Weight(b, scales16, g, n, k, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    y32 = w.matmul(xt.cuda(), out_dtype=torch.float32).cpu().numpy()
    d, rel = int4_tolerances(y32, ref, k, x)
    # m <= 16: exact integer weights, f32 scales; above: weights decoded to fp16 with the scale folded in
    assert rel < (5e-5 if m <= 16 else 1e-3), rel
    # bf16 output = RNE narrowing of the f32 result (crates/yscv-tensor/src/tensor.rs:764-769)
    ybf = w.matmul(xt.cuda()).float().cpu().numpy()
    assert np.array_equal(ybf, bf16_round(y32))
    int4_tolerances(ybf, bf16_round(ref), k, x)


@pytest.mark.parametrize("n,k,g", [(37, 160, 32), (1, 32, 32), (17, 96, 32), (33, 192, 64)])
def test_ragged_shapes(oracle, K, torch_cuda, n, k, g):
    """N not a multiple of 16, K not a multiple of 128: padding must not leak into results."""
    torch = torch_cuda
    rng = np.random.default_rng(n * 1000 + k)
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    for m in (1, 7, 20):
        x = rng.standard_normal((m, k)).astype(np.float32)
        ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales, x, m, n, k, g)
        w = K.PackedInt4Weight(b, scales, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
        canary = torch.full((m + 1, n), 777.0, device="cuda")
        w.matmul(torch.from_numpy(x).cuda(), out=canary[:m])
        y = canary.cpu().numpy()
        assert (y[m] == 777.0).all()  # nothing written past the m rows
        d, rel = int4_tolerances(y[:m], ref, k, x)
        assert rel < 2e-5, rel


def test_activation_range_is_normalised(oracle, K, torch_cuda):
    """Huge and tiny activation rows go through the power-of-two normalisation unharmed."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    n, k, g = 64, 512, 32
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    x = rng.standard_normal((4, k)).astype(np.float32)
    x[0] *= 1e6
    x[1] *= 1e-6
    x[2] = 0
    ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales, x, 4, n, k, g)
    w = K.PackedInt4Weight(b, scales, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    y = w.matmul(torch.from_numpy(x).cuda()).cpu().numpy()
    for i in range(4):
        if i == 2:
            assert (y[i] == 0).all()
        else:
            int4_tolerances(y[i], ref[i], k, x[i])
            assert np.abs(y[i] - ref[i]).max() <= 2e-5 * np.abs(ref[i]).max()


def test_invalid_arguments_are_rejected(K, torch_cuda):
    import yscv_amd

    with pytest.raises(yscv_amd.YscvHipError) as ei:
        K.PackedInt4Weight(np.zeros(9, np.uint8), np.zeros(6, np.float32), 3, 2, 9)  # odd group size
    assert ei.value.code == -1
    with pytest.raises(yscv_amd.YscvHipError):
        K.PackedInt4Weight(np.zeros(10, np.uint8), np.zeros(2, np.float32), 6, 2, 10)  # g does not divide k
    w = K.PackedInt4Weight(np.zeros(32 * 16, np.uint8), np.ones(32, np.float32), 32, 32, 32)
    x = torch_cuda.zeros(17, 32, device="cuda")
    with pytest.raises(yscv_amd.YscvHipError):
        w.matmul(x, mode="gemv")  # skinny kernel is m <= 16


@pytest.mark.parametrize("m,n,k,g,sf16,zp", [(17, 40, 128, 32, True, False), (33, 300, 256, 64, False, True), (100, 129, 1536, 128, True, True),
                                               (128, 128, 512, 32, False, False), (130, 200, 1024, 128, True, True),
                                               (257, 1000, 640, 64, True, True), (512, 136, 2048, 32, True, False),
                                               (300, 264, 768, 256, False, True), (1100, 520, 1152, 128, False, False),
                                               (200, 24011, 256, 32, True, True), (250, 16499, 256, 64, True, True),
                                               (250, 40997, 128, 32, True, False)])  # the last three: 128 x 256 tiles, 256 x 128 tiles, and one round of
                                                                                      # 256 x 128 tiles followed by a second launch with 128 x 128 tiles
@pytest.mark.parametrize("xdt", ["bf16", "f16", "f32"])
def test_wide_m_ring_kernel(oracle, K, torch_cuda, m, n, k, g, sf16, zp, xdt):
    """m > 16: the LDS-ring GEMM (weights decoded to fp16 with the scale folded in) for 16-bit activations and, when
    the weight's scales are fp16, for f32 activations as well; f32 activations against f32 scales take the exact-scale
    kernel and meet the same bars with room to spare.
    Row / column tails, every group mode, f32 and fp16 scales, with and without zero points, all output types."""
    torch = torch_cuda
    rng = np.random.default_rng(m + n * 3 + k * 7 + g)
    groups = k // g
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * groups).astype(np.float16 if sf16 else np.float32)
    zq = rng.integers(6, 11, (n, groups)) if zp else np.full((n, groups), 8)
    zps = pack_zero_points(zq) if zp else None
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32))
    xt = xt.bfloat16() if xdt == "bf16" else (xt.half() if xdt == "f16" else xt)
    x = xt.float().numpy()
    ref = oracle.matmul_nbits(b, scales.astype(np.float32), pack_zero_points(zq), x, m, n, k, g)
    w = K.PackedInt4Weight(b, scales, g, n, k, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    canary = torch.full((m + 1, n), 777.0, device="cuda")
    w.matmul(xt.cuda(), out=canary[:m])
    y32 = canary.cpu().numpy()
    assert (y32[m] == 777.0).all()
    d, rel = int4_tolerances(y32[:m], ref, k, x)
    assert rel < 1e-3, rel  # fp16 rounding of (q - zp) * scale: about 2^-11 per weight, averaged over k
    y16 = w.matmul(xt.cuda(), out_dtype=torch.bfloat16).float().cpu().numpy()
    assert np.array_equal(y16, bf16_round(y32[:m]))
    yh = w.matmul(xt.cuda(), out_dtype=torch.float16).float().cpu().numpy()
    assert np.array_equal(yh, y32[:m].astype(np.float16).astype(np.float32))
    # the same rows through the m <= 16 kernel (exact integer weights, f32 scales) agree to the same bar
    ys = w.matmul(xt[:16].cuda(), out_dtype=torch.float32).cpu().numpy()
    assert np.abs(ys - y32[:16]).max() <= 1e-3 * np.abs(ref).max()


def test_prefill_gemm_sampled_at_full_size(oracle, K, torch_cuda):
    """BASELINE config 3 at full size (M=2048 K=4096 N=14336, g=128, fp16 scales, zero points 6..10,
    bf16 in/out); the oracle is evaluated on a sample of rows and columns."""
    torch = torch_cuda
    rng = np.random.default_rng(3)
    m, k, n, g = 2048, 4096, 14336, 128
    groups = k // g
    b = _rand_packed(rng, n, k)
    scales16 = rng.uniform(0.005, 0.02, n * groups).astype(np.float16)
    zq = rng.integers(6, 11, (n, groups))
    zps = pack_zero_points(zq)
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16()
    w = K.PackedInt4Weight(b, scales16, g, n, k, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    y = w.matmul(xt.cuda())
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, n)
    rows = np.sort(rng.choice(m, 24, replace=False))
    cols = np.sort(rng.choice(n, 96, replace=False))
    xs = xt.float().numpy()[rows]
    bs = b.reshape(n, k // 2)[cols]
    ss = scales16.reshape(n, groups)[cols].astype(np.float32)
    zs = pack_zero_points(zq[cols])
    ref = oracle.matmul_nbits(bs, ss, zs, xs, len(rows), len(cols), k, g)
    got = y.float().cpu().numpy()[np.ix_(rows, cols)]
    int4_tolerances(got, bf16_round(ref), k, xs)
    # bf16 output: at most one bf16 ulp away from the rounded oracle
    assert np.abs(got - bf16_round(ref)).max() <= np.abs(ref).max() * 2.0 ** -7


@pytest.mark.parametrize("layout", ["kn", "nk"])
@pytest.mark.parametrize("g", [32, 128])
def test_int4_weight_from_f32_matches_the_packing_pass(oracle, K, torch_cuda, layout, g):
    """quantize_matmul_weights_int4_packed (packed_int4.rs:50-128) on one f32 initialiser: transposition for the
    [K, N] layouts, symmetric per-group packing bit-exact with pack_int4_symmetric_per_group, skip rules."""
    torch = torch_cuda
    rng = np.random.default_rng(g + len(layout))
    n, k = 48, 256
    w_nk = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    w_nk[3, :g] = 0.0  # an all-zero group: scale 1.0
    dev = torch.from_numpy(w_nk if layout == "nk" else np.ascontiguousarray(w_nk.T)).cuda()
    w = K.PackedInt4Weight.from_f32(dev, g, transposed_nk=(layout == "nk"))
    assert w is not None and (w.m_w, w.k) == (n, k)
    packed, scales = oracle.pack_int4_symmetric_per_group(w_nk.ravel(), n, k, g)
    x = rng.standard_normal((3, k)).astype(np.float32)
    ref = oracle.packed_int4_gemm_scalar(packed, scales, x, 3, n, k, g)
    y = w.matmul(torch.from_numpy(x).cuda()).cpu().numpy()
    d, rel = int4_tolerances(y, ref, k, x)
    assert rel < 2e-5, rel  # same packed nibbles and scales as the reference pass, exact-weight kernel
    # skip rules and the group-size error
    assert K.PackedInt4Weight.from_f32(torch.zeros(100, 8, device="cuda"), 32) is None          # K % group != 0
    assert K.PackedInt4Weight.from_f32(torch.zeros(2, 8, device="cuda"), 2, transposed_nk=True) is None  # K * N < 32
    import yscv_amd

    for bad in (0, 7):
        with pytest.raises(yscv_amd.YscvHipError) as ei:
            K.PackedInt4Weight.from_f32(dev, bad, transposed_nk=(layout == "nk"))
        assert ei.value.code == -1 and "group_size must be even" in ei.value.message


def test_lm_head_sweep_sampled_at_full_size(oracle, K, torch_cuda):
    """BASELINE config 5 at full size (K=4096, N=128256, g=32, bf16 activations), M across the switch from the skinny
    kernel (m <= 16) to the LDS-ring GEMM: the oracle is evaluated on a sample of columns, every row."""
    torch = torch_cuda
    rng = np.random.default_rng(55)
    k, n, g = 4096, 128256, 32
    groups = k // g
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales16 = rng.uniform(0.005, 0.02, n * groups).astype(np.float16)
    w = K.PackedInt4Weight(b, scales16, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    cols = np.sort(rng.choice(n, 80, replace=False))
    cols[-1] = n - 1  # the last row of the weight: the column tail of the last tile
    bs = b.reshape(n, k // 2)[cols]
    ss = scales16.reshape(n, groups)[cols].astype(np.float32)
    for m in (1, 2, 4, 5, 8, 16, 17, 32, 64, 128, 256):  # every M of the BASELINE sweep + both sides of the switch
        xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16()
        xs = xt.float().numpy()
        ref = oracle.packed_int4_gemm_scalar(bs ^ 0x88, ss, xs, m, len(cols), k, g)
        y = w.matmul(xt.cuda())
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, n)
        got = y.float().cpu().numpy()[:, cols]
        int4_tolerances(got, bf16_round(ref), k, xs)
        assert np.abs(got - bf16_round(ref)).max() <= np.abs(ref).max() * 2.0 ** -7, m
    w.close()


def test_every_output_at_lm_head_shape(K, torch_cuda):
    """Every element of the output at the LM-head shape (K=4096, N=128256), for row counts that select the skinny kernel
    with one, two and four accumulators and each tile shape of the MFMA GEMM (32-, 64-row, 128 x 256, 256 x 128), three
    calls each: against an fp32 product with the dequantised weight on the GPU (tolerance of the bf16 output), and
    bit-identical from call to call.  A sampled check misses a weight tile that goes wrong now and then (a few
    16-column blocks of a hundred thousand columns)."""
    torch = torch_cuda
    rng = np.random.default_rng(56)
    k, n, g = 4096, 128256, 32
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales16 = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    w = K.PackedInt4Weight(b, scales16, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    bt = torch.from_numpy(b.reshape(n, k // 2)).cuda()
    wd = torch.stack(((bt & 15).float() - 8.0, (bt >> 4).float() - 8.0), dim=2).reshape(n, k // g, g)
    del bt
    wd = (wd * torch.from_numpy(scales16.reshape(n, k // g).astype(np.float32)).cuda()[:, :, None]).reshape(n, k)
    x_all = torch.from_numpy(rng.standard_normal((256, k)).astype(np.float32)).bfloat16().cuda()
    for m in (1, 4, 8, 16, 24, 64, 96, 128, 200, 256):
        x = x_all[:m].contiguous()
        ref = x.float() @ wd.T
        bound = float(ref.abs().max()) * 2.0 ** -7
        first = None
        for rep in range(3):
            y = w.matmul(x)
            err = float((y.float() - ref).abs().nan_to_num(1e9).max())
            assert err <= bound, (m, rep, err, bound)
            if first is None:
                first = y
            else:
                assert torch.equal(y, first), (m, rep)
        del ref
    w.close()


def test_every_output_at_the_prefill_shape(K, torch_cuda):
    """Every element of BASELINE config 3's output (M=2048, K=4096, N=14336, g=128, fp16 scales, zero points 6..10,
    bf16 in and out) -- the 128-k-group instantiation with explicit zero points and every column range the call is
    cut into -- against an fp32 product with the dequantised weight on the GPU (tolerance: the bf16 rounding of
    the output), three calls, bit-identical from call to call.  Also with 2000 rows: a last row tile that is not full."""
    torch = torch_cuda
    rng = np.random.default_rng(57)
    m, k, n, g = 2048, 4096, 14336, 128
    groups = k // g
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales16 = rng.uniform(0.005, 0.02, n * groups).astype(np.float16)
    zq = rng.integers(6, 11, (n, groups))
    w = K.PackedInt4Weight(b, scales16, g, n, k, zero_points=pack_zero_points(zq), nibble_format=K.NIBBLE_UNSIGNED)
    bt = torch.from_numpy(b.reshape(n, k // 2)).cuda()
    wd = torch.stack(((bt & 15).float(), (bt >> 4).float()), dim=2).reshape(n, groups, g)
    del bt
    wd = wd - torch.from_numpy(zq.astype(np.float32)).cuda()[:, :, None]
    wd = (wd * torch.from_numpy(scales16.reshape(n, groups).astype(np.float32)).cuda()[:, :, None]).reshape(n, k)
    x_all = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16().cuda()
    for rows in (m, 2000):
        x = x_all[:rows].contiguous()
        ref = x.float() @ wd.T
        bound = float(ref.abs().max()) * 2.0 ** -7
        first = None
        for rep in range(3):
            y = w.matmul(x)
            assert y.dtype == torch.bfloat16 and tuple(y.shape) == (rows, n)
            err = float((y.float() - ref).abs().nan_to_num(1e9).max())
            assert err <= bound, (rows, rep, err, bound)
            if first is None:
                first = y
            else:
                assert torch.equal(y, first), (rows, rep)
        del ref
    w.close()


def test_weight_loaded_from_a_file_equals_the_uploaded_one(K, torch_cuda, tmp_path):
    """yscv_hip_int4_weight_load: the on-disk form carries exactly the arguments of the upload call."""
    torch = torch_cuda
    rng = np.random.default_rng(77)
    n, k, g = 272, 768, 64
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    zq = rng.integers(5, 12, (n, k // g))
    zps = pack_zero_points(zq)
    path = tmp_path / "w.yi4"
    K.int4_file_write(path, b, scales, g, n, k, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    w0 = K.PackedInt4Weight(b, scales, g, n, k, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    w1 = K.PackedInt4Weight.load(path)
    assert (w1.m_w, w1.k, w1.group_size) == (n, k, g) and w1.device_bytes() == w0.device_bytes()
    for m in (1, 9, 40):
        x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).half().cuda()
        assert torch.equal(w0.matmul(x, out_dtype=torch.float32), w1.matmul(x, out_dtype=torch.float32))


@pytest.mark.parametrize("m,xdt", [(3, "bf16"), (3, "f32"), (40, "bf16"), (300, "f16")])
def test_caller_workspace_gives_the_same_bits(K, torch_cuda, m, xdt):
    """yscv_hip_int4_matmul_ws: scratch from the caller instead of the stream-ordered allocator, same result."""
    torch = torch_cuda
    rng = np.random.default_rng(91 + m)
    n, k, g = 300, 1000 if xdt == "f32" else 1024, 8 if xdt == "f32" else 64   # k = 1000: padded K, activation pass needed
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    w = K.PackedInt4Weight(b, scales, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[xdt]
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(tdt).cuda()
    need = w.workspace_bytes(m, tdt)
    ws = torch.full((need + 256,), 0xA5, dtype=torch.uint8, device="cuda")
    y0 = w.matmul(x, out_dtype=torch.float32)
    y1 = w.matmul(x, out_dtype=torch.float32, workspace=ws[: max(need, 1)])
    assert torch.equal(y0, y1)
    assert bool((ws[need:] == 0xA5).all())  # nothing written past the announced size
    if need > 0:
        with pytest.raises(Exception, match="workspace too small"):
            w.matmul(x, out_dtype=torch.float32, workspace=ws[: need - 1])


def test_f32_rows_beyond_16_run_as_skinny_passes(oracle, K, torch_cuda):
    """f32 activations against f32 scales with 16 < m <= 128: 16-row passes of the exact skinny kernel (K-split and
    caller workspace included) -- every row equals what a call with that row alone gives."""
    torch = torch_cuda
    rng = np.random.default_rng(123)
    n, k, g, m = 272, 14336, 32, 40
    b = _rand_packed(rng, n, k)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float32)
    w = K.PackedInt4Weight(b, scales, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).cuda()
    ws = torch.empty(w.workspace_bytes(m, torch.float32), dtype=torch.uint8, device="cuda")
    canary = torch.full((m + 1, n), 777.0, device="cuda")
    w.matmul(x, out=canary[:m], workspace=ws)
    y = canary[:m].clone()
    assert bool((canary[m] == 777.0).all())
    assert torch.equal(y, w.matmul(x))  # allocator-backed call: same bits
    for r0 in (0, 16, 32):
        assert torch.equal(y[r0:r0 + 16], w.matmul(x[r0:r0 + 16], mode="gemv"))
    ref = oracle.packed_int4_gemm_scalar(b ^ 0x88, scales, x[:3].cpu().numpy(), 3, n, k, g)
    d, rel = int4_tolerances(y[:3].cpu().numpy(), ref, k, x[:3].cpu().numpy())
    assert rel < 5e-5, rel


@pytest.mark.parametrize("n,k", [(4096, 14336), (4096, 4096), (28672, 4096)])
@pytest.mark.parametrize("m", [1, 3, 16])
def test_fused_epilogues_at_decoder_shapes(oracle, K, torch_cuda, n, k, m):
    """yscv_hip_int4_matmul_fused at the projection shapes of the 7B-shape decoder: the down projection (K = 14336, grid
    K split with the second-pass kernel) adding into an f32 residual, and the gate / up projection (rows interleaved)
    with SwiGLU, against the scalar oracle on a sample of output rows; fp16 activations and scales like the decoder."""
    torch = torch_cuda
    rng = np.random.default_rng(1000 + n + k + m)
    g = 32
    b = _rand_packed(rng, n, k)
    scales16 = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    w = K.PackedInt4Weight(b, scales16, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    xt = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).half()
    xs = xt.float().numpy()
    pairs = np.sort(rng.choice(n // 2, 48, replace=False))
    pairs[-1] = n // 2 - 1
    rows = np.stack([2 * pairs, 2 * pairs + 1], 1).reshape(-1)  # gate_i, up_i of the sampled pairs
    bs = b.reshape(n, k // 2)[rows]
    ss = scales16.reshape(n, k // g)[rows].astype(np.float32)
    ref = oracle.packed_int4_gemm_scalar(bs ^ 0x88, ss, xs, m, len(rows), k, g).reshape(m, len(rows))
    # store
    y = torch.full((m, n), 7.0, device="cuda")
    w.matmul_fused(xt.cuda(), y, K.EPILOGUE_STORE)
    int4_tolerances(y.cpu().numpy()[:, rows], ref, k, xs)
    assert torch.equal(y, w.matmul(xt.cuda(), out_dtype=torch.float32, mode="gemv"))
    # residual add: y += x W^T on an f32 residual
    resid = rng.standard_normal((m, n)).astype(np.float32) * 10
    y = torch.from_numpy(resid).cuda()
    w.matmul_fused(xt.cuda(), y, K.EPILOGUE_ADD_F32)
    got = y.cpu().numpy()
    int4_tolerances(got[:, rows] - resid[:, rows], ref, k, xs)  # f32 add of the two: one rounding of |resid + y| on top
    # SwiGLU: out[i] = silu(gate_i) * up_i, fp16 out like the decoder and f32 out
    gate, up = ref[:, 0::2].astype(np.float64), ref[:, 1::2].astype(np.float64)
    want = gate / (1.0 + np.exp(-gate)) * up
    for odt in (torch.float16, torch.float32):
        act = torch.full((m, n // 2), 7.0, device="cuda", dtype=odt)
        w.matmul_fused(xt.cuda(), act, K.EPILOGUE_SWIGLU)
        ga = act.float().cpu().numpy()[:, pairs]
        err = np.abs(ga - want).max() / np.abs(want).max()
        assert err < (2e-3 if odt == torch.float16 else 1e-3), (odt, err)
    with pytest.raises(Exception, match="m <= 16"):
        w.matmul_fused(torch.zeros(17, k, device="cuda"), torch.zeros(17, n, device="cuda"), K.EPILOGUE_ADD_F32)
    w.close()


@pytest.mark.parametrize("n,k,m", [(4096, 14336, 200), (28672, 4096, 300), (4096, 4096, 17), (1000, 512, 40)])
def test_fused_epilogues_above_16_rows(K, torch_cuda, n, k, m):
    """The same epilogues on the LDS-ring GEMM (what the prompt pass runs): every output against the unfused call of the
    same kernel -- the residual add is one f32 addition on top of it, SwiGLU the same expression on its f32 sums."""
    torch = torch_cuda
    rng = np.random.default_rng(1100 + n + k + m)
    g = 32
    w = K.PackedInt4Weight(_rand_packed(rng, n, k), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16), g, n, k,
                           nibble_format=K.NIBBLE_UNSIGNED)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).half().cuda()
    plain = w.matmul(x, out_dtype=torch.float32)
    resid = torch.from_numpy((rng.standard_normal((m, n)) * 10).astype(np.float32)).cuda()
    y = torch.empty(m + 1, n, device="cuda")
    y[:m] = resid
    y[m] = 3.0
    w.matmul_fused(x, y[:m], K.EPILOGUE_ADD_F32)
    assert torch.equal(y[:m], resid + plain) and bool((y[m] == 3.0).all())
    want = torch.nn.functional.silu(plain[:, 0::2].double()) * plain[:, 1::2].double()
    for odt in (torch.float16, torch.float32):
        act = torch.full((m + 1, n // 2), 7.0, device="cuda", dtype=odt)
        w.matmul_fused(x, act[:m], K.EPILOGUE_SWIGLU)
        err = float((act[:m].double() - want).abs().max() / want.abs().max())
        assert err < (2e-3 if odt == torch.float16 else 1e-5), (odt, err)
        assert bool((act[m] == 7.0).all())
    w.close()


def _dequant_on_gpu(torch, b, scales, n, k, g, zq=None):
    """[n][k] f32 weight from packed nibbles (element 2i in the low nibble), per-group scales and zero points."""
    bt = torch.from_numpy(b.reshape(n, k // 2)).cuda()
    q = torch.stack(((bt & 15).float(), (bt >> 4).float()), dim=2).reshape(n, k // g, g)
    z = 8.0 if zq is None else torch.from_numpy(zq.astype(np.float32)).cuda()[:, :, None]
    sc = torch.from_numpy(scales.reshape(n, k // g).astype(np.float32)).cuda()[:, :, None]
    return ((q - z) * sc).reshape(n, k)


def test_random_shapes_every_output(K, torch_cuda):
    """Forty shapes drawn from a fixed seed -- row counts on both sides of every kernel and tile switch, ragged N, K from
    one tile to the down projection's 14336, all group sizes, zero points, f32 / fp16 scales, every activation type --
    with EVERY output element held against an fp32 product on the GPU (bar: the int4 tolerance of the kernels, plus the
    rounding of a 16-bit output), twice, the second call bit-identical to the first."""
    torch = torch_cuda
    rng = np.random.default_rng(20260)
    ms = [1, 2, 4, 5, 8, 9, 16, 17, 31, 32, 33, 64, 65, 100, 128, 129, 255, 256, 257, 384, 513]
    for case in range(40):
        m = int(rng.choice(ms))
        g = int(rng.choice([32, 32, 64, 128]))
        k = int(rng.choice([128, 256, 384, 1024, 2048, 4096, 14336]))
        if k % g:
            k = (k // g) * g
        n = int(rng.choice([16, 48, 100, 257, 1000, 4096, 6144, 11008, 24011]))
        if m * n * k > 2.2e11:  # keep the case under a second
            n = 1000
        sf16 = bool(rng.integers(0, 2))
        has_zp = bool(rng.integers(0, 2))
        xdt = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
        b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
        scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16 if sf16 else np.float32)
        zq = rng.integers(5, 12, (n, k // g)) if has_zp else None
        w = K.PackedInt4Weight(b, scales, g, n, k, zero_points=pack_zero_points(zq) if has_zp else None,
                               nibble_format=K.NIBBLE_UNSIGNED)
        wd = _dequant_on_gpu(torch, b, scales, n, k, g, zq)
        x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(xdt).cuda()
        ref = x.float() @ wd.T
        y = w.matmul(x)
        tag = (case, m, n, k, g, sf16, has_zp, str(xdt))
        assert tuple(y.shape) == (m, n) and y.dtype == xdt, tag
        err = float((y.float() - ref).abs().nan_to_num(1e9).max())
        top = float(ref.abs().max())
        out_round = {torch.float32: 0.0, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[xdt]
        assert err <= top * (1e-3 + out_round) + 1e-6, tag + (err, top)
        assert err <= 1e-3 * np.sqrt(k) * float(x.float().abs().max()), tag + (err,)
        assert torch.equal(w.matmul(x), y), tag
        w.close()
        del wd, ref


@pytest.mark.parametrize("m,n,k,g,has_zp", [
    (17, 4096, 4096, 32, False),    # 17 .. 32 rows: the register-resident kernel, one workgroup covers all of K
    (24, 1000, 14336, 32, True),    # the same kernel with K cut into four parts (f32 partial sums + second kernel), ragged N
    (32, 6144, 4608, 128, False),   # K not a multiple of what a workgroup covers: the last part's trailing waves idle
    (40, 1001, 2048, 64, True),     # ragged N (scalar stores of the partial sums), zero points
    (64, 6144, 4096, 32, False),    # the q/k/v projection of a 64-token prompt
    (100, 4096, 14336, 128, True),  # the down projection of a 100-token prompt: 64-row tiles, long K
    (200, 512, 4096, 32, False),    # few columns
    (256, 4096, 4096, 128, False),  # 64-row tiles preferred to 128-row ones, split in two
    (512, 4096, 4096, 32, False),   # 64-row tiles fill the CUs without a split
])
def test_k_split_shapes_every_output(K, torch_cuda, m, n, k, g, has_zp):
    """Shapes with fewer output tiles than half the CUs: the LDS-ring GEMM is cut along K as well, the splits' f32
    partial sums go through the workspace and a second kernel adds them in a fixed order and applies the epilogue;
    17 .. 32 rows take the kernel of int4_mid.hip, which cuts K into parts beyond 4096.
    Every output of the plain call against an fp32 product on the GPU, twice with the same bits, the same bits with a
    caller's workspace (nothing written past the announced size), and both fused epilogues against the plain result."""
    torch = torch_cuda
    rng = np.random.default_rng(7000 + m + n)
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    zq = rng.integers(5, 12, (n, k // g)) if has_zp else None
    w = K.PackedInt4Weight(b, scales, g, n, k, zero_points=pack_zero_points(zq) if has_zp else None,
                           nibble_format=K.NIBBLE_UNSIGNED)
    wd = _dequant_on_gpu(torch, b, scales, n, k, g, zq)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).half().cuda()
    ref = x.float() @ wd.T
    y = w.matmul(x, out_dtype=torch.float32)
    err, top = float((y - ref).abs().nan_to_num(1e9).max()), float(ref.abs().max())
    assert err <= top * 1e-3 + 1e-6, (err, top)
    assert torch.equal(w.matmul(x, out_dtype=torch.float32), y)
    need = w.workspace_bytes(m, torch.float16)
    ws = torch.full((need + 256,), 0xA5, dtype=torch.uint8, device="cuda")
    assert torch.equal(w.matmul(x, out_dtype=torch.float32, workspace=ws[: max(need, 1)]), y)
    assert bool((ws[need:] == 0xA5).all())
    resid = torch.from_numpy((rng.standard_normal((m, n)) * 10).astype(np.float32)).cuda()
    acc = torch.empty(m + 1, n, device="cuda")
    acc[:m] = resid
    acc[m] = 3.0
    w.matmul_fused(x, acc[:m], K.EPILOGUE_ADD_F32)
    assert torch.equal(acc[:m], resid + y) and bool((acc[m] == 3.0).all())
    if n % 2 == 0:
        want = torch.nn.functional.silu(y[:, 0::2].double()) * y[:, 1::2].double()
        act = torch.full((m + 1, n // 2), 7.0, device="cuda", dtype=torch.float32)
        w.matmul_fused(x, act[:m], K.EPILOGUE_SWIGLU)
        assert float((act[:m].double() - want).abs().max() / want.abs().max()) < 1e-5
        assert bool((act[m] == 7.0).all())
    w.close()

"""GPU parity of the operator layer (MatMulInteger, QLinearMatMul, QuantizeLinear, DequantizeLinear,
DynamicQuantizeLinear on f32 carriers) against the CPU restatement of the reference runner, through the C ABI."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))

SHAPES = [(1, 1, 1), (2, 3, 4), (5, 17, 6), (4, 64, 16), (8, 127, 33), (33, 200, 70), (64, 512, 128)]


@pytest.fixture(scope="module")
def torch_cuda():
    import torch

    assert torch.cuda.is_available()
    return torch


@pytest.fixture(scope="module")
def ops():
    from yscv_amd import onnx_ops

    return onnx_ops


def _dev(torch, a, shape=None):
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
    return t.reshape(shape) if shape is not None else t


def test_reference_known_answers(torch_cuda, ops):
    torch = torch_cuda
    for c in KATS["matmul_integer"]["cases"]:  # coverage.rs:359-390, gemm_matmul.rs:73-87
        out, path = ops.exec_matmul_integer(_dev(torch, c["a"], (c["m"], c["k"])), _dev(torch, c["b"], (c["k"], c["n"])),
                                            a_zp=float(c["a_zp"]))
        assert out.cpu().numpy().ravel().tolist() == [float(v) for v in c["expected"]]
        assert path == (ops.PATH_FAST if c["a_zp"] == 0 else ops.PATH_FALLBACK_EXACT)
    q = KATS["qlinear_matmul"]  # qlinear.rs:150-194
    m, k, n = q["m"], q["k"], q["n"]
    a = np.array([v - 16 for v in range(m * k)], np.float32)
    b = np.array([(7 * v) % 31 - 15 for v in range(k * n)], np.float32)
    comp = np.float32(np.float32(q["a_scale"]) * np.float32(q["b_scale"])) / np.float32(q["y_scale"])
    acc = a.reshape(m, k).astype(np.int64) @ b.reshape(k, n).astype(np.int64)
    v = acc.astype(np.float32) * comp
    exp = np.clip(np.where(v >= 0, np.floor(v + np.float32(0.5)), -np.floor(-v + np.float32(0.5))), -128, 127)
    out, path = ops.exec_qlinear_matmul(_dev(torch, a, (m, k)), q["a_scale"], 0.0, _dev(torch, b, (k, n)), q["b_scale"], 0.0,
                                        q["y_scale"], 0.0)
    assert path == ops.PATH_FAST and np.array_equal(out.cpu().numpy(), exp.astype(np.float32))
    for c in KATS["dynamic_quantize_linear"]["cases"]:  # coverage.rs:210-249
        y, s, z = ops.exec_dynamic_quantize_linear(_dev(torch, c["x"]))
        assert abs(float(s) - c["scale"]) < 1e-6 and float(z) == c["zero_point"] and y.cpu().numpy().tolist() == c["y"]
    for c in KATS["quantize_linear"]["cases"]:
        out = ops.exec_quantize_linear(_dev(torch, c["data"]), c["scale"], c["zero_point"])
        assert out.cpu().numpy().tolist() == [float(v) for v in c["expected"]]


@pytest.mark.parametrize("shape", SHAPES)
def test_matmul_integer_fast_path_bit_exact(oracle, torch_cuda, ops, shape):
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(m * 1000 + k * 10 + n)
    a = rng.integers(-128, 128, m * k).astype(np.float32)
    b = rng.integers(-128, 128, k * n).astype(np.float32)
    # carriers outside the i8 range and non-integers exercise the saturating, truncating `as i8` cast
    a[:: 7] = a[:: 7] * 3.5 + 0.75
    b[:: 5] = b[:: 5] * 2.25 - 0.5
    if a.size > 3:
        a[3] = np.nan
    exp, fast = oracle.exec_matmul_integer(a, b, 0.0, 0.0, m, k, n)
    assert fast
    out, path = ops.exec_matmul_integer(_dev(torch, a, (m, k)), _dev(torch, b, (k, n)))
    assert path == ops.PATH_FAST and np.array_equal(out.cpu().numpy(), exp)
    # the load-time prepack rounds before the cast (plan/build.rs:1367-1369): same result on integer weights
    bi = np.trunc(np.clip(b, -128, 127))
    pre = ops.PrepackedI8B(_dev(torch, bi, (k, n)))
    exp2, _ = oracle.exec_matmul_integer(a, bi, 0.0, 0.0, m, k, n)
    out2, _ = ops.exec_matmul_integer(_dev(torch, a, (m, k)), None, prepacked=pre)
    assert np.array_equal(out2.cpu().numpy(), exp2)
    pre.close()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("domain", ["u8_i8", "i8_u8", "u8_u8"])
def test_matmul_integer_asymmetric_is_integer_exact(oracle, torch_cuda, ops, shape, domain):
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(m * 77 + k * 3 + n + len(domain))
    alo, ahi = (0, 256) if domain.startswith("u8") else (-128, 128)
    blo, bhi = (0, 256) if domain.endswith("u8") else (-128, 128)
    a = rng.integers(alo, ahi, (m, k))
    b = rng.integers(blo, bhi, (k, n))
    a_zp = int(rng.integers(alo, ahi))
    b_zp = int(rng.integers(blo, bhi)) if domain != "u8_i8" else 0
    if a_zp == 0 and b_zp == 0:
        a_zp = 1 if alo == 0 else -1
    exact = (a.astype(np.int64) - a_zp) @ (b.astype(np.int64) - b_zp)
    out, path = ops.exec_matmul_integer(_dev(torch, a), _dev(torch, b), a_zp=float(a_zp), b_zp=float(b_zp))
    assert path == ops.PATH_FALLBACK_EXACT
    assert np.array_equal(out.cpu().numpy(), exact.astype(np.float32))
    if np.abs(a - a_zp).max() * np.abs(b - b_zp).max() * k < 2 ** 24:
        # every partial sum is exact in f32, so the reference's float fallback gives the same numbers
        exp, fast = oracle.exec_matmul_integer(a.ravel(), b.ravel(), float(a_zp), float(b_zp), m, k, n)
        assert not fast and np.array_equal(out.cpu().numpy(), exp)


def test_matmul_integer_f32_route_follows_the_float_fallback(oracle, torch_cuda, ops):
    torch = torch_cuda
    m, k, n = 7, 45, 19
    rng = np.random.default_rng(5)
    a = (rng.integers(0, 256, m * k) + rng.choice([0.0, 0.25, 0.5], m * k)).astype(np.float32)
    b = rng.integers(-128, 128, k * n).astype(np.float32)
    exp, fast = oracle.exec_matmul_integer(a, b, 3.0, 1.0, m, k, n)
    out, path = ops.exec_matmul_integer(_dev(torch, a, (m, k)), _dev(torch, b, (k, n)), a_zp=3.0, b_zp=1.0)
    assert not fast and path == ops.PATH_FALLBACK_F32
    assert np.array_equal(out.cpu().numpy(), exp)


@pytest.mark.parametrize("shape", SHAPES)
def test_qlinear_matmul_fast_path_bit_exact(oracle, torch_cuda, ops, shape):
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(m + 31 * k + 977 * n)
    a = rng.integers(-128, 128, m * k).astype(np.float32)
    b = rng.integers(-128, 128, k * n).astype(np.float32)
    for a_s, b_s, y_s, y_zp in ((0.05, 0.1, 0.25, 0.0), (0.02, 0.004, 0.5, -7.0), (1.0, 0.5, 64.0, 3.0)):
        exp, fast = oracle.exec_qlinear_matmul(a, a_s, 0.0, b, b_s, 0.0, y_s, y_zp, m, k, n)
        out, path = ops.exec_qlinear_matmul(_dev(torch, a, (m, k)), a_s, 0.0, _dev(torch, b, (k, n)), b_s, 0.0, y_s, y_zp)
        assert fast and path == ops.PATH_FAST
        assert np.array_equal(out.cpu().numpy(), exp)
        if ops.should_use_prepacked_i8_b(m, k, n):
            pre = ops.PrepackedI8B(_dev(torch, b, (k, n)))
            out2, _ = ops.exec_qlinear_matmul(_dev(torch, a, (m, k)), a_s, 0.0, None, b_s, 0.0, y_s, y_zp, prepacked=pre)
            assert np.array_equal(out2.cpu().numpy(), exp)
            pre.close()


@pytest.mark.parametrize("shape", SHAPES)
def test_qlinear_matmul_asymmetric(oracle, torch_cuda, ops, shape):
    """Asymmetric zero points: the exact sum, scaled once, against (a) the same expression in float64 and (b) the
    reference's float fallback, whose per-product rounding can move a value sitting on a rounding boundary by one."""
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(k * 13 + n)
    a = rng.integers(0, 256, (m, k))
    b = rng.integers(-128, 128, (k, n))
    a_zp, b_zp, a_s, b_s, y_s, y_zp = 128.0, 0.0, 0.02, 0.01, 0.8, 5.0
    out, path = ops.exec_qlinear_matmul(_dev(torch, a), a_s, a_zp, _dev(torch, b), b_s, b_zp, y_s, y_zp)
    assert path == ops.PATH_FALLBACK_EXACT
    got = out.cpu().numpy()
    acc = (a.astype(np.int64) - 128) @ b.astype(np.int64)
    v = (acc.astype(np.float64) * (float(np.float32(a_s)) * float(np.float32(b_s)))).astype(np.float32)
    t = v / np.float32(y_s) + np.float32(y_zp)
    want = np.clip(np.where(t >= 0, np.floor(t + np.float32(0.5)), -np.floor(-t + np.float32(0.5))), -128, 127)
    assert np.array_equal(got, want.astype(np.float32))
    exp, fast = oracle.exec_qlinear_matmul(a.ravel(), a_s, a_zp, b.ravel(), b_s, b_zp, y_s, y_zp, m, k, n)
    assert not fast
    assert np.abs(got - exp).max() <= 1.0
    assert (got != exp).mean() <= 0.02


def test_qlinear_prepacked_shape_mismatch_is_an_error(torch_cuda, ops):
    import yscv_amd

    torch = torch_cuda
    pre = ops.PrepackedI8B(torch.zeros(8, 32, device="cuda"))
    with pytest.raises(yscv_amd.YscvHipError) as ei:  # linear.rs:468-475
        yscv_amd.lib().exec_qlinear_matmul(torch.zeros(4, 16, device="cuda").data_ptr(), 1.0, 0.0, None, pre.handle, 1.0, 0.0,
                                           1.0, 0.0, 4, 16, 32, torch.zeros(4, 32, device="cuda").data_ptr(), None, None)
    assert ei.value.code == -1 and "shape mismatch" in ei.value.message
    pre.close()


def test_counters_follow_the_reference_gates(torch_cuda, ops):
    torch = torch_cuda
    a = torch.ones(4, 8, device="cuda")
    b = torch.ones(8, 16, device="cuda")
    ops.reset_quant_runtime_stats()
    ops.exec_qlinear_matmul(a, 1.0, 0.0, b, 1.0, 0.0, 1.0, 0.0)
    ops.exec_qlinear_matmul(a, 1.0, 0.0, b, 1.0, 0.0, 1.0, 0.0)
    ops.exec_qlinear_matmul(a, 1.0, 1.0, b, 1.0, 0.0, 1.0, 0.0)
    ops.exec_matmul_integer(a, b)
    ops.exec_matmul_integer(a, b, a_zp=2.0)
    ops.exec_matmul_integer(a, b, b_zp=2.0)
    s = ops.quant_runtime_stats()
    assert (s.qlinear_matmul_fast, s.qlinear_matmul_fallback, s.matmul_integer_fast, s.matmul_integer_fallback) == (2, 1, 1, 2)
    # int4: tiled layouts count as fast, the generic per-group kernel as fallback
    from yscv_amd import kernels as K

    rng = np.random.default_rng(0)
    for g, want in ((32, "int4_fast"), (16, "int4_fallback")):
        n, k = 16, 128
        w = K.PackedInt4Weight(rng.integers(0, 256, n * k // 2, dtype=np.uint8), np.ones(n * k // g, np.float32), g, n, k)
        before = ops.quant_runtime_stats()
        w.matmul(torch.ones(1, k, device="cuda"))
        after = ops.quant_runtime_stats()
        assert getattr(after, want) == getattr(before, want) + 1
        w.close()
    ops.reset_quant_runtime_stats()
    assert ops.quant_runtime_stats() == ops.QuantRuntimeStats()


def test_quantize_dequantize_linear(oracle, torch_cuda, ops):
    torch = torch_cuda
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(10_007) * 40).astype(np.float32)
    x[:8] = [0.5, 1.5, 2.5, -0.5, -1.5, np.nan, 1e9, -1e9]
    for scale, zp in ((1.0, 0.0), (0.37, 3.0), (0.011, -100.0)):
        exp = oracle.quantize_linear_f32_to_f32_i8(x, scale, zp)
        got = ops.exec_quantize_linear(_dev(torch, x), scale, zp).cpu().numpy()
        assert np.array_equal(got, exp, equal_nan=True)
        back = ops.exec_dequantize_linear(_dev(torch, np.nan_to_num(exp)), torch.tensor([scale], device="cuda"),
                                          torch.tensor([zp], device="cuda")).cpu().numpy()
        assert np.array_equal(back, oracle.dequantize_linear(np.nan_to_num(exp), scale, zp))
    # per-channel along axis 1 and along the last axis (misc.rs:136-170), written out with numpy broadcasting
    q = rng.integers(-128, 128, (3, 5, 4, 2)).astype(np.float32)
    for axis in (1, -1, 0):
        chan = q.shape[axis]
        s = (rng.random(chan) + 0.1).astype(np.float32)
        z = rng.integers(-5, 5, chan).astype(np.float32)
        shp = [1] * q.ndim
        shp[axis] = chan
        want = (q - z.reshape(shp)) * s.reshape(shp)
        got = ops.exec_dequantize_linear(_dev(torch, q), _dev(torch, s), _dev(torch, z), axis=axis).cpu().numpy()
        assert np.array_equal(got, want)
        got = ops.exec_dequantize_linear(_dev(torch, q), _dev(torch, s), None, axis=axis).cpu().numpy()
        assert np.array_equal(got, q * s.reshape(shp))
    import yscv_amd

    with pytest.raises(yscv_amd.YscvHipError):  # misc.rs:146-153: scale length must equal the axis extent
        ops.exec_dequantize_linear(_dev(torch, q), _dev(torch, np.ones(3, np.float32)), None, axis=1)


def test_dynamic_quantize_linear_matches_checker(oracle, torch_cuda, ops):
    torch = torch_cuda
    rng = np.random.default_rng(3)
    for x in (rng.standard_normal(4099).astype(np.float32) * 3, np.abs(rng.standard_normal(300)).astype(np.float32),
              np.zeros(17, np.float32), -np.abs(rng.standard_normal(64)).astype(np.float32)):
        ey, es, ez = oracle.dynamic_quantize_linear(x)
        y, s, z = ops.exec_dynamic_quantize_linear(_dev(torch, x))
        assert float(s) == float(es) and float(z) == float(ez)
        assert np.array_equal(y.cpu().numpy(), np.asarray(ey, np.float32))
    # DynamicQuantizeLinear -> MatMulInteger, the dynamic-quantisation pattern: integer-exact downstream
    x = (rng.standard_normal((6, 96)) * 2).astype(np.float32)
    w = rng.integers(-128, 128, (96, 48))
    y, s, z = ops.exec_dynamic_quantize_linear(_dev(torch, x))
    out, path = ops.exec_matmul_integer(y, _dev(torch, w), a_zp=float(z))
    assert path == ops.PATH_FALLBACK_EXACT
    exact = (y.cpu().numpy().astype(np.int64) - int(float(z))) @ w.astype(np.int64)
    assert np.array_equal(out.cpu().numpy(), exact.astype(np.float32))


@pytest.mark.parametrize("shape", [(5, 64, 48), (33, 200, 70), (130, 1024, 260), (512, 512, 1040)])
def test_qdq_matmul_equals_the_three_operators(oracle, torch_cuda, ops, shape):
    """The rewriter's QuantizeLinear -> QLinearMatMul -> DequantizeLinear triple (rewriter.rs:586-673) as one call:
    bit-identical to the oracle's three operators chained, and to this library's three entry points chained."""
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(m + k + n)
    x = (rng.standard_normal((m, k)) * 2.0).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    a_s = float(np.abs(x).max() / 127.0)
    b_s = float(np.abs(w).max() / 127.0)
    wq = np.clip(np.rint(w / np.float32(b_s)), -127, 127).astype(np.float32)
    y_s, y_zp = 0.37, 3.0
    aq = oracle.quantize_linear_f32_to_f32_i8(x.ravel(), a_s, 0.0)
    q, fast = oracle.exec_qlinear_matmul(aq, a_s, 0.0, wq.ravel(), b_s, 0.0, y_s, y_zp, m, k, n)
    want = oracle.dequantize_linear(q.ravel(), y_s, y_zp).reshape(m, n)
    assert fast
    pre = ops.PrepackedI8B(_dev(torch, wq))
    ops.reset_quant_runtime_stats()
    got = ops.exec_qdq_matmul(_dev(torch, x), a_s, pre, b_s, y_s, y_zp).cpu().numpy()
    assert ops.quant_runtime_stats().qlinear_matmul_fast == 1
    assert np.array_equal(got, want)
    a_dev = ops.exec_quantize_linear(_dev(torch, x), a_s, 0.0)
    q_dev, _ = ops.exec_qlinear_matmul(a_dev, a_s, 0.0, None, b_s, 0.0, y_s, y_zp, prepacked=pre)
    chained = ops.exec_dequantize_linear(q_dev, torch.tensor([y_s], device="cuda"), torch.tensor([y_zp], device="cuda"))
    assert np.array_equal(got, chained.cpu().numpy())
    pre.close()


# ---- MatMulNBits and the int4 Gemm ------------------------------------------------------------------------------
@pytest.mark.parametrize("m,k,n,g,with_zp,sdt", [(1, 4096, 512, 32, False, "f32"), (5, 256, 48, 32, True, "f16"),
                                                   (16, 1024, 300, 128, True, "f16"), (40, 512, 272, 64, False, "f32"),
                                                   (3, 96, 20, 16, True, "f32"), (200, 1024, 256, 128, True, "f16")])
def test_matmul_nbits_operator(oracle, torch_cuda, ops, m, k, n, g, with_zp, sdt):
    """MatMulNBits = A x dequant(B)^T + bias on the node's initialisers (uint4 nibbles, per-block scales, optional
    packed uint4 zero points), against the checker's dequantise-then-dot definition, within the int4 float bar."""
    from gpu_util import int4_tolerances, pack_zero_points

    torch = torch_cuda
    rng = np.random.default_rng(m * 1000 + k + n)
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16 if sdt == "f16" else np.float32)
    zps = pack_zero_points(rng.integers(6, 11, (n, k // g))) if with_zp else None
    w = ops.MatMulNBitsWeight(b, scales, zps, K=k, N=n, bits=4, block_size=g)
    x = rng.standard_normal((m, k)).astype(np.float32)
    ref = oracle.matmul_nbits(b, scales.astype(np.float32), zps, x, m, n, k, g)
    bias = rng.standard_normal(n).astype(np.float32)
    y = ops.exec_matmul_nbits(_dev(torch, x), w)
    assert tuple(y.shape) == (m, n) and y.dtype == torch.float32
    int4_tolerances(y.cpu().numpy(), ref, k, x)
    yb = ops.exec_matmul_nbits(_dev(torch, x), w, bias=_dev(torch, bias))
    assert np.array_equal(yb.cpu().numpy(), y.cpu().numpy() + bias[None, :])  # one f32 add on top of the product
    # rank-3 activations, 16-bit types: [2][m][k] -> [2][m][n], rounded once after the bias
    x3 = torch.from_numpy(np.stack([x, -x])).bfloat16().cuda()
    y3 = ops.exec_matmul_nbits(x3, w, bias=_dev(torch, bias))
    assert tuple(y3.shape) == (2, m, n) and y3.dtype == torch.bfloat16
    xs = x3.float().cpu().numpy().reshape(2 * m, k)
    ref3 = oracle.matmul_nbits(b, scales.astype(np.float32), zps, xs, 2 * m, n, k, g) + bias[None, :]
    from gpu_util import bf16_round
    got3 = y3.float().cpu().numpy().reshape(2 * m, n)
    assert np.abs(got3 - bf16_round(ref3)).max() <= np.abs(ref3).max() * 2.0 ** -7
    w.close()


def test_matmul_nbits_attribute_errors(torch_cuda, ops):
    import yscv_amd

    torch = torch_cuda
    rng = np.random.default_rng(3)
    k, n, g = 128, 16, 32
    w = ops.MatMulNBitsWeight(rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.01, 0.02, n * (k // g)).astype(np.float32),
                              None, K=k, N=n, block_size=g)
    x = torch.zeros(2, k, device="cuda")
    for kw, frag in [(dict(K=256), "attributes K=256"), (dict(N=8), "N=8"), (dict(block_size=64), "block_size=64")]:
        with pytest.raises(yscv_amd.YscvHipError, match=frag) as ei:
            ops.exec_matmul_nbits(x, w, **kw)
        assert ei.value.code == -1
    with pytest.raises(yscv_amd.YscvHipError, match="only 4 is supported") as ei:
        ops.exec_matmul_nbits(x, w, bits=8)
    assert ei.value.code == -4
    with pytest.raises(ValueError):
        ops.MatMulNBitsWeight(np.zeros(8, np.uint8), np.zeros(1, np.float32), None, K=16, N=1, bits=2, block_size=16)
    w.close()


@pytest.mark.parametrize("m,k,n,g,nk", [(1, 256, 64, 32, True), (7, 512, 40, 64, False), (32, 1024, 128, 128, True)])
def test_gemm_through_the_int4_branch(oracle, torch_cuda, ops, m, k, n, g, nk):
    """Gemm(alpha, beta, C) whose B the int4 packing pass quantised (packed_int4.rs:155-168): the weight is packed on the
    device from the f32 initialiser in either layout, the product equals the int4 matmul of the same weight, and alpha /
    beta / C follow exec_gemm's order of operations (linear.rs:54-66) bit for bit."""
    from gpu_util import int4_tolerances
    from yscv_amd import kernels as K

    torch = torch_cuda
    rng = np.random.default_rng(m + k + n)
    w_nk = rng.standard_normal((n, k)).astype(np.float32)
    wt = _dev(torch, w_nk if nk else np.ascontiguousarray(w_nk.T))
    w = K.PackedInt4Weight.from_f32(wt, g, transposed_nk=nk)
    packed, scales = oracle.pack_int4_symmetric_per_group(w_nk.ravel(), n, k, g)
    x = rng.standard_normal((m, k)).astype(np.float32)
    ref = oracle.packed_int4_gemm_scalar(packed, scales, x, m, n, k, g).reshape(m, n)
    a = _dev(torch, x)
    prod = ops.exec_gemm_int4(a, w)
    int4_tolerances(prod.cpu().numpy(), ref, k, x)
    assert torch.equal(prod, w.matmul(a))
    p = prod.cpu().numpy()
    c_row = rng.standard_normal(n).astype(np.float32)
    c_full = rng.standard_normal((m, n)).astype(np.float32)
    for alpha, beta, c in [(1.0, 1.0, c_row), (0.5, 1.0, c_row), (1.0, 2.5, c_full), (-1.25, 0.3, c_full), (3.0, 1.0, None),
                           (1.0 + 1e-8, 1.0, c_row)]:
        got = ops.exec_gemm_int4(a, w, c=None if c is None else _dev(torch, c), alpha=alpha, beta=beta).cpu().numpy()
        want = p.copy()
        if abs(np.float32(alpha) - np.float32(1.0)) > np.finfo(np.float32).eps:
            want = want * np.float32(alpha)
        if c is not None:
            add = c * np.float32(beta) if abs(np.float32(beta) - np.float32(1.0)) > np.finfo(np.float32).eps else c
            want = want + (add[None, :] if add.ndim == 1 else add)
        assert np.array_equal(got, want.astype(np.float32)), (alpha, beta)
    with pytest.raises(ValueError):
        ops.exec_gemm_int4(a, w, c=_dev(torch, np.zeros(n + 1, np.float32)))


@pytest.mark.parametrize("shape", [(1, 64, 16), (5, 200, 70), (33, 512, 128), (64, 4096, 256), (130, 1024, 48)])
def test_dql_fused_into_matmul_integer(oracle, torch_cuda, ops, shape):
    """DynamicQuantizeLinear -> MatMulInteger as one call: bit-identical to the two operators chained, and equal to the
    checker's DynamicQuantizeLinear followed by the exact integer product."""
    torch = torch_cuda
    m, k, n = shape
    rng = np.random.default_rng(m * 7 + k + n)
    x = (rng.standard_normal((m, k)) * 3.0 + 0.7).astype(np.float32)
    b = rng.integers(-127, 128, (k, n)).astype(np.float32)
    pre = ops.PrepackedI8B(_dev(torch, b))
    out, ys, yz = ops.exec_dql_matmul_integer(_dev(torch, x), pre)
    y, s2, z2 = ops.exec_dynamic_quantize_linear(_dev(torch, x))
    chained, _ = ops.exec_matmul_integer(y, None, a_zp=float(z2.item()), b_zp=0.0, prepacked=pre)
    assert torch.equal(out, chained) and torch.equal(ys, s2) and torch.equal(yz, z2)
    yq, sc, zp = oracle.dynamic_quantize_linear(x.ravel())
    assert float(ys.item()) == np.float32(sc) and float(yz.item()) == float(zp)
    want = (yq.reshape(m, k).astype(np.int64) - int(zp)) @ b.astype(np.int64)
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))
    # constant input: range 0 .. c, every value quantises to 255 or to 0
    xc = np.full((4, k), 2.5, np.float32)
    out, ys, yz = ops.exec_dql_matmul_integer(_dev(torch, xc), pre)
    yq, sc, zp = oracle.dynamic_quantize_linear(xc.ravel())
    want = (yq.reshape(4, k).astype(np.int64) - int(zp)) @ b.astype(np.int64)
    assert np.array_equal(out.cpu().numpy(), want.astype(np.float32))

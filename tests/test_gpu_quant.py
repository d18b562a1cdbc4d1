"""GPU parity (bit-exact) of the elementwise quantisation kernels, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import torch

    assert torch.cuda.is_available()
    from yscv_amd import kernels

    return kernels


def test_quantize_linear_goldens_and_random(oracle, K):
    data = np.array([-1000.0, -1.5, -0.5, 0.49, 0.5, 1.5, 1000.0], np.float32)
    out = np.zeros(7, np.int8)
    K.quantize_linear_f32_to_i8_dispatch(data, 1.0, 0.0, out)  # quantize.rs:826-832
    assert out.tolist() == [-128, -2, 0, 0, 0, 2, 127]
    # quantize.rs:803-814 inputs
    i = np.arange(257, dtype=np.float32)
    data = (np.sin(i * np.float32(0.37)) * 40.0 + (np.arange(257) % 7) * np.float32(0.11)).astype(np.float32)
    out = np.zeros(257, np.int8)
    K.quantize_linear_f32_to_i8_dispatch(data, 3.25, -2.0, out)
    assert np.array_equal(out, oracle.quantize_linear_f32_to_i8(data, 3.25, -2.0))
    rng = np.random.default_rng(41)
    v = np.concatenate([rng.uniform(-60, 60, 100000), [np.nan, np.inf, -np.inf, 0.0, -0.0]]).astype(np.float32)
    for scale, zp in [(0.3, -2.0), (0.007, 5.0), (1.0, 0.5)]:
        out = np.zeros(v.size, np.int8)
        K.quantize_linear_f32_to_i8_dispatch(v, scale, zp, out)
        assert np.array_equal(out, oracle.quantize_linear_f32_to_i8(v, scale, zp))


def test_requant_goldens_and_random(oracle, K):
    out = np.zeros(8, np.int8)
    K.requant_i32_row_to_i8_dispatch([1, -1, 3, -3, 5, -5, 7, -7], None, 0.5, 0.0, False, out, 8)  # int8_requant.rs:1217-1226
    assert out.tolist() == [0, 0, 2, -2, 2, -2, 4, -4]
    acc = np.array([1_000_000] * 8 + [-1_000_000] * 8, np.int32)
    out = np.zeros(16, np.int8)
    K.requant_i32_row_to_i8_dispatch(acc, None, 0.001, 0.0, False, out, 16)  # :1197-1214
    assert out.tolist() == [127] * 8 + [-128] * 8
    out = np.ones(24, np.int8)
    K.requant_i32_row_to_i8_dispatch(np.full(24, -100, np.int32), None, 1.0, 0.0, True, out, 8)  # :1187-1194
    assert (out == 0).all()
    rng = np.random.default_rng(42)
    for c in (4, 5, 16, 17, 24, 40, 72):  # int8_requant.rs:1045-1075
        pixels = 37
        acc = rng.integers(-2**20, 2**20, pixels * c, dtype=np.int32)
        acc[:3] = [2**31 - 1, -2**31, 0]
        corr = rng.integers(-2**16, 2**16, c, dtype=np.int32)
        comp = rng.uniform(1e-5, 1e-3, c).astype(np.float32)
        out = np.zeros(acc.size, np.int8)
        K.requant_i8_per_channel_dispatch(acc, corr, comp, -3.0, out, c)
        assert np.array_equal(out, oracle.requant_i8_per_channel(acc, corr, comp, -3.0, c))
        out2 = np.zeros(acc.size, np.int8)
        K.requant_i32_row_to_i8_dispatch(acc, corr, 0.00037, 2.0, True, out2, c)
        assert np.array_equal(out2, oracle.requant_i32_row_to_i8(acc, corr, 0.00037, 2.0, True, c))
    # exact ties under both signs: composite 0.5
    acc = np.arange(-41, 42, dtype=np.int32)
    out = np.zeros(acc.size, np.int8)
    K.requant_i32_row_to_i8_dispatch(acc, None, 0.5, 0.0, False, out, 1)
    assert np.array_equal(out, oracle.requant_i32_row_to_i8(acc, None, 0.5, 0.0, False, 1))


def test_dynamic_quantize_linear(oracle, K):
    y, s, z = K.dynamic_quantize_linear(np.array([-2.0, -1.0, 0.0, 1.0], np.float32))  # coverage.rs:210-249
    assert abs(s - 3.0 / 255.0) < 1e-6 and z == 170.0 and y.tolist() == [0, 85, 170, 255]
    rng = np.random.default_rng(43)
    cases = [rng.standard_normal(5000).astype(np.float32) * 3, np.array([2.0, 4.0], np.float32),
             np.zeros(3, np.float32), rng.uniform(1, 2, (512, 4096)).astype(np.float32),
             np.array([-5.0], np.float32), np.concatenate([rng.standard_normal(100), [np.nan]]).astype(np.float32)]
    for x in cases:
        y, s, z = K.dynamic_quantize_linear(x)
        ye, se, ze = oracle.dynamic_quantize_linear(x)
        assert s == se and z == ze
        # the reference keeps NaN in its f32 carrier; a uint8 output stores what `NaN as u8` gives: 0
        assert np.array_equal(y.astype(np.float32), np.nan_to_num(ye, nan=0.0))
    y, s, z = K.dynamic_quantize_linear(np.zeros(0, np.float32))
    assert y.size == 0 and s == 1.0 and z == 0.0


def test_kv_cache_int8_rows_bit_exact(oracle, K):
    """KvCache I8 append / read (kv_cache.rs:45-79): per-row scale abs_max / 127, f32::round, clamp [-127, 127]."""
    import torch

    rng = np.random.default_rng(21)
    for rows, kv_dim in ((1, 1024), (7, 1024), (33, 96), (5, 1)):
        src = (rng.standard_normal((rows, kv_dim)) * rng.uniform(0.01, 30, (rows, 1))).astype(np.float32)
        src[0, : min(3, kv_dim)] = [0.5, -0.5, 1.5][: min(3, kv_dim)]
        if rows > 2:
            src[1] = 0.0          # abs_max <= EPSILON: scale 1
            src[2, 0] = np.nan    # NaN does not enter the abs-max and quantises to 0
        ed, es = oracle.kv_i8_quantize_rows(src, rows, kv_dim)
        d, s = K.kv_i8_quantize_rows(torch.from_numpy(src).cuda())
        assert np.array_equal(s.cpu().numpy(), es)
        assert np.array_equal(d.cpu().numpy().ravel(), ed)
        back = K.kv_i8_dequantize_rows(d, s).cpu().numpy()
        assert np.array_equal(back, ed.reshape(rows, kv_dim).astype(np.float32) * es[:, None])
    # ties: v * inv exactly on .5 rounds away from zero
    src = np.array([[127.0, 0.5, -0.5, 1.5, -2.5, 63.5]], np.float32)
    d, s = K.kv_i8_quantize_rows(torch.from_numpy(src).cuda())
    assert float(s[0]) == 1.0 and d.cpu().numpy().ravel().tolist() == [127, 1, -1, 2, -3, 64]


def test_measured_peaks_are_plausible(K):
    """yscv_hip_measure_peaks: a sustained figure can neither exceed the published peak nor sit far below what this
    class of GPU reaches (the probes are registers-only MFMA loops and a 1 GiB read stream)."""
    import ctypes as C

    from yscv_amd import capi

    r, f, i = C.c_double(), C.c_double(), C.c_double()
    capi.lib().measure_peaks(C.byref(r), C.byref(f), C.byref(i))
    assert 3000.0 < r.value <= 8000.0, r.value
    assert 1000.0 < f.value <= 2500.0, f.value
    assert 2000.0 < i.value <= 5000.0, i.value
    # yscv_hip_measure_fill: what one CU takes in through LDS-direct loads, from L2 and from behind it
    l2, far = C.c_double(), C.c_double()
    capi.lib().measure_fill(C.byref(l2), C.byref(far))
    assert 20.0 < far.value <= l2.value * 1.05 and l2.value < 270.0, (l2.value, far.value)  # 64 B per clock = 154 GB/s at 2.4 GHz


def test_quantize_f32_to_int4_bit_exact(oracle, K):
    """quantize_f32_to_int4 (ops/quantize.rs:69-95): ties-even rounding, clamp after the zero point, low nibble first,
    odd tails, the epsilon-scale rule, NaN / inf -- host-pointer form and device-pointer form."""
    import ctypes as C

    import torch

    from yscv_amd import lib

    rng = np.random.default_rng(43)
    base = np.concatenate([rng.uniform(-6, 6, 100001), np.arange(-9, 9) + 0.5, [np.nan, np.inf, -np.inf, 0.0, -0.0, 3e38, -3e38]])
    for scale, zp in [(1.0, 0), (0.5, 3), (0.37, -4), (-0.8, 1), (1e-8, -2), (0.0, 5), (1e-30, 0)]:
        v = base.astype(np.float32)
        want = oracle.quantize_f32_to_int4(v, scale, zp)
        got = np.full((v.size + 1) // 2, 0xEE, np.uint8)
        K.quantize_f32_to_int4(v, scale, zp, got)
        assert np.array_equal(got, want), (scale, zp)
        x = torch.from_numpy(v).cuda()
        out = torch.full(((v.size + 1) // 2 + 1,), 0xEE, dtype=torch.uint8, device="cuda")
        lib().quantize_f32_to_int4_dev(C.c_void_p(x.data_ptr()), C.c_size_t(v.size), C.c_float(scale), C.c_int8(zp),
                                       C.c_void_p(out.data_ptr()), None)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy()[:-1], want) and int(out[-1]) == 0xEE
    # round trip through dequantize_int4_to_f32 stays within one step (quantize.rs:739-757)
    original = (np.arange(-8, 8) * 0.5).astype(np.float32)
    packed = np.zeros(8, np.uint8)
    K.quantize_f32_to_int4(original, 0.5, 0, packed)
    rec = np.zeros(16, np.float32)
    K.dequantize_int4_to_f32(packed, 0.5, 0, rec)
    assert np.abs(rec - original).max() <= 0.5 + 1e-6

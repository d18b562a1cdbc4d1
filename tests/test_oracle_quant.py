"""Pins the quantize / requantize / DynamicQuantizeLinear part of the CPU checker against the
reference's unit-test vectors (ops/quantize.rs:789-832, ops/int8_requant.rs:1185-1226,
crates/yscv-onnx/src/tests/coverage.rs:90-249, runner/kv_cache.rs).  No GPU."""
import numpy as np


def test_quantize_linear_goldens(oracle):
    data = [-1000.0, -1.5, -0.5, 0.49, 0.5, 1.5, 1000.0]
    # quantize.rs:817-832
    assert oracle.quantize_linear_f32_to_i8(data, 1.0, 0.0).tolist() == [-128, -2, 0, 0, 0, 2, 127]
    assert oracle.quantize_linear_f32_to_f32_i8(data, 1.0, 0.0).tolist() == [-128.0, -2.0, 0.0, 0.0, 0.0, 2.0, 127.0]
    # coverage.rs:90-126
    assert oracle.quantize_linear_f32_to_f32_i8([-1.5, -0.5, 0.0, 0.5, 1.5], 0.5, 0.0).tolist() == [-3.0, -1.0, 0.0, 1.0, 3.0]
    assert oracle.quantize_linear_f32_to_f32_i8([100.0, 0.0, -100.0], 0.5, 10.0).tolist() == [127.0, 10.0, -128.0]
    # NaN -> clamp keeps NaN -> `as i8` gives 0
    assert oracle.quantize_linear_f32_to_i8([np.nan], 1.0, 0.0).tolist() == [0]


def test_quantize_linear_divides(oracle):
    # v / scale, not v * (1/scale): 3 candidates where the two differ in f32
    rng = np.random.default_rng(9)
    v = rng.uniform(-50, 50, 20000).astype(np.float32)
    scale = np.float32(0.3)
    exp = np.clip(np.rint(v / scale + np.float32(-2.0)), -128, 127).astype(np.int8)
    assert np.array_equal(oracle.quantize_linear_f32_to_i8(v, scale, -2.0), exp)


def test_requant_goldens(oracle):
    # int8_requant.rs:1217-1226 ties to even
    got = oracle.requant_i32_row_to_i8([1, -1, 3, -3, 5, -5, 7, -7], None, 0.5, 0.0, False, 8)
    assert got.tolist() == [0, 0, 2, -2, 2, -2, 4, -4]
    # :1197-1214 saturation
    acc = [1_000_000] * 8 + [-1_000_000] * 8
    got = oracle.requant_i32_row_to_i8(acc, None, 0.001, 0.0, False, 16)
    assert got.tolist() == [127] * 8 + [-128] * 8
    # :1187-1194 relu
    assert (oracle.requant_i32_row_to_i8([-100] * 24, None, 1.0, 0.0, True, 8) == 0).all()
    # bias is added with wrapping arithmetic before the float conversion (:155-158)
    got = oracle.requant_i32_row_to_i8([2**31 - 1, 5], [1, -5], 1.0, 0.0, False, 2)
    assert got.tolist() == [-128, 0]


def test_per_channel_equals_per_tensor_when_uniform(oracle):
    rng = np.random.default_rng(4)
    c, pixels = 17, 9
    acc = rng.integers(-50000, 50000, pixels * c, dtype=np.int32)
    corr = rng.integers(-1000, 1000, c, dtype=np.int32)
    a = oracle.requant_i8_per_channel(acc, corr, np.full(c, 0.0021, np.float32), 3.0, c)
    b = oracle.requant_i32_row_to_i8(acc, corr, 0.0021, 3.0, False, c)
    assert np.array_equal(a, b)
    g = oracle.requant_general(acc, c, corr, np.full(c, 0.0021, np.float32), 3.0, oracle.ROUND_TIES_EVEN, -128, 127)
    assert np.array_equal(g, a.astype(np.int32))


def test_requant_general_discriminating_kats(oracle):
    # composite 1/4096 (exact), y_zp 128, clamp [0,255]; values chosen so that a wrong rounding
    # rule, a fused multiply-add, or adding zp after rounding each change an output.
    acc = [4096, -2048, -6144, 2048, 600_000, -600_000]
    away = oracle.requant_general(acc, 1, None, 1.0 / 4096, 128.0, oracle.ROUND_HALF_AWAY, 0, 255)
    even = oracle.requant_general(acc, 1, None, 1.0 / 4096, 128.0, oracle.ROUND_TIES_EVEN, 0, 255)
    assert away.tolist() == [129, 128, 127, 129, 255, 0]
    assert even.tolist() == [129, 128, 126, 128, 255, 0]


def test_dynamic_quantize_linear_reference_example(oracle):
    # coverage.rs:210-249
    y, s, z = oracle.dynamic_quantize_linear([-2.0, -1.0, 0.0, 1.0])
    assert abs(s - 3.0 / 255.0) < 1e-6 and z == 170.0
    assert y.tolist() == [0.0, 85.0, 170.0, 255.0]
    # range is forced to include zero (misc.rs:260-261); constant input -> scale 1 (:262-263)
    y, s, z = oracle.dynamic_quantize_linear([2.0, 4.0])
    assert s == np.float32(4.0 / 255.0) and z == 0.0
    y, s, z = oracle.dynamic_quantize_linear([0.0, 0.0, 0.0])
    assert s == 1.0 and z == 0.0 and (y == 0).all()
    # closed form on random data
    rng = np.random.default_rng(8)
    x = rng.standard_normal(5000).astype(np.float32) * 3
    y, s, z = oracle.dynamic_quantize_linear(x)
    mn, mx = min(x.min(), np.float32(0)), max(x.max(), np.float32(0))
    s_exp = (mx - mn) / np.float32(255)
    t = np.float32(0) - mn / s_exp
    z_exp = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), 0, 255)
    v = x / s_exp + z_exp
    y_exp = np.clip(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)), 0, 255)
    assert s == s_exp and z == z_exp and np.array_equal(y, y_exp.astype(np.float32))
    assert y.min() >= 0 and y.max() <= 255  # gather_scatter.rs:249-264


def test_dequantize_linear(oracle):
    # coverage.rs:128-160 form: (q - zp) * s
    assert oracle.dequantize_linear([0, 10, 20], 0.5, 10.0).tolist() == [-5.0, 0.0, 5.0]


def test_kv_int8_rows(oracle):
    # kv_cache.rs:45-61: scale = absmax/127, q = round(v/scale) clamped to +-127, error <= scale
    rng = np.random.default_rng(12)
    rows, dim = 5, 64
    src = rng.standard_normal((rows, dim)).astype(np.float32)
    src[3] = 0
    data, scales = oracle.kv_i8_quantize_rows(src, rows, dim)
    assert scales[3] == 1.0 and (data.reshape(rows, dim)[3] == 0).all()
    assert np.array_equal(scales[[0, 1, 2, 4]], (np.abs(src).max(1) / np.float32(127))[[0, 1, 2, 4]])
    rec = data.reshape(rows, dim).astype(np.float32) * scales[:, None]
    assert (np.abs(rec - src) <= scales[:, None]).all()
    assert np.abs(data).max() == 127


def test_argmax_takes_last_maximum(oracle):
    # Iterator::max_by returns the last of equal maxima (apps/llm-bench/src/main.rs:538-543)
    assert oracle.argmax_last([1.0, 5.0, 2.0, 5.0, 0.0]) == 3
    assert oracle.argmax_last([7.0]) == 0
    assert oracle.argmax_last([3.0, 2.0, 1.0]) == 0

"""Known-answer vectors of the reference's own unit tests (tests/golden/reference_kats.json), applied to the
CPU checker (no GPU needed) and, marked gpu, to the HIP library through the C ABI."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))


def _qlinear_inputs():
    q = KATS["qlinear_matmul"]
    m, k, n = q["m"], q["k"], q["n"]
    a = np.array([v - 16 for v in range(m * k)], np.int8)
    b = np.array([(7 * v) % 31 - 15 for v in range(k * n)], np.int8)
    comp = np.float32(np.float32(q["a_scale"]) * np.float32(q["b_scale"])) / np.float32(q["y_scale"])
    acc = a.reshape(m, k).astype(np.int64) @ b.reshape(k, n).astype(np.int64)
    # f32::round = half away from zero, written out by hand (not through the checker)
    v = acc.astype(np.float32) * comp
    r = np.where(v >= 0, np.floor(v + np.float32(0.5)), -np.floor(-v + np.float32(0.5)))
    return a, b, comp, np.clip(r, -128, 127).astype(np.int32)


# ---- CPU checker ------------------------------------------------------------------------------------
def test_oracle_nibbles_and_dequant(oracle):
    for c in KATS["nibble_decode"]["cases"]:
        out = oracle.dequantize_int4_to_f32(np.array([c["byte"]], np.uint8), 1.0, 0)
        assert out.tolist() == [float(c["lo"]), float(c["hi"])]
    for c in KATS["dequantize_int4"]["cases"]:
        out = oracle.dequantize_int4_to_f32(np.array(c["packed"], np.uint8), c["scale"], c["zero_point"])
        assert np.abs(out - np.array(c["expected"], np.float32)).max() <= c.get("tol", 0.0)
    for c in KATS["quantize_f32_to_int4"]["cases"]:
        packed = oracle.quantize_f32_to_int4(c["data"], c["scale"], c["zero_point"])
        assert packed.size == (len(c["data"]) + 1) // 2
        assert oracle.dequantize_int4_to_f32(packed, 1.0, 0).tolist() == [float(v) for v in c["expected_nibbles"]]


def test_oracle_matmuls(oracle):
    for c in KATS["int4_gemv_hand"]["cases"]:
        y = oracle.packed_int4_gemv_scalar(np.array(c["packed"], np.uint8), c["scales"], c["x"], c["m_w"], c["k"], c["group_size"])
        assert y.tolist() == c["expected"]
    for c in KATS["int8_matmul"]["cases"]:
        a = np.array(c["a"], np.int8) if "a" in c else np.full(c["m"] * c["k"], c["a_fill"], np.int8)
        b = np.array(c["b"], np.int8) if "b" in c else np.full(c["k"] * c["n"], c["b_fill"], np.int8)
        assert oracle.int8_matmul_scalar(a, b, c["m"], c["k"], c["n"]).ravel().tolist() == c["expected"]
    for c in KATS["matmul_integer"]["cases"]:
        out, _ = oracle.exec_matmul_integer(c["a"], c["b"], float(c["a_zp"]), 0.0, c["m"], c["k"], c["n"])
        assert out.ravel().tolist() == [float(v) for v in c["expected"]]
    a, b, _, exp = _qlinear_inputs()
    q = KATS["qlinear_matmul"]
    out, fast = oracle.exec_qlinear_matmul(a.astype(np.float32), q["a_scale"], 0.0, b.astype(np.float32), q["b_scale"], 0.0,
                                           q["y_scale"], 0.0, q["m"], q["k"], q["n"])
    assert fast and np.array_equal(out.ravel().astype(np.int32), exp.ravel())


def test_oracle_quantizers(oracle):
    for c in KATS["quantize_linear"]["cases"]:
        assert oracle.quantize_linear_f32_to_i8(c["data"], c["scale"], c["zero_point"]).tolist() == c["expected"]
    for c in KATS["requant_ties_even"]["cases"]:
        assert oracle.requant_i32_row_to_i8(c["acc"], None, c["composite"], c["y_zp"], False, c["c"]).tolist() == c["expected"]
    r = KATS["requant_rounding_modes"]
    for mode, key in ((oracle.ROUND_HALF_AWAY, "expected_half_away"), (oracle.ROUND_TIES_EVEN, "expected_ties_even")):
        got = oracle.requant_general(r["acc"], 1, None, r["composite"], r["y_zp"], mode, r["lo"], r["hi"])
        assert got.tolist() == r[key]
    for c in KATS["dynamic_quantize_linear"]["cases"]:
        y, s, z = oracle.dynamic_quantize_linear(c["x"])
        assert abs(s - c["scale"]) < 1e-6 and z == c["zero_point"] and y.tolist() == [float(v) for v in c["y"]]
    for bits, val in KATS["fp16_bf16_bits"]["fp16"].items():
        assert oracle.fp16_bits_to_f32(np.array([int(bits)], np.uint16))[0] == val
    for bits, val in KATS["fp16_bf16_bits"]["bf16"].items():
        assert oracle.bf16_bits_to_f32(np.array([int(bits)], np.uint16))[0] == val


# ---- HIP library, same vectors ------------------------------------------------------------------------
@pytest.mark.gpu
def test_hip_library_matches_reference_kats():
    import torch

    from yscv_amd import kernels as K

    assert torch.cuda.is_available()
    for c in KATS["nibble_decode"]["cases"]:
        out = np.empty(2, np.float32)
        K.dequantize_int4_to_f32(np.array([c["byte"]], np.uint8), 1.0, 0, out)
        assert out.tolist() == [float(c["lo"]), float(c["hi"])]
    for c in KATS["dequantize_int4"]["cases"]:
        out = np.empty(2 * len(c["packed"]), np.float32)
        K.dequantize_int4_to_f32(np.array(c["packed"], np.uint8), c["scale"], c["zero_point"], out)
        assert np.abs(out - np.array(c["expected"], np.float32)).max() <= c.get("tol", 0.0)
    for c in KATS["quantize_f32_to_int4"]["cases"]:
        packed = np.full((len(c["data"]) + 1) // 2, 0xEE, np.uint8)
        K.quantize_f32_to_int4(np.array(c["data"], np.float32), c["scale"], c["zero_point"], packed)
        out = np.empty(2 * packed.size, np.float32)
        K.dequantize_int4_to_f32(packed, 1.0, 0, out)
        assert out.tolist() == [float(v) for v in c["expected_nibbles"]]
    for c in KATS["int4_gemv_hand"]["cases"]:
        out = np.zeros(c["m_w"], np.float32)
        K.packed_int4_gemv_dispatch(np.array(c["packed"], np.uint8), np.array(c["scales"], np.float32),
                                    np.array(c["x"], np.float32), out, c["m_w"], c["k"], c["group_size"])
        assert out.tolist() == c["expected"]
    for c in KATS["int8_matmul"]["cases"]:
        a = np.array(c["a"], np.int8) if "a" in c else np.full(c["m"] * c["k"], c["a_fill"], np.int8)
        b = np.array(c["b"], np.int8) if "b" in c else np.full(c["k"] * c["n"], c["b_fill"], np.int8)
        out = np.zeros(c["m"] * c["n"], np.int32)
        K.int8_matmul_dispatch(a, b, c["m"], c["k"], c["n"], out)
        assert out.tolist() == c["expected"]
    for c in KATS["matmul_integer"]["cases"]:
        pb = K.pack_i8_b_for_matmul(np.array(c["b"], np.int8).reshape(c["k"], c["n"]), c["k"], c["n"])
        a = torch.tensor(c["a"], dtype=torch.uint8).reshape(c["m"], c["k"]).cuda()
        assert pb.matmul(a, a_zp=c["a_zp"]).cpu().numpy().ravel().tolist() == c["expected"]
    a, b, comp, exp = _qlinear_inputs()
    q = KATS["qlinear_matmul"]
    pb = K.pack_i8_b_for_matmul(b.reshape(q["k"], q["n"]), q["k"], q["n"])
    got = pb.matmul_requant(torch.from_numpy(a.reshape(q["m"], q["k"])).cuda(), 0, float(comp), 0.0, K.ROUND_HALF_AWAY, -128, 127)
    assert np.array_equal(got.cpu().numpy().astype(np.int32), exp)
    for c in KATS["quantize_linear"]["cases"]:
        out = np.zeros(len(c["data"]), np.int8)
        K.quantize_linear_f32_to_i8_dispatch(np.array(c["data"], np.float32), c["scale"], c["zero_point"], out)
        assert out.tolist() == c["expected"]
    for c in KATS["requant_ties_even"]["cases"]:
        out = np.zeros(len(c["acc"]), np.int8)
        K.requant_i32_row_to_i8_dispatch(np.array(c["acc"], np.int32), None, c["composite"], c["y_zp"], False, out, c["c"])
        assert out.tolist() == c["expected"]
    for c in KATS["dynamic_quantize_linear"]["cases"]:
        y, s, z = K.dynamic_quantize_linear(np.array(c["x"], np.float32))
        assert abs(s - c["scale"]) < 1e-6 and z == c["zero_point"] and y.tolist() == c["y"]

"""CPU-side checks of the operator layer: the gates and counters need no device."""
import itertools
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_prepack_gates_match_the_checker(oracle):
    from yscv_amd import onnx_ops as ops

    dims = [0, 1, 3, 4, 15, 16, 31, 32, 48, 63, 64, 65, 511, 512, 1023, 1024, 1040, 4096]
    for m, k, n in itertools.product(dims, dims, dims):
        assert ops.should_use_prepacked_i8_b(m, k, n) == oracle.should_use_prepacked_i8_b(m, k, n), (m, k, n)
    for k, n in itertools.product(dims, dims):
        assert ops.should_prepack_i8_b(k, n) == oracle.should_prepack_i8_b(k, n), (k, n)
    # layout.rs:6-11 spelled out on the corner cases
    assert ops.should_use_prepacked_i8_b(4, 4, 32) and not ops.should_use_prepacked_i8_b(3, 4, 32)
    assert ops.should_use_prepacked_i8_b(64, 512, 1024) and not ops.should_use_prepacked_i8_b(65, 512, 1025)
    assert not ops.should_use_prepacked_i8_b(4, 4, 40) and ops.should_use_prepacked_i8_b(1, 512, 1025)


def test_counters_start_at_zero_and_reset():
    from yscv_amd import onnx_ops as ops

    ops.reset_quant_runtime_stats()
    s = ops.quant_runtime_stats()
    assert s == ops.QuantRuntimeStats()
    assert set(vars(s)) == {"qlinear_matmul_fast", "qlinear_matmul_fallback", "matmul_integer_fast",
                            "matmul_integer_fallback", "int4_fast", "int4_fallback"}


def test_fast_switch_reads_the_environment():
    # quant_stats.rs:64-69: only the exact string "0" switches the fast paths off
    code = "from yscv_amd import onnx_ops as o; print(int(o.quant_int8_fast_enabled()))"
    for val, want in ((None, "1"), ("0", "0"), ("1", "1"), ("00", "1"), ("", "1")):
        env = dict(os.environ)
        env.pop("YSCV_QUANT_INT8_FAST", None)
        if val is not None:
            env["YSCV_QUANT_INT8_FAST"] = val
        out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == want, (val, out.stdout)


def test_bench_lcg_equals_the_reference_generator(oracle):
    """bench.py draws the stand-alone kernels' inputs from the reference micro-benchmark's generator
    (apps/llm-bench/src/bin/kernel_bench.rs:28-50), vectorised; it must equal the sequential restatement."""
    import numpy as np

    import bench

    for seed in (0xAA, 0xBB, 0x100, 0x200, 0x300 + 64, 7):
        assert np.array_equal(bench.lcg_i8(seed, 5000), oracle.lcg_i8(seed, 5000))
        assert np.array_equal(bench.lcg_f32(seed, 5000), oracle.lcg_f32(seed, 5000))
    # first values by hand: s1 = seed * a + c (mod 2^64)
    s1 = (0xAA * 6364136223846793005 + 1442695040888963407) % (1 << 64)
    assert int(bench.lcg_i8(0xAA, 1)[0]) == ((s1 >> 33) % 256) - 128

"""Generated-code check of the kernels that pipeline hand-written asynchronous loads (no GPU needed: hipcc
cross-compiles to assembly).  See isa_lint.py for the hazard."""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from isa_lint import copies_of_inflight_registers, scratch_bytes_per_kernel

CSRC = os.path.join(os.path.dirname(__file__), "..", "yscv_amd", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only"]
# the sources with asm loads whose wait is a separate statement, and their extra flags in the Makefile
SOURCES = {"int4_gemm_ring.hip": [], "decode_persistent.hip": [], "i8_gemm.hip": ["-ffp-contract=off"]}


def test_checker_sees_a_copy_between_load_and_wait():
    asm = "\n".join([
        "_Zkernel:",
        "\t;;#ASMSTART", "\tglobal_load_dwordx4 v[4:7], v1, s[2:3]", "\t;;#ASMEND",
        "\tv_mov_b64_e32 v[10:11], v[4:5]",
        "\t;;#ASMSTART", "\ts_waitcnt vmcnt(0)", "\t;;#ASMEND",
        "\tv_mov_b32_e32 v12, v6",
        "\ts_endpgm"])
    hits = copies_of_inflight_registers(asm)
    assert [(h[1], h[3]) for h in hits] == [(5, 3)]  # the copy before the wait, not the one after
    # a register that is written again is no longer waited for
    asm2 = asm.replace("\tv_mov_b64_e32 v[10:11], v[4:5]", "\tv_mov_b32_e32 v4, 0\n\tv_mov_b32_e32 v5, 0\n\tv_mov_b64_e32 v[10:11], v[4:5]")
    assert copies_of_inflight_registers(asm2) == []


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_register_of_a_load_in_flight_is_moved(tmp_path):
    def compile_one(item):
        name, extra = item
        out = tmp_path / (name + ".s")
        cmd = ["hipcc"] + FLAGS + extra + ["-o", str(out), os.path.join(CSRC, name)]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert proc.returncode == 0, proc.stdout[-2000:]
        return name, out.read_text()

    with ThreadPoolExecutor(max_workers=3) as pool:
        results = list(pool.map(compile_one, SOURCES.items()))
    report = []
    for name, text in results:
        hits = copies_of_inflight_registers(text)
        if hits:
            report.append(f"{name}: {len(hits)} moves of registers whose load is in flight, first {hits[0]}")
        # The LDS-ring GEMMs count their loads in flight with literal wait counts and name the registers of pending
        # loads in asm statements: an instantiation that spills (a tile whose accumulators, fragments and epilogue terms
        # exceed the 256 registers two waves per SIMD leave each) gets scratch traffic on the same counter and spill
        # code the pipeline was not written for.  Every instantiation in the library must fit its registers.
        for kern, scratch in scratch_bytes_per_kernel(text).items():
            if ("gemm_ring_kernel" in kern) and scratch != 0:
                report.append(f"{name}: {kern} uses {scratch} bytes of scratch per lane (register spills in a pipelined kernel)")
    assert not report, "\n".join(report)


def test_scratch_parser():
    asm = "_Zfoo:\n\ts_endpgm\n; NumVgprs: 12\n; ScratchSize: 120\n_Zbar:\n\ts_endpgm\n; ScratchSize: 0\n"
    assert scratch_bytes_per_kernel(asm) == {"_Zfoo": 120, "_Zbar": 0}

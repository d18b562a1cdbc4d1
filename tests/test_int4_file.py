"""Packed-int4 weight files: header, payload round trip and every rejection path (host only, no GPU call)."""
import numpy as np
import pytest

from yscv_amd import capi
from yscv_amd import kernels as K


def _weight(rng, n, k, g, sdt, zp):
    packed = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, n * (k // g)).astype(sdt)
    zps = rng.integers(0, 256, n * ((k // g + 1) // 2), dtype=np.uint8) if zp else None
    return packed, scales, zps


@pytest.mark.parametrize("n,k,g,sdt,zp", [(5, 96, 6, np.float32, False), (48, 256, 32, np.float16, True),
                                          (1, 2, 2, np.float32, False), (33, 384, 128, np.float16, True)])
def test_round_trip(tmp_path, n, k, g, sdt, zp):
    rng = np.random.default_rng(n * 1000 + k)
    packed, scales, zps = _weight(rng, n, k, g, sdt, zp)
    path = tmp_path / "w.yi4"
    fmt = K.NIBBLE_UNSIGNED if zp else K.NIBBLE_SIGNED
    K.int4_file_write(path, packed, scales, g, n, k, zero_points=zps, nibble_format=fmt)
    h = K.int4_file_read_header(path)
    assert (h.n, h.k, h.group_size, h.nibble_format, h.has_zero_points) == (n, k, g, fmt, int(zp))
    assert h.scale_dtype == (capi.F32 if sdt == np.float32 else capi.F16)
    assert (h.packed_bytes, h.scales_bytes, h.zero_points_bytes) == (packed.nbytes, scales.nbytes, 0 if zps is None else zps.nbytes)
    p2, s2, z2, _ = K.int4_file_read(path)
    assert np.array_equal(p2, packed) and np.array_equal(s2, scales) and s2.dtype == sdt
    assert (z2 is None) == (zps is None) and (zps is None or np.array_equal(z2, zps))
    # layout: 64-byte header, sections on 64-byte boundaries, in the documented order
    raw = path.read_bytes()
    up = lambda b: (b + 63) // 64 * 64
    assert raw[:8] == b"YSCVI4W\0" and len(raw) == 64 + up(packed.nbytes) + up(scales.nbytes) + up(0 if zps is None else zps.nbytes)
    assert raw[64:64 + packed.nbytes] == packed.tobytes()
    off = 64 + up(packed.nbytes)
    assert raw[off:off + scales.nbytes] == scales.tobytes()
    # the checksum is FNV-1a 64 over the payload sections
    hsh = 0xCBF29CE484222325
    for b in packed.tobytes() + scales.tobytes() + (b"" if zps is None else zps.tobytes()):
        hsh = ((hsh ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    assert h.checksum == hsh == int.from_bytes(raw[48:56], "little")


def test_rejections(tmp_path):
    rng = np.random.default_rng(7)
    packed, scales, zps = _weight(rng, 8, 64, 32, np.float32, True)
    good = tmp_path / "good.yi4"
    K.int4_file_write(good, packed, scales, 32, 8, 64, zero_points=zps, nibble_format=K.NIBBLE_UNSIGNED)
    raw = bytearray(good.read_bytes())

    def bad(name, data, match):
        p = tmp_path / name
        p.write_bytes(bytes(data))
        with pytest.raises(capi.YscvHipError, match=match):
            K.int4_file_read(p)

    bad("magic", b"NOTAFILE" + raw[8:], "bad magic")
    v2 = bytearray(raw); v2[8] = 2
    bad("version", v2, "version 2")
    bad("short_header", raw[:40], "shorter than")
    bad("truncated", raw[:-64], "bytes on disk")
    bad("trailing", raw + b"\0" * 64, "bytes on disk")
    flip = bytearray(raw); flip[64 + 5] ^= 0x10
    bad("payload", flip, "checksum mismatch")
    odd = bytearray(raw); odd[40:48] = (31).to_bytes(8, "little")
    bad("odd_group", odd, "must be even")
    huge = bytearray(raw); huge[24:32] = (1 << 50).to_bytes(8, "little")
    bad("huge", huge, "beyond what a file may hold")
    signed_zp = bytearray(raw); signed_zp[16:20] = (K.NIBBLE_SIGNED).to_bytes(4, "little")
    bad("signed_zp", signed_zp, "zero points need")
    with pytest.raises(capi.YscvHipError, match="cannot open"):
        K.int4_file_read_header(tmp_path / "missing.yi4")
    # writer-side contract
    with pytest.raises(capi.YscvHipError, match="zero points need"):
        K.int4_file_write(tmp_path / "x", packed, scales, 32, 8, 64, zero_points=zps, nibble_format=K.NIBBLE_SIGNED)
    with pytest.raises(ValueError):
        K.int4_file_write(tmp_path / "x", packed[:-1], scales, 32, 8, 64)

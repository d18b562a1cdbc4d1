"""yscv_hip_int4_matmul_static (scratch in a static device array, nothing allocated by the call) against
yscv_hip_int4_matmul on the same inputs: bit-identical, on two calls in a row of which the second is smaller, so
that whatever the first call left in the shared scratch must not leak into the second."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class _PoolProbe:
    """hipMemPoolAttrReservedMemCurrent of device 0's default stream-ordered pool, read through the HIP runtime the
    library itself is linked against (symbol lookup on its handle reaches its dependencies)."""

    def __init__(self):
        import ctypes as C

        from yscv_amd import capi

        self.C = C
        self.hip = capi.lib()._cdll
        self.pool = C.c_void_p()
        assert self.hip.hipDeviceGetDefaultMemPool(C.byref(self.pool), 0) == 0

    def reserved(self):
        v = self.C.c_uint64(0)
        assert self.hip.hipMemPoolGetAttribute(self.pool, 5, self.C.byref(v)) == 0  # hipMemPoolAttrReservedMemCurrent
        return int(v.value)


def _weight(K, rng, n, k, g, f16_scales):
    b = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16 if f16_scales else np.float32)
    return K.PackedInt4Weight(b, s, g, n, k, nibble_format=K.NIBBLE_UNSIGNED)


@pytest.mark.parametrize("n,k,g,xdt,f16s,m_first,m_second", [
    (4096, 14336, 32, "f16", True, 16, 3),      # skinny kernel, grid K split: partial sums in the scratch
    (1000, 1000, 8, "f32", False, 16, 1),       # padded K: hi / lo activation planes + row scales in the scratch
    (4096, 4096, 128, "bf16", True, 300, 40),   # LDS-ring GEMM: prepared activations in the scratch
    (768, 2048, 64, "f32", False, 200, 130),    # exact-scale GEMM (f32 scales, m > 128)
    (272, 14336, 32, "f32", False, 40, 17),     # 16-row skinny passes sharing the scratch
])
def test_static_scratch_call_equals_the_allocating_call(n, k, g, xdt, f16s, m_first, m_second):
    import torch

    from yscv_amd import kernels as K

    assert torch.cuda.is_available()
    rng = np.random.default_rng(n + k + m_first)
    w = _weight(K, rng, n, k, g, f16s)
    tdt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[xdt]
    for m in (m_first, m_second):
        x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(tdt).cuda()
        for odt in (torch.float32, tdt):
            want = w.matmul(x, out_dtype=odt)
            got = torch.full((m + 1, n), 5.0, device="cuda", dtype=odt)
            w.matmul_static(x, got[:m])
            torch.cuda.synchronize()
            assert torch.equal(got[:m], want), (m, odt)
            assert bool((got[m] == 5.0).all())
            # the property the entry point exists for: a batch of calls leaves the device's free memory and the
            # stream-ordered pool's reservation where they were (the allocating call takes its scratch from that pool)
            pool = _PoolProbe()
            free_before, reserved_before = torch.cuda.mem_get_info()[0], pool.reserved()
            for _ in range(8):
                w.matmul_static(x, got[:m])
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, (m, odt)
            assert pool.reserved() == reserved_before, (m, odt)
            assert torch.equal(got[:m], want), (m, odt)
    w.close()


def test_static_scratch_rejects_what_does_not_fit():
    import torch

    import yscv_amd
    from yscv_amd import capi
    from yscv_amd import kernels as K

    rng = np.random.default_rng(5)
    n, k, g = 256, 4096, 128
    w = _weight(K, rng, n, k, g, True)
    m = 8192  # f32 rows become two fp16 planes: 2 * 8192 * 4096 * 2 B = 128 MiB
    assert w.workspace_bytes(m, torch.float32) > capi.STATIC_SCRATCH_BYTES
    x = torch.zeros(m, k, device="cuda")
    out = torch.zeros(m, n, device="cuda")
    with pytest.raises(yscv_amd.YscvHipError, match="static scratch holds"):
        w.matmul_static(x, out)
    # the largest bf16 prefill named in the header fits
    m = 2048
    assert w.workspace_bytes(m, torch.bfloat16) <= capi.STATIC_SCRATCH_BYTES
    xb = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).bfloat16().cuda()
    got = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    w.matmul_static(xb, got)
    assert torch.equal(got, w.matmul(xb))
    w.close()

"""Two host threads share weight handles and call the library at the same time, each on its own stream: the runner of
the reference executes operators from its caller thread, a rayon worker or one of two branch threads
(crates/yscv-onnx/src/runner/mod.rs:339-400), with the weights shared immutably."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_two_threads_share_int4_and_int8_weights():
    import torch

    from yscv_amd import kernels as K

    rng = np.random.default_rng(5)
    n, k, g = 1040, 1024, 32
    w4 = K.PackedInt4Weight(rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16),
                            g, n, k, nibble_format=K.NIBBLE_UNSIGNED)
    bm = rng.integers(-127, 128, (k, n), dtype=np.int8)
    w8 = K.pack_i8_b_for_matmul(bm, k, n)
    cases = []
    for t in range(2):
        xs = torch.from_numpy(rng.standard_normal((3 + t, k)).astype(np.float32)).cuda()          # skinny kernel, f32 split in-kernel
        xw = torch.from_numpy(rng.standard_normal((70 + 9 * t, k)).astype(np.float32)).half().cuda()  # ring GEMM
        a8 = torch.from_numpy(rng.integers(0, 256, (100 + 30 * t, k), dtype=np.uint8)).cuda()
        cases.append((xs, xw, a8))
    torch.cuda.synchronize()
    expect = [(w4.matmul(xs).clone(), w4.matmul(xw, out_dtype=torch.float32).clone(), w8.matmul(a8, a_zp=128).clone()) for xs, xw, a8 in cases]
    torch.cuda.synchronize()
    errors = []
    start = threading.Barrier(2)

    def worker(t):
        try:
            xs, xw, a8 = cases[t]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                start.wait()
                for it in range(40):
                    got = (w4.matmul(xs), w4.matmul(xw, out_dtype=torch.float32), w8.matmul(a8, a_zp=128))
                    if it % 8 == 7:
                        stream.synchronize()
                        for gi, ei in zip(got, expect[t]):
                            if not torch.equal(gi, ei):
                                errors.append((t, it, "result differs"))
                stream.synchronize()
        except Exception as e:  # noqa: BLE001 -- reported by the main thread
            errors.append((t, -1, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads), "a worker did not finish"
    assert not errors, errors[:3]
    w4.close()
    w8.close()

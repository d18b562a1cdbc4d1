"""The operators between the MatMuls of an LLM graph as stand-alone device entry points (yscv_hip_rms_norm_dev,
yscv_hip_rope_dev, yscv_hip_gqa_attention_dev) against the numpy restatements of oracle/decoder_ref.py, which
tests/test_oracle_decoder.py pins to the reference's vectors and closed forms."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch

    assert torch.cuda.is_available()
    from yscv_amd import onnx_ops

    return onnx_ops


@pytest.mark.parametrize("shape", [(1, 8), (3, 4096), (2, 5, 1000), (7, 33), (4, 9000)])
def test_rms_norm_matches_the_restatement(ops, shape):
    """ops/norm.rs:1497-1518: y = x * (1 / sqrt(mean(x^2) + eps)) * gamma; the GPU adds the squares in another order
    (relative 1e-6 of a row's sum), every other step is the same f32 operation."""
    import torch

    from oracle.decoder_ref import rmsnorm

    rng = np.random.default_rng(sum(shape))
    x = (rng.standard_normal(shape) * rng.uniform(0.01, 30.0)).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, shape[-1]).astype(np.float32)
    for eps in (1e-5, 1e-3):
        y = ops.rms_norm(torch.from_numpy(x).cuda(), torch.from_numpy(gamma).cuda(), eps).cpu().numpy()
        want = rmsnorm(x, gamma, eps)
        assert y.shape == want.shape
        assert np.abs(y - want).max() <= 4e-6 * np.abs(want).max()
    # the reference's own vector (normalization.rs:347-390 form): [3, 4] with gamma 1 -> rms = sqrt(12.5 + eps)
    y = ops.rms_norm(torch.tensor([[3.0, 4.0]]).cuda(), torch.ones(2).cuda(), 1e-5).cpu().numpy()
    assert np.allclose(y, np.array([[3.0, 4.0]]) / np.sqrt(12.5 + 1e-5), rtol=1e-6)


def test_rms_norm_rejects_a_bad_epsilon(ops):
    import torch

    import yscv_amd

    x, g = torch.ones(2, 4).cuda(), torch.ones(4).cuda()
    for eps in (0.0, -1.0, float("nan"), float("inf")):
        with pytest.raises(yscv_amd.YscvHipError, match="epsilon"):
            ops.rms_norm(x, g, eps)


@pytest.mark.parametrize("hq,hkv,d,seq,offset,theta", [(4, 2, 64, 5, 0, 10000.0), (16, 2, 64, 43, 7, 1000000.0),
                                                        (3, 1, 128, 1, 2047, 10000.0), (2, 2, 6, 9, 3, 500.0)])
def test_rope_matches_the_restatement(ops, hq, hkv, d, seq, offset, theta):
    """ops/rope.rs:24-117 in place on q [seq][heads][d] and k; sin / cos of the device against numpy's: a few ulp of
    the angle at position ~2000 (absolute 2e-4 of |x|), so tolerance, not bits."""
    import torch

    from oracle.decoder_ref import rope

    rng = np.random.default_rng(hq * 100 + d + seq)
    q = rng.standard_normal((seq, hq, d)).astype(np.float32)
    k = rng.standard_normal((seq, hkv, d)).astype(np.float32)
    qd, kd = torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda()
    ops.apply_rotary_embedding(qd, kd, hq, hkv, d, seq, offset, theta)
    for got, src in ((qd.cpu().numpy(), q), (kd.cpu().numpy(), k)):
        want = np.stack([rope(src[p], p + offset, theta) for p in range(seq)])
        assert np.abs(got - want).max() <= 5e-4 * np.abs(want).max()
        # rotations preserve the norm of every (i, i + d/2) pair (proptest of the reference: proptest_tests.rs:176-210)
        assert np.allclose((got ** 2).sum(-1), (src ** 2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("B,Sq,Sk,hq,hkv,d", [
    (1, 1, 1, 4, 4, 64),        # a single position: the softmax is 1
    (2, 5, 37, 16, 2, 64),      # the reference benchmark model's head layout: eight query heads per kv head
    (1, 43, 43, 8, 2, 64),      # a prompt against itself (the operator has no mask)
    (2, 17, 300, 6, 2, 128),    # three query heads per kv head, more than one query tile
    (1, 3, 129, 4, 1, 32),
    (1, 2, 65, 3, 3, 96),
    (1, 150, 170, 8, 2, 64),    # 64 queries and more: one wave per 32 queries, no split over the keys
    (2, 64, 33, 2, 1, 128),
    (1, 97, 97, 3, 3, 32),
])
def test_gqa_attention_matches_the_restatement(ops, B, Sq, Sk, hq, hkv, d):
    """runner/linear.rs:552-646 against gqa_attend per query position (every query sees every key position).  The GPU
    takes q, k, v and the softmax weights into the matrix cores as fp16: about 1e-3 relative."""
    import torch

    from oracle.decoder_ref import gqa_attend

    rng = np.random.default_rng(B + Sq * 7 + Sk * 13 + d)
    q = rng.standard_normal((B, Sq, hq * d)).astype(np.float32)
    k = rng.standard_normal((B, Sk, hkv * d)).astype(np.float32)
    v = rng.standard_normal((B, Sk, hkv * d)).astype(np.float32)
    out = ops.exec_grouped_query_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                                           hq, hkv).cpu().numpy()
    assert out.shape == (B, Sq, hq * d)
    for b in range(B):
        kc, vc = k[b].reshape(Sk, hkv, d), v[b].reshape(Sk, hkv, d)
        for s in range(Sq):
            want = gqa_attend(q[b, s].reshape(hq, d), kc, vc, hq // hkv).reshape(-1)
            assert np.abs(out[b, s] - want).max() <= 4e-3 * np.abs(want).max() + 1e-5, (b, s)


def test_gqa_attention_with_large_scores_and_equal_keys(ops):
    """Closed forms: equal keys give the mean of the values; one key with a far larger score takes all the weight
    (scores of several hundred: the maximum is subtracted before the exponential)."""
    import torch

    d, Sk = 64, 50
    q = np.full((1, 1, d), 3.0, np.float32)
    k = np.tile(np.full((1, 1, d), 0.5, np.float32), (1, Sk, 1))
    v = np.random.default_rng(0).standard_normal((1, Sk, d)).astype(np.float32)
    out = ops.exec_grouped_query_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), 1).cpu().numpy()
    assert np.abs(out[0, 0] - v[0].mean(0)).max() < 2e-3
    k[0, 17] = 40.0  # score 40 * 3 * 64 / 8 = 960 against 12
    out = ops.exec_grouped_query_attention(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), 1).cpu().numpy()
    assert np.abs(out[0, 0] - v[0, 17]).max() < 2e-3


def test_gqa_attention_rejects_what_it_cannot_run(ops):
    import torch

    import yscv_amd

    q = torch.zeros(1, 1, 2 * 48).cuda()
    kv = torch.zeros(1, 4, 2 * 48).cuda()
    with pytest.raises(yscv_amd.YscvHipError, match="head width"):
        ops.exec_grouped_query_attention(q, kv, kv, 2, 2)
    with pytest.raises(yscv_amd.YscvHipError, match="query heads"):
        ops.exec_grouped_query_attention(torch.zeros(1, 1, 3 * 64).cuda(), torch.zeros(1, 4, 2 * 64).cuda(),
                                         torch.zeros(1, 4, 2 * 64).cuda(), 3, 2)

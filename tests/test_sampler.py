"""Host-side sampler (sample_token of crates/yscv-onnx/src/generate.rs:121-208): needs no GPU.  Pinned by the
reference's own test vectors, by values worked out by hand and by the statistics of many draws -- not by a second copy
of the algorithm."""
import numpy as np


def _xorshift64(x):
    x ^= (x << 13) & 0xFFFFFFFFFFFFFFFF
    x ^= x >> 7
    x ^= (x << 17) & 0xFFFFFFFFFFFFFFFF
    return x


def test_reference_vector_greedy():
    from yscv_amd import kernels as K

    # generate.rs:267-274: top_k = 1 forces the highest logit
    logits = np.array([0.0, 0.0, 10.0, 0.0, 0.0], np.float32)
    tok, rng = K.sample_token(logits, 1, 1.0, 42)
    assert tok == 2
    assert rng == _xorshift64(42)                      # the draw advances the xorshift64 state exactly once
    assert logits.tolist() == [0.0, 0.0, 1.0, 0.0, 0.0]  # in place: the distribution the draw was made from


def test_generate_basic_vector_all_42():
    from yscv_amd import kernels as K

    # generate.rs:214-242: logit 10 at token 42 of 100, no top-k / top-p, five draws from state 0xdeadbeef: all 42
    rng = 0xDEADBEEF
    for _ in range(5):
        logits = np.zeros(100, np.float32)
        logits[42] = 10.0
        tok, rng = K.sample_token(logits, 0, 1.0, rng)
        assert tok == 42


def test_hand_worked_top_k_top_p_and_draw():
    from yscv_amd import kernels as K

    # logits ln(1), ln(2), ln(3), ln(4): probabilities 0.1, 0.2, 0.3, 0.4
    base = np.log(np.array([1.0, 2.0, 3.0, 4.0])).astype(np.float32)
    # top_k = 2 keeps tokens 2 and 3: 3/7 and 4/7
    l = base.copy()
    K.sample_token(l, 2, 1.0, 1)
    assert np.allclose(l, [0, 0, 3 / 7, 4 / 7], atol=1e-6) and l[0] == 0.0 and l[1] == 0.0
    # top_p = 0.65: 0.4 + 0.3 = 0.7 > 0.65 cuts after the second most probable token
    l = base.copy()
    K.sample_token(l, 0, 0.65, 1)
    assert np.allclose(l, [0, 0, 3 / 7, 4 / 7], atol=1e-6)
    # top_p = 0.35 keeps only the most probable one (0.4 > 0.35)
    l = base.copy()
    tok, _ = K.sample_token(l, 0, 0.35, 1)
    assert l.tolist() == [0.0, 0.0, 0.0, 1.0] and tok == 3
    # the draw: u = state / 2^64 in f32, first index whose cumulative probability exceeds it
    for seed in (1, 7, 0xDEADBEEF, 2**63 + 12345):
        l = base.copy()
        tok, rng = K.sample_token(l, 0, 1.0, seed)
        assert rng == _xorshift64(seed)
        u = np.float32(rng) / np.float32(2.0**64)
        cum = np.cumsum(np.array([0.1, 0.2, 0.3, 0.4]))
        want = int(np.searchsorted(cum, float(u), side="right"))
        assert abs(float(u) - cum).min() < 1e-5 or tok == min(want, 3)


def test_draw_frequencies_follow_the_softmax():
    from yscv_amd import kernels as K

    rng_np = np.random.default_rng(3)
    base = rng_np.standard_normal(12).astype(np.float32) * 1.5
    p = np.exp(base - base.max())
    p /= p.sum()
    counts = np.zeros(12)
    state = 0x1234567
    n = 40000
    for _ in range(n):
        l = base.copy()
        tok, state = K.sample_token(l, 0, 1.0, state)
        counts[tok] += 1
    assert np.abs(counts / n - p).max() < 0.012  # ~5 sigma for the largest probabilities
    # with top_k = 3 only the three largest logits ever come out, in their renormalised proportions
    top = np.argsort(base)[-3:]
    counts = np.zeros(12)
    for _ in range(n // 4):
        l = base.copy()
        tok, state = K.sample_token(l, 3, 1.0, state)
        counts[tok] += 1
    assert set(np.nonzero(counts)[0]) <= set(top.tolist())
    q = p[top] / p[top].sum()
    assert np.abs(counts[top] / counts.sum() - q).max() < 0.025


def test_fallback_and_edge_cases():
    import pytest

    import yscv_amd
    from yscv_amd import kernels as K

    # all logits -inf: softmax gives NaN sums; the reference falls through to max_by (last maximal element)
    l = np.full(4, -np.inf, np.float32)
    tok, _ = K.sample_token(l, 0, 1.0, 5)
    assert 0 <= tok < 4
    # top_k >= vocab and top_k = 0 leave the logits alone before the softmax
    a = np.array([1.0, 2.0, 3.0], np.float32)
    b = a.copy()
    K.sample_token(a, 3, 1.0, 9)
    K.sample_token(b, 0, 1.0, 9)
    assert np.array_equal(a, b)
    with pytest.raises(yscv_amd.YscvHipError):
        yscv_amd.lib().sample_token(None, 0, 0, 1.0, None, None)

"""Pins oracle/decoder_ref.py (the numpy checker of the decode loop) without a GPU.

Every glue function is held to the reference's own unit-test vectors where it has some, and otherwise to
closed forms chosen so that a plausible mistake fails one of them: mean-vs-sum in RMSNorm, the rotary pairing
(i, i + d/2) against (2i, 2i + 1), the sign of the rotation, kv_h = qh / groups against qh % kv_heads, the
1/sqrt(d) score scale, a missing max subtraction, first-vs-last maximum in the greedy pick, the nibble order and
the zero point of the int4 weights, and the wiring of one whole decoder step.
"""
import math

import numpy as np
import pytest

from oracle import decoder_ref as R


# ---- RMSNorm: crates/yscv-kernels/src/tests/normalization.rs:347-390 -----------------------------------------------
def test_rmsnorm_reference_vectors():
    x = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    rms = np.sqrt(np.float32(30.0 / 4.0 + 1e-5))
    for g in (1.0, 2.0):
        out = R.rmsnorm(x, np.full(4, g, np.float32), 1e-5)
        assert out.shape == (1, 4)
        np.testing.assert_allclose(out[0], g * np.array([1, 2, 3, 4], np.float32) / rms, atol=1e-4)  # the reference's bound
        np.testing.assert_allclose(out[0], g * np.array([1, 2, 3, 4], np.float64) / math.sqrt(7.5 + 1e-5), rtol=3e-7)


def test_rmsnorm_is_mean_not_sum_and_per_row():
    # a sum instead of a mean would give 1/sqrt(4 c^2) = half of this; gamma is per element
    x = np.array([[3.0, 3.0, 3.0, 3.0], [0.5, -0.5, 0.5, -0.5]], np.float32)
    g = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    out = R.rmsnorm(x, g, 0.0 + 1e-12)
    np.testing.assert_allclose(out[0], g, rtol=1e-6)
    np.testing.assert_allclose(out[1], g * np.array([1, -1, 1, -1]), rtol=1e-6)
    # eps sits inside the square root, added to the mean
    out = R.rmsnorm(np.zeros((1, 4), np.float32) + 1e-3, np.ones(4, np.float32), 1.0)
    np.testing.assert_allclose(out[0], 1e-3 / math.sqrt(1e-6 + 1.0), rtol=1e-6)


# ---- RoPE: crates/yscv-kernels/src/ops/rope.rs:24-117, tests :186-286 ----------------------------------------------
def test_rope_position_zero_is_identity_and_norm_is_kept():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 16)).astype(np.float32)
    np.testing.assert_array_equal(R.rope(x, 0, 10000.0), x)
    # rope_orthogonality (rope.rs:260-286): ones of d = 16 at offset 5 keep their norm to 1e-4
    y = R.rope(np.ones((1, 16), np.float32), 5, 10000.0)
    assert abs(float(np.linalg.norm(y)) - 4.0) < 1e-4
    for pos in (1, 7, 2047):
        yy = R.rope(x, pos, 10000.0)
        np.testing.assert_allclose(np.linalg.norm(yy, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)


def test_rope_hand_pair_d4():
    # d = 4: inv_freq = [1, theta^(-1/2)] = [1, 0.01]; pairs are (0, 2) and (1, 3), NOT (0, 1) and (2, 3)
    pos = 3
    x = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    a0, a1 = 1.0 * pos, 0.01 * pos
    want = np.array([1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                     1 * math.sin(a0) + 3 * math.cos(a0), 2 * math.sin(a1) + 4 * math.cos(a1)])
    np.testing.assert_allclose(R.rope(x, pos, 10000.0)[0], want, rtol=2e-6, atol=2e-6)
    # what the interleaved pairing (2i, 2i+1) would give differs by far more than the tolerance
    inter = np.array([1 * math.cos(a0) - 2 * math.sin(a0), 1 * math.sin(a0) + 2 * math.cos(a0),
                      3 * math.cos(a1) - 4 * math.sin(a1), 3 * math.sin(a1) + 4 * math.cos(a1)])
    assert np.abs(inter - want).max() > 0.5
    # a unit vector on the first axis turns towards its partner with a positive sine
    e = R.rope(np.array([[1.0, 0.0, 0.0, 0.0]], np.float32), 1, 10000.0)[0]
    np.testing.assert_allclose(e, [math.cos(1.0), 0.0, math.sin(1.0), 0.0], atol=1e-6)


def test_rope_offsets_add():
    # rope_kv_cache_offset (rope.rs:214-258): rotating by a then b equals rotating by a + b
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 128)).astype(np.float32)
    np.testing.assert_allclose(R.rope(R.rope(x, 2, 10000.0), 3, 10000.0), R.rope(x, 5, 10000.0), atol=1e-5)
    # the slowest frequency of d = 128 is theta^(-126/128)
    y = R.rope(np.eye(1, 128, 63, dtype=np.float32), 1000, 10000.0)[0]
    ang = 1000.0 * 10000.0 ** (-126.0 / 128.0)
    np.testing.assert_allclose([y[63], y[127]], [math.cos(ang), math.sin(ang)], atol=1e-5)


# ---- grouped-query attention: crates/yscv-onnx/src/runner/linear.rs:552-646 ------------------------------------------
def test_gqa_single_position_returns_its_value_row():
    rng = np.random.default_rng(3)
    q = rng.standard_normal((4, 8)).astype(np.float32)
    kc = rng.standard_normal((1, 2, 8)).astype(np.float32)
    vc = rng.standard_normal((1, 2, 8)).astype(np.float32)
    out = R.gqa_attend(q, kc, vc, 2)
    # heads 0, 1 read kv head 0 and heads 2, 3 kv head 1 (kv_h = qh / groups; qh % kv_heads would give 0 1 0 1)
    np.testing.assert_allclose(out, vc[0][[0, 0, 1, 1]], rtol=1e-6)


def test_gqa_equal_scores_give_the_mean_of_v():
    rng = np.random.default_rng(4)
    vc = rng.standard_normal((5, 1, 8)).astype(np.float32)
    kc = np.tile(rng.standard_normal((1, 1, 8)).astype(np.float32), (5, 1, 1))
    q = rng.standard_normal((2, 8)).astype(np.float32)
    out = R.gqa_attend(q, kc, vc, 2)
    np.testing.assert_allclose(out, np.tile(vc[:, 0].mean(0), (2, 1)), rtol=1e-5, atol=1e-6)
    # zero query: uniform weights whatever the keys
    out = R.gqa_attend(np.zeros((2, 8), np.float32), rng.standard_normal((5, 1, 8)).astype(np.float32), vc, 2)
    np.testing.assert_allclose(out, np.tile(vc[:, 0].mean(0), (2, 1)), rtol=1e-5, atol=1e-6)


def test_gqa_score_scale_two_positions_closed_form():
    # d = 16, q = k0 = e0 * c, k1 = 0: scores (c^2 / 4, 0) -> weights sigmoid(c^2 / 4); without the 1/sqrt(d) factor
    # the weight would be sigmoid(c^2)
    d, c = 16, 2.0
    q = np.zeros((1, d), np.float32)
    q[0, 0] = c
    kc = np.zeros((2, 1, d), np.float32)
    kc[0, 0, 0] = c
    vc = np.zeros((2, 1, d), np.float32)
    vc[0, 0, :] = 1.0
    vc[1, 0, :] = -1.0
    w0 = 1.0 / (1.0 + math.exp(-(c * c) / math.sqrt(d)))
    out = R.gqa_attend(q, kc, vc, 1)
    np.testing.assert_allclose(out[0], np.full(d, w0 - (1 - w0)), rtol=1e-6)
    assert abs((2 / (1 + math.exp(-c * c)) - 1) - (2 * w0 - 1)) > 0.3


def test_gqa_large_scores_do_not_overflow():
    # max-subtracted softmax: scores of 400 and 399 give finite weights e / (1 + e)
    d = 4
    q = np.array([[800.0, 0, 0, 0]], np.float32)
    kc = np.array([[[1.0, 0, 0, 0]], [[0.9975, 0, 0, 0]]], np.float32)
    vc = np.array([[[1.0, 0, 0, 0]], [[0.0, 1, 0, 0]]], np.float32)
    out = R.gqa_attend(q, kc, vc, 1)
    w = 1.0 / (1.0 + math.exp(-1.0))
    np.testing.assert_allclose(out[0], [w, 1 - w, 0, 0], rtol=1e-4)


def test_gqa_matches_reference_loops():
    """The triple loop of exec_grouped_query_attention (linear.rs:583-633) written out in Python floats."""
    rng = np.random.default_rng(5)
    nh, nkv, d, S = 6, 2, 8, 7
    groups = nh // nkv
    q = rng.standard_normal((nh, d)).astype(np.float32)
    kc = rng.standard_normal((S, nkv, d)).astype(np.float32)
    vc = rng.standard_normal((S, nkv, d)).astype(np.float32)
    want = np.zeros((nh, d))
    for qh in range(nh):
        kv_h = qh // groups
        scores, mx = [], -math.inf
        for sk in range(S):
            s = sum(float(q[qh, t]) * float(kc[sk, kv_h, t]) for t in range(d)) * (1.0 / math.sqrt(d))
            mx = max(mx, s)
            scores.append(s)
        ex = [math.exp(s - mx) for s in scores]
        tot = sum(ex)
        for t in range(d):
            want[qh, t] = sum(ex[sk] / tot * float(vc[sk, kv_h, t]) for sk in range(S))
    np.testing.assert_allclose(R.gqa_attend(q, kc, vc, groups), want, rtol=1e-5, atol=1e-6)


# ---- SwiGLU, greedy pick ---------------------------------------------------------------------------------------
def test_swiglu_closed_form():
    g = np.array([0.0, 1.0, -1.0, 20.0, -20.0], np.float32)
    u = np.array([3.0, 2.0, 2.0, 0.5, 0.5], np.float32)
    want = [0.0, 2.0 / (1 + math.exp(-1.0)), -2.0 / (1 + math.exp(1.0)), 10.0 / (1 + math.exp(-20.0)), -10.0 / (1 + math.exp(20.0))]
    np.testing.assert_allclose(R.swiglu(g, u), want, rtol=1e-6, atol=1e-12)


def test_greedy_pick_takes_the_last_maximum():
    # Iterator::max_by returns the last of several equal maxima (apps/llm-bench/src/main.rs:538-543)
    assert R.greedy_pick(np.array([1.0, 5.0, 2.0, 5.0, 0.0], np.float32)) == 3
    assert R.greedy_pick(np.array([7.0, 5.0], np.float32)) == 0
    assert R.greedy_pick(np.zeros(9, np.float32)) == 8


# ---- int4 weights --------------------------------------------------------------------------------------------
def test_dequant_hand_vector_and_oracle(oracle):
    # MatMulNBits form of the hand-derived vector: bytes [0xA9, 0x70] are nibbles 9, 10, 0, 7 = 1, 2, -8, -1 after the
    # zero point 8; scales 0.5, 0.25 with group size 2
    w = R.dequant_uint4(np.array([0xA9, 0x70], np.uint8), np.array([0.5, 0.25], np.float16), 1, 4, 2)
    np.testing.assert_array_equal(w, [[0.5, 1.0, -2.0, -0.25]])
    assert float(w[0] @ np.array([1, 2, 3, 4], np.float32)) == -4.5
    # against the C restatement of packed_int4_gemm_scalar (pinned by the reference's goldens in test_oracle_int4.py)
    rng = np.random.default_rng(6)
    n, k, g, m = 24, 128, 32, 3
    p = rng.integers(0, 256, n * k // 2, dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float32)
    ref = oracle.packed_int4_gemm_scalar(p ^ 0x88, s.astype(np.float32), x, m, n, k, g)
    got = x @ R.dequant_uint4(p, s, n, k, g).T
    np.testing.assert_allclose(got, ref.reshape(m, n), rtol=1e-5, atol=1e-5)


# ---- one whole step against an independent float64 transcription of the block structure ---------------------------
CFG = dict(n_layers=2, d_model=64, n_heads=4, n_kv_heads=2, head_dim=16, d_ff=96, vocab=40, group_size=32,
           max_batch=2, max_ctx=16, max_steps=4, rope_theta=10000.0, rms_eps=1e-5)


def _tiny_model(rng, cfg):
    D, hd, g = cfg["d_model"], cfg["head_dim"], cfg["group_size"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    shapes = {"q": (hq, D), "k": (hkv, D), "v": (hkv, D), "o": (D, hq), "gate": (ff, D), "up": (ff, D), "down": (D, ff)}
    lin, norms = {}, {}
    for l in range(cfg["n_layers"]):
        for kind, (n, k) in shapes.items():
            lin[(l, kind)] = (rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.01, 0.05, n * (k // g)).astype(np.float16))
        norms[(l, "attn")] = rng.uniform(0.5, 1.5, D).astype(np.float32)
        norms[(l, "ffn")] = rng.uniform(0.5, 1.5, D).astype(np.float32)
    lin[("lm_head",)] = (rng.integers(0, 256, cfg["vocab"] * D // 2, dtype=np.uint8),
                         rng.uniform(0.01, 0.05, cfg["vocab"] * (D // g)).astype(np.float16))
    norms[("final",)] = rng.uniform(0.5, 1.5, D).astype(np.float32)
    emb = rng.standard_normal((cfg["vocab"], D)).astype(np.float16)
    return lin, norms, emb, shapes


def _step_f64(cfg, lin, norms, emb, shapes, kc, vc, token, pos):
    """Pre-norm Llama block in float64 without any fp16 rounding: h += o(attn(rope(q), cache)), h += down(silu(gate) * up)."""
    D, hd, nh, nkv, g = cfg["d_model"], cfg["head_dim"], cfg["n_heads"], cfg["n_kv_heads"], cfg["group_size"]

    def W(key):
        n, k = (cfg["vocab"], D) if key == ("lm_head",) else shapes[key[1]]
        p, s = lin[key]
        out = np.zeros((n, k))
        for r in range(n):
            for c in range(k):
                b = int(p[(r * k + c) // 2])
                qv = (b & 15) if c % 2 == 0 else (b >> 4)
                out[r, c] = (qv - 8) * float(s[r * (k // g) + c // g])
        return out

    def norm(x, gam):
        return x / math.sqrt(float((x * x).sum()) / len(x) + cfg["rms_eps"]) * gam.astype(np.float64)

    def rot(vec):
        out = vec.copy()
        for i in range(hd // 2):
            a = pos * cfg["rope_theta"] ** (-2.0 * i / hd)
            out[i] = vec[i] * math.cos(a) - vec[i + hd // 2] * math.sin(a)
            out[i + hd // 2] = vec[i] * math.sin(a) + vec[i + hd // 2] * math.cos(a)
        return out

    h = emb[token].astype(np.float64)
    for l in range(cfg["n_layers"]):
        xn = norm(h, norms[(l, "attn")])
        q = (W((l, "q")) @ xn).reshape(nh, hd)
        k = (W((l, "k")) @ xn).reshape(nkv, hd)
        v = (W((l, "v")) @ xn).reshape(nkv, hd)
        kc[l].append(np.stack([rot(k[j]) for j in range(nkv)]))
        vc[l].append(v)
        ao = np.zeros((nh, hd))
        for qh in range(nh):
            kvh = qh // (nh // nkv)
            qr = rot(q[qh])
            sc = np.array([float(kk[kvh] @ qr) / math.sqrt(hd) for kk in kc[l]])
            pr = np.exp(sc - sc.max())
            pr /= pr.sum()
            ao[qh] = sum(pr[t] * vc[l][t][kvh] for t in range(len(pr)))
        h = h + W((l, "o")) @ ao.reshape(-1)
        xn = norm(h, norms[(l, "ffn")])
        gt, up = W((l, "gate")) @ xn, W((l, "up")) @ xn
        h = h + W((l, "down")) @ (gt / (1 + np.exp(-gt)) * up)
    return W(("lm_head",)) @ norm(h, norms[("final",)])


def test_ref_decoder_steps_match_float64_transcription():
    rng = np.random.default_rng(7)
    cfg = dict(CFG)
    lin, norms, emb, shapes = _tiny_model(rng, cfg)
    ref = R.RefDecoder(cfg, lin, norms, emb)
    ref32 = R.RefDecoder(cfg, lin, norms, emb, round_f16=False)
    kc = [[] for _ in range(cfg["n_layers"])]
    vc = [[] for _ in range(cfg["n_layers"])]
    tok = 3
    for pos in range(3):
        got = ref.step(np.array([tok, tok]), pos)
        got32 = ref32.step(np.array([tok, tok]), pos)
        want = _step_f64(cfg, lin, norms, emb, shapes, kc, vc, tok, pos)
        # fp16 roundings of the checker's activations are the only difference: ~1e-3 relative; without them
        # (round_f16=False) what is left is f32 against float64 arithmetic
        scale = np.abs(want).max()
        assert np.abs(got[0] - want).max() / scale < 5e-3, pos
        assert np.abs(got32[0] - want).max() / scale < 2e-5, pos
        assert not np.array_equal(got[0], got32[0])
        np.testing.assert_array_equal(got[0], got[1])  # batch rows are independent
        tok = R.greedy_pick(got[0])


def test_ref_decoder_set_kv_and_overwrite_at_pos():
    """A cache loaded with set_kv gives the same logits as one built step by step, and step() at position p
    discards anything cached at or beyond p."""
    rng = np.random.default_rng(8)
    cfg = dict(CFG)
    lin, norms, emb, _ = _tiny_model(rng, cfg)
    a = R.RefDecoder(cfg, lin, norms, emb)
    toks = [5, 9, 11]
    for pos, t in enumerate(toks):
        la = a.step(np.array([t]), pos)
    b = R.RefDecoder(cfg, lin, norms, emb)
    for l in range(cfg["n_layers"]):
        b.set_kv(l, a.kc[l][0][None, :2], a.vc[l][0][None, :2])
    lb = b.step(np.array([toks[2]]), 2)
    np.testing.assert_array_equal(la, lb)
    la2 = a.step(np.array([toks[2]]), 2)  # position 2 again: the old entry is replaced, not appended to
    np.testing.assert_array_equal(la2, la)
    assert a.kc[0][0].shape[0] == 3


# ---- int8 cache mode of the checker (KvCache with KvDtype::I8, crates/yscv-onnx/src/runner/kv_cache.rs:45-79) ---------
def test_kv_i8_roundtrip_hand_vector_and_bounds(oracle):
    # kv_cache.rs:321-358 holds a bound test (|error| <= scale); a hand vector on top: absmax 2.54 -> scale 0.02,
    # 1.27 -> 63.5 -> 64 (half away from zero, round_ties_even would give 64 too), 0.25 -> 12.5 -> 13, -0.01 -> -0.5 -> -1
    row = np.array([[2.54, 1.27, 0.25, -0.01, 0.0, -2.54]], np.float32)
    got = R.kv_i8_roundtrip(row)
    scale = np.float32(2.54) / np.float32(127.0)
    np.testing.assert_allclose(got[0], np.array([127, 64, 13, -1, 0, -127], np.float32) * scale, rtol=1e-6)
    rng = np.random.default_rng(9)
    rows = (rng.standard_normal((7, 256)) * rng.uniform(0.1, 30, (7, 1))).astype(np.float32)
    back = R.kv_i8_roundtrip(rows)
    step = np.abs(rows).max(1, keepdims=True) / 127.0
    assert (np.abs(back - rows) <= step * 0.5 * (1 + 1e-5)).all()      # the scale is per row, not per tensor or per head
    assert np.array_equal(R.kv_i8_roundtrip(np.zeros((2, 8), np.float32)), np.zeros((2, 8), np.float32))


def test_ref_decoder_kv_i8_quantises_rows_over_all_kv_heads():
    rng = np.random.default_rng(10)
    cfg = dict(CFG)
    lin, norms, emb, _ = _tiny_model(rng, cfg)
    a = R.RefDecoder(cfg, lin, norms, emb, kv_i8=True)
    f = R.RefDecoder(cfg, lin, norms, emb)
    la, lf = a.step(np.array([5]), 0), f.step(np.array([5]), 0)
    for l in range(cfg["n_layers"]):
        for cache in (a.kc[l][0], a.vc[l][0]):
            row = cache[0].reshape(-1)                                   # one position, both kv heads: one scale
            scale = np.abs(row).max() / 127.0
            q = row / scale
            assert np.abs(q - np.round(q)).max() < 1e-3 and np.abs(q).max() <= 127.0 + 1e-3
    # quantisation noise of a few 1e-3 of the value range, not a different computation
    assert 0 < np.abs(la - lf).max() < 0.05 * np.abs(lf).max()
    # a cache loaded with set_kv is quantised the same way
    b = R.RefDecoder(cfg, lin, norms, emb, kv_i8=True)
    k = rng.standard_normal((1, 3, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float32)
    b.set_kv(0, k, k)
    np.testing.assert_array_equal(b.kc[0][0].reshape(3, -1), R.kv_i8_roundtrip(k[0].reshape(3, -1)))

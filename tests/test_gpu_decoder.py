"""GPU decode loop vs the numpy restatement (tolerance only: RoPE / softmax / SiLU use libm-class
functions, and the activations between kernels are fp16)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# Logits against the numpy restatement, as a fraction of max|logit|: the float bar of the int4 path (relative error
# <= 1e-2 of the reference CPU kernel's output), the same bar tests/test_gpu_decoder_7b.py holds at the 7B widths.
LOGIT_TOL = 1e-2

CFG = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=128, d_ff=384, vocab=512, group_size=32,
           max_batch=3, max_ctx=256, max_steps=16, rope_theta=10000.0, rms_eps=1e-5)


def _build(rng, cfg, kv_dtype="f16", emb_scale=1.0, symmetric=False, v_mul=1.0, qkv_bias=False):
    from oracle.decoder_ref import RefDecoder
    from yscv_amd.decoder import Decoder

    D, hd, g = cfg["d_model"], cfg["head_dim"], cfg["group_size"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    shapes = {"q": (hq, D), "k": (hkv, D), "v": (hkv, D), "o": (D, hq), "gate": (ff, D), "up": (ff, D), "down": (D, ff)}
    dec = Decoder(kv_dtype=kv_dtype, **cfg)
    linears, norms, biases = {}, {}, {}

    def nibbles(count):
        # symmetric: nibbles 1..15 only, mean zero after the zero point 8.  Uniform bytes give every projection output a
        # common offset, q and k then sit where an fp16 ulp is 0.03 and the softmax amplifies one-ulp differences
        # between two correct implementations (tests/test_gpu_decoder_7b.py has the numbers)
        if not symmetric:
            return rng.integers(0, 256, count, dtype=np.uint8)
        return (rng.integers(1, 16, count, dtype=np.uint8) | (rng.integers(1, 16, count, dtype=np.uint8) << 4)).astype(np.uint8)

    for l in range(cfg["n_layers"]):
        for kind, (n, k) in shapes.items():
            p = nibbles(n * k // 2)
            s = rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)
            if kind == "v":
                s = (s.astype(np.float32) * v_mul).astype(np.float16)  # small values: rows of the V cache far below 1
            linears[(l, kind)] = (p, s)
            dec.set_linear(l, kind, p, s, n, k)
        for kind in ("attn", "ffn"):
            gmm = rng.uniform(0.5, 1.5, D).astype(np.float32)
            norms[(l, kind)] = gmm
            dec.set_norm(l, kind, gmm)
        if qkv_bias:
            bias = (rng.standard_normal(hq + 2 * hkv) * 0.5).astype(np.float16)
            biases[l] = bias.astype(np.float32)
            dec.set_qkv_bias(l, bias)
    p = nibbles(cfg["vocab"] * D // 2)
    s = rng.uniform(0.005, 0.02, cfg["vocab"] * (D // g)).astype(np.float16)
    linears[("lm_head",)] = (p, s)
    dec.set_linear(0, "lm_head", p, s, cfg["vocab"], D)
    gmm = rng.uniform(0.5, 1.5, D).astype(np.float32)
    norms[("final",)] = gmm
    dec.set_norm(0, "final", gmm)
    emb = rng.standard_normal((cfg["vocab"], D)) * emb_scale
    if symmetric:  # rows of different magnitude: a row factor applied to the wrong row is then off by 2x or more
        emb *= (2.0 ** (np.arange(cfg["vocab"]) % 4))[:, None]
    emb = emb.astype(np.float16)
    dec.set_embedding(emb)
    dec.finalize()
    ref = RefDecoder(cfg, linears, norms, emb, kv_i8=kv_dtype == "i8", biases=biases)
    return dec, ref


@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_steps_match_numpy(use_graph):
    import torch

    assert torch.cuda.is_available()
    rng = np.random.default_rng(4000)
    cfg = dict(CFG)
    dec, ref = _build(rng, cfg)
    B, prefill = 3, 133  # prefill crosses a 128-position chunk and is not a multiple of 8
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = np.array([5, 17, 300], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    for step in range(6):
        dec.run(1, use_graph=use_graph)
        got_logits = dec.logits()
        got_tok = dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        scale = np.abs(exp_logits).max()
        err = np.abs(got_logits - exp_logits).max() / scale
        assert err < LOGIT_TOL, (step, err)
        # the greedy pick is the LAST maximal logit of the GPU's own logits (exact rule)
        for b in range(B):
            row = got_logits[b]
            assert got_tok[b] == np.flatnonzero(row == row.max())[-1]
        cur = got_tok.copy()  # teacher-force the restatement with the GPU's picks


@pytest.mark.parametrize("kv_dtype", ["f16", "i8"])
@pytest.mark.parametrize("heads", [(3, 3), (6, 2), (4, 1)], ids=["group1", "group3", "group4"])
def test_query_heads_per_kv_head(heads, kv_dtype):
    """1, 3 and 4 query heads per kv head (kv_h = q_h / groups, runner/linear.rs:552-646): the other tests here run 2."""
    rng = np.random.default_rng(4500 + 10 * heads[0] + heads[1])
    cfg = dict(CFG, n_heads=heads[0], n_kv_heads=heads[1])
    dec, ref = _build(rng, cfg, kv_dtype=kv_dtype, symmetric=True)
    B, prefill = 3, 141
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = np.array([5, 17, 300], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    for step in range(3):
        dec.run(1, use_graph=bool(step & 1))
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        err = np.abs(got_logits - exp_logits).max() / np.abs(exp_logits).max()
        assert err < LOGIT_TOL, (step, err)
        cur = got_tok.copy()


@pytest.mark.parametrize("seed", range(12))
def test_random_model_shapes_match_numpy(seed):
    """Seeded random shapes (widths that fold the norms and widths that do not, 1..4 kv heads with 1..4 query heads each,
    K-split and unsplit projections, 1..8 sequences, either cache type, any prefill) against the checker, eager and
    replayed."""
    rng = np.random.default_rng(4600 + seed)
    n_kv = int(rng.integers(1, 5))
    group = int(rng.integers(1, 5))
    B = int(rng.integers(1, 9))
    cfg = dict(CFG, d_model=int(rng.choice([256, 384, 512, 768, 1024, 1536])), n_heads=n_kv * group, n_kv_heads=n_kv,
               d_ff=int(rng.choice([256, 384, 512, 1024, 2048, 4608])), vocab=int(rng.choice([320, 512, 1000])),
               max_batch=B, max_ctx=384)
    kv_dtype = "i8" if rng.integers(0, 2) else "f16"
    prefill = int(rng.integers(0, 300))
    dec, ref = _build(rng, cfg, kv_dtype=kv_dtype, symmetric=True)
    if prefill:
        for l in range(cfg["n_layers"]):
            k = rng.standard_normal((B, prefill, n_kv, cfg["head_dim"])).astype(np.float16)
            v = rng.standard_normal((B, prefill, n_kv, cfg["head_dim"])).astype(np.float16)
            dec.set_kv(l, k, v)
            ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = rng.integers(0, cfg["vocab"], B).astype(np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    for step in range(3):
        dec.run(1, use_graph=bool(step & 1))
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        err = np.abs(got_logits - exp_logits).max() / np.abs(exp_logits).max()
        assert err < LOGIT_TOL, (cfg, kv_dtype, prefill, step, err)
        cur = got_tok.copy()
    dec.close()


@pytest.mark.parametrize("kv_dtype", ["f16", "i8"])
def test_long_context_matches_numpy(kv_dtype):
    """4 230 cached positions = 34 chunks of 128: more than the chunk merge takes in its one-pass form (32), so the
    general merge runs, against the checker; the attention output of the last layer is also held to a float64 softmax
    over the cache rows the GPU holds."""
    import math

    rng = np.random.default_rng(4300)
    cfg = dict(CFG, max_ctx=4352, max_batch=2)
    dec, ref = _build(rng, cfg, kv_dtype=kv_dtype, symmetric=True)
    B, prefill = 2, 4230
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = np.array([7, 201], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    nh, nkv, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    for step in range(2):
        dec.run(1, use_graph=bool(step))
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        err = np.abs(got_logits - exp_logits).max() / np.abs(exp_logits).max()
        assert err < LOGIT_TOL, (step, err)
        # the last layer's attention from the GPU's own rotated q against the checker's cache of that layer (which
        # holds what the int8 mode reads back), in float64
        qkv, ao = dec.activation("qkv"), dec.activation("attn_out")
        L = cfg["n_layers"] - 1
        for b in range(B):
            q = qkv[b][: nh * hd].reshape(nh, hd).astype(np.float64)
            kc, vc = ref.kc[L][b].astype(np.float64), ref.vc[L][b].astype(np.float64)
            for h in range(nh):
                sc = kc[:, h // (nh // nkv), :] @ q[h] / math.sqrt(hd)
                pr = np.exp(sc - sc.max())
                want = (pr / pr.sum()) @ vc[:, h // (nh // nkv), :]
                got = ao[b].reshape(nh, hd)[h]
                assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max() + 1e-3, (step, b, h)
        cur = got_tok.copy()


@pytest.mark.parametrize("v_mag", [1e-3, 1e-4])
@pytest.mark.parametrize("use_graph", [False, True])
def test_int8_cache_with_small_values(v_mag, use_graph):
    """V rows of absmax 1e-3 .. 1e-4 in the int8 cache (cached rows and the appended one): the per-row scale absmax / 127
    is then 1e-5 .. 1e-6, far below fp16's normal range, and must not be lost where it meets the softmax weights.  The
    last layer's attention output against a float64 softmax over the checker's cache (dequantised q * scale in f32, as
    runner/kv_cache.rs:65-79 reads it back), relative to the output's own magnitude."""
    import math

    rng = np.random.default_rng(4700 + int(-math.log10(v_mag)))
    cfg = dict(CFG)
    dec, ref = _build(rng, cfg, kv_dtype="i8", symmetric=True, v_mul=v_mag)
    B, prefill = 2, 141
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = (rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])) * v_mag).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = np.array([9, 33], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    nh, nkv, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    for step in range(2):
        dec.run(1, use_graph=use_graph)
        ref.step(cur, prefill + step)
        qkv, ao = dec.activation("qkv"), dec.activation("attn_out")
        L = cfg["n_layers"] - 1
        for b in range(B):
            q = qkv[b][: nh * hd].reshape(nh, hd).astype(np.float64)
            kc, vc = ref.kc[L][b].astype(np.float64), ref.vc[L][b].astype(np.float64)
            assert np.abs(vc).max() < 20 * v_mag
            for h in range(nh):
                sc = kc[:, h // (nh // nkv), :] @ q[h] / math.sqrt(hd)
                pr = np.exp(sc - sc.max())
                want = (pr / pr.sum()) @ vc[:, h // (nh // nkv), :]
                got = ao[b].reshape(nh, hd)[h]
                assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max(), (step, b, h, np.abs(got - want).max(), np.abs(want).max())
        cur = dec.tokens(step, 1)[0].copy()


@pytest.mark.parametrize("kv_dtype,heads", [("f16", (4, 2, 128)), ("i8", (4, 2, 128)), ("f16", (8, 1, 64)), ("f16", (4, 4, 32)),
                                            ("f16", (12, 4, 96))],
                         ids=["f16-4q2kv-hd128", "i8-4q2kv-hd128", "f16-8q1kv-hd64", "f16-4q4kv-hd32", "f16-12q4kv-hd96"])
@pytest.mark.parametrize("prefill", [5, 127, 128, 133, 250])
def test_fused_attention_equals_the_separate_rope_append(prefill, kv_dtype, heads):
    """Rotary embedding and cache append inside the attention kernel against the separate rope_append launch in front
    of it: same arithmetic, so tokens, logits, the attention output, the rotated q and the appended cache rows must be
    identical bit for bit.  The prefills put the current position at the start, the end and the middle of a
    128-position chunk and leave chunks unused.  With the int8 cache the appended row's scales span all kv heads, which
    every workgroup that appends works out for itself.  Head shapes other than the first run the general attention
    kernel, whose fused form patches the new row into the 16-position key block that holds it (fp16 cache only)."""
    import ctypes as C

    from yscv_amd.capi import lib

    nh, nkv, hd = heads
    rng = np.random.default_rng(4100 + prefill)
    cfg = dict(CFG, n_heads=nh, n_kv_heads=nkv, head_dim=hd)
    dec, _ = _build(rng, cfg, kv_dtype=kv_dtype)
    B, steps = 3, 5
    kv = []
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        kv.append((k, v))
    tokens = np.array([9, 130, 511], np.int32)
    got = {}
    for fused in (1, 0):
        lib().decoder_debug_set_fused_attention(dec._h, C.c_int32(fused))
        for l, (k, v) in enumerate(kv):
            dec.set_kv(l, k, v)
        dec.reset(tokens, prefill)
        trace = []
        for step in range(steps):
            dec.run(1, use_graph=bool(step & 1))
            trace.append((dec.logits().copy(), dec.activation("attn_out").copy(), dec.activation("qkv").copy()))
        rows = [dec.get_kv(l, B, prefill, steps) for l in range(cfg["n_layers"])]
        got[fused] = (dec.tokens(0, steps).copy(), trace, rows)
    lib().decoder_debug_set_fused_attention(dec._h, C.c_int32(1))
    assert np.array_equal(got[1][0], got[0][0])
    for step in range(steps):
        for a, b_, name in zip(got[1][1][step], got[0][1][step], ("logits", "attention output", "qkv")):
            assert np.array_equal(a, b_), (step, name, np.abs(a - b_).max())
    for l in range(cfg["n_layers"]):
        for a, b_, name in zip(got[1][2][l], got[0][2][l], ("k", "v")):
            assert np.array_equal(a, b_), ("appended rows", l, name, np.argwhere(a != b_)[:8].tolist())


@pytest.mark.parametrize("d_ff,emb_scale,d_model,B", [
    (512, 1.0, 512, 3), (6144, 1.0, 512, 3), (512, 2.0 ** -10, 512, 3), (6144, 2.0 ** -10, 512, 3), (512, 2.0 ** 9, 512, 3),
    (6144, 1.0, 1024, 6), (1024, 1.0, 1024, 8), (6144, 1.0, 2048, 12), (2048, 1.0, 2048, 16)],
    ids=["d_ff512", "d_ff6144", "d_ff512-embedding-2^-10", "d_ff6144-embedding-2^-10", "d_ff512-embedding-2^9",
         "d_model1024-batch6-d_ff6144", "d_model1024-batch8", "d_model2048-batch12-d_ff6144", "d_model2048-batch16"])
def test_folded_norm_agrees_with_rmsnorm_launches(d_ff, emb_scale, d_model, B):
    """Every RMSNorm folded into the projections around it (unnormalised fp16 activations + per-row sums of squares,
    row factor applied to the projection's sums) against RMSNorm as a launch of its own: the same product with one
    fp16 rounding in a different place, so logits agree to a few fp16 ulps of the activations (the embedding rows differ
    in magnitude by up to 8x, so a row factor that reached the wrong row would be off by far more) and the normalised
    activations the consumer saw agree with RMSNorm of the residual.  d_ff 512 updates the residual inside the projection
    kernel, 6144 through the second pass of a K split.  (Widths that are no multiple of 512, like the 384 of the other
    tests here, keep RMSNorm as a launch of its own.)  The unnormalised activations carry a power of two per row taken
    from the norm before: with an embedding of 1e-3 the first residual update raises a row's rms a thousandfold within
    one kernel, with one of 512 the rows stay large throughout -- fp16 holds both.  Batches of 6 .. 16 rows run the two- and
    four-accumulator forms of the projection kernel (one row factor per accumulator)."""
    import ctypes as C

    from oracle import decoder_ref as R
    from yscv_amd.capi import lib

    rng = np.random.default_rng(4700 + d_ff)
    cfg = dict(CFG, d_ff=d_ff, d_model=d_model, max_batch=B)
    dec, ref = _build(rng, cfg, emb_scale=emb_scale, symmetric=True)
    prefill, steps = 70, 4
    kv = []
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        kv.append((k, v))
    tokens = (np.array([4, 99, 301], np.int32)[np.arange(B) % 3] + 7 * (np.arange(B, dtype=np.int32) // 3)) % cfg["vocab"]
    for l, (k, v) in enumerate(kv):
        dec.set_kv(l, k, v)
    # both forms run every step from the same tokens and the same cache (the rows the first appends are overwritten by
    # the second, whose picks feed the next step)
    cur, differed = tokens.copy(), False
    for step in range(steps):
        out = {}
        for fold in (1, 0):
            lib().decoder_debug_set_folded_norm(dec._h, C.c_int32(fold))
            dec.reset(cur, prefill + step)
            dec.run(1, use_graph=bool(step & 1))
            normed, resid = dec.activation("normed"), dec.activation("residual")
            want = R.rmsnorm(resid, ref.norms[("final",)], cfg["rms_eps"])
            assert np.abs(normed - want).max() <= 2.0 ** -9 * np.abs(want).max() + 1e-6, (fold, step)
            out[fold] = (dec.logits().copy(), dec.tokens(0, 1)[0].copy())
        a, b_ = out[1][0], out[0][0]
        for row in range(B):
            err = np.abs(a[row] - b_[row]).max() / np.abs(b_[row]).max()
            # two fp16 pipelines that round at different points: up to 6e-3 of a row's largest logit seen here
            assert err <= 1e-2, (step, row, err)
        differed = differed or np.abs(a - b_).max() > 0
        cur = out[0][1]
    lib().decoder_debug_set_folded_norm(dec._h, C.c_int32(1))
    assert differed  # the two forms round at different points: identical logits would mean the switch did nothing


@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_with_int8_kv_cache_matches_numpy(use_graph):
    """--kv-dtype i8 (apps/llm-bench/src/main.rs:232-265; KvCache I8 storage, kv_cache.rs:45-79): rows quantised on
    append with one scale per position over all kv heads, attention over q * scale, against the checker in the same
    mode.  The cache read back from the GPU holds exactly the checker's rows up to the rounding of the new keys."""
    import torch

    import yscv_amd

    assert torch.cuda.is_available()
    rng = np.random.default_rng(4300)
    cfg = dict(CFG)
    dec, ref = _build(rng, cfg, kv_dtype="i8")
    B, prefill = 3, 133
    for l in range(cfg["n_layers"]):
        k = (rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])) * 1.7).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
        gk, gv = dec.get_kv(l, B, 0, prefill)   # q * scale narrowed to fp16
        for b in range(B):
            assert np.abs(gk[b].astype(np.float32) - ref.kc[l][b]).max() <= 2.0 ** -10 * np.abs(ref.kc[l][b]).max()
            assert np.abs(gv[b].astype(np.float32) - ref.vc[l][b]).max() <= 2.0 ** -10 * np.abs(ref.vc[l][b]).max()
    tokens = np.array([5, 17, 300], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    for step in range(6):
        dec.run(1, use_graph=use_graph)
        got_logits = dec.logits()
        got_tok = dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        err = np.abs(got_logits - exp_logits).max() / np.abs(exp_logits).max()
        assert err < LOGIT_TOL, (step, err)
        for b in range(B):
            row = got_logits[b]
            assert got_tok[b] == np.flatnonzero(row == row.max())[-1]
        cur = got_tok.copy()
    # appended rows: the GPU's cache against the checker's (a one-step difference of a quantised value at most, where
    # sincosf and numpy disagree in the last bit of a rotated key)
    L = cfg["n_layers"] - 1
    gk, gv = dec.get_kv(L, B, prefill, 6)
    for b in range(B):
        rk, rv = ref.kc[L][b][prefill:], ref.vc[L][b][prefill:]
        step_k = np.abs(rk).reshape(6, -1).max(1) / 127.0
        assert (np.abs(gk[b].astype(np.float32) - rk).reshape(6, -1).max(1) <= 1.01 * step_k + 2.0 ** -10 * np.abs(rk).max()).all()
        step_v = np.abs(rv).reshape(6, -1).max(1) / 127.0
        assert (np.abs(gv[b].astype(np.float32) - rv).reshape(6, -1).max(1) <= 1.01 * step_v + 2.0 ** -10 * np.abs(rv).max()).all()
    # the single-launch kernel reads an fp16 cache only
    dec.reset(tokens[:1], prefill)
    with pytest.raises(yscv_amd.YscvHipError, match="fp16 KV cache only"):
        dec.run(1, persistent=True)


def test_graph_replay_equals_eager():
    """Several graph replays with eager work in between reproduce the eager token stream."""
    import torch

    rng = np.random.default_rng(4001)
    cfg = dict(CFG)
    dec, _ = _build(rng, cfg)
    tokens = np.array([1, 2, 3], np.int32)
    dec.reset(tokens, 0)
    dec.run(8, use_graph=False)
    eager = dec.tokens(0, 8)
    eager_logits = dec.logits()
    for _ in range(3):
        dec.reset(tokens, 0)
        dec.run(3, use_graph=True)
        _ = torch.ones(10, device="cuda").sum().item()  # unrelated eager work between replays
        dec.run(5, use_graph=True)
        assert np.array_equal(dec.tokens(0, 8), eager)
        assert np.array_equal(dec.logits(), eager_logits)


def test_cache_overflow_is_an_error():
    import yscv_amd

    rng = np.random.default_rng(4002)
    cfg = dict(CFG)
    dec, _ = _build(rng, cfg)
    dec.reset(np.array([1], np.int32), cfg["max_ctx"] - 2)
    dec.run(2)
    with pytest.raises(yscv_amd.YscvHipError):
        dec.run(1)


# ---- single-launch (persistent) decode path ---------------------------------------------------------------
# per-wave k slice = K / 4: K = 2048 -> two 256-k tiles (one full record), K = 3072 -> three tiles (full + single record)
PCFG = dict(n_layers=2, d_model=2048, n_heads=16, n_kv_heads=4, head_dim=128, d_ff=3072, vocab=1000, group_size=32,
            max_batch=2, max_ctx=512, max_steps=32, rope_theta=10000.0, rms_eps=1e-5)


def _prefill(rng, dec, ref, cfg, B, prefill):
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((B, prefill, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        dec.set_kv(l, k, v)
        if ref is not None:
            ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))


def test_persistent_decode_at_34_context_chunks():
    """The single-launch kernel over 4 230 cached positions (each workgroup takes several attention items and several
    merge heads): against the checker, and against the multi-kernel path from the same state."""
    rng = np.random.default_rng(4400)
    cfg = dict(PCFG, max_ctx=4352)
    dec, ref = _build(rng, cfg, symmetric=True)
    prefill = 4230
    _prefill(rng, dec, ref, cfg, 1, prefill)
    tokens = np.array([7], np.int32)
    cur = tokens.copy()
    for step in range(2):
        dec.reset(cur, prefill + step)
        dec.run(1, use_graph=True)
        graph_logits = dec.logits()[0].copy()
        dec.reset(cur, prefill + step)
        dec.run(1, persistent=True)
        got, tok = dec.logits()[0].copy(), dec.tokens(0, 1)[0]
        exp = ref.step(cur, prefill + step)[0]
        assert np.abs(got - exp).max() / np.abs(exp).max() < LOGIT_TOL, step
        assert np.abs(got - graph_logits).max() / np.abs(graph_logits).max() < 5e-3, step
        cur = tok.copy()


@pytest.mark.parametrize("prefill", [0, 133, 300])
def test_persistent_decode_matches_numpy_and_graph_path(prefill):
    import torch

    assert torch.cuda.is_available()
    rng = np.random.default_rng(4100 + prefill)
    cfg = dict(PCFG)
    dec, ref = _build(rng, cfg)
    _prefill(rng, dec, ref, cfg, 1, prefill)
    tokens = np.array([7], np.int32)
    dec.reset(tokens, prefill)
    cur = tokens.copy()
    for step in range(5):
        dec.run(1, persistent=True)
        got_logits = dec.logits()
        got_tok = dec.tokens(step, 1)[0]
        exp_logits = ref.step(cur, prefill + step)
        err = np.abs(got_logits - exp_logits).max() / np.abs(exp_logits).max()
        assert err < LOGIT_TOL, (step, err)
        row = got_logits[0]
        assert got_tok[0] == np.flatnonzero(row == row.max())[-1]
        cur = got_tok.copy()
    # several steps inside one launch reproduce the step-by-step token stream, and so does the graph path
    first = dec.tokens(0, 5)[:, 0].copy()
    logits5 = dec.logits().copy()
    dec.reset(tokens, prefill)
    dec.run(5, persistent=True)
    assert np.array_equal(dec.tokens(0, 5)[:, 0], first)
    assert np.abs(dec.logits() - logits5).max() <= 1e-5 * np.abs(logits5).max()
    dec.reset(tokens, prefill)
    dec.run(5, use_graph=True)
    graph_logits = dec.logits()
    assert np.array_equal(dec.tokens(0, 5)[:, 0], first)
    assert np.abs(graph_logits - logits5).max() / np.abs(logits5).max() < 5e-3


def test_single_launch_tags_wrap_around_cleanly():
    """The 24-bit tags of the single-launch path: runs that straddle the end of the tag space (the host clears the
    exchange buffers and restarts the count) give the same tokens and logits as a run far from it."""
    import ctypes as C

    from yscv_amd import lib

    rng = np.random.default_rng(4400)
    cfg = dict(PCFG)
    dec, _ = _build(rng, cfg)
    tokens = np.array([9], np.int32)
    dec.reset(tokens, 0)
    dec.run(12, persistent=True)
    want_tok, want_logits = dec.tokens(0, 12)[:, 0].copy(), dec.logits().copy()
    per_step = cfg["n_layers"] + 2
    last_epoch = (1 << 24) // per_step
    for back in (30, 13, 12, 5, 2, 1):      # the 12 steps start `back` epochs before the tag space ends
        lib().decoder_debug_set_tag_epoch(dec._h, C.c_uint32(last_epoch - back))
        dec.reset(tokens, 0)
        dec.run(5, persistent=True)         # two launches, so that the wrap may fall between them or inside the window
        dec.run(7, persistent=True)
        assert np.array_equal(dec.tokens(0, 12)[:, 0], want_tok), back
        assert np.array_equal(dec.logits(), want_logits), back


@pytest.mark.parametrize("shape", ["graph", "single_launch"])
def test_generate_matches_device_greedy_and_stops_at_eos(shape):
    """generate() (generate.rs:58-118) with the decoder as the model: top_k = 1 reproduces the tokens the device picks
    greedily; an EOS token ends the loop without being stored; the sampling path runs with the default configuration.
    Two shapes: one only the multi-kernel path takes, and one (widths in multiples of 1024) that generate() runs on the
    single-launch kernel, one cooperative launch per prompt token."""
    import numpy as np

    from yscv_amd.decoder import Decoder

    cfg = dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=2, head_dim=128, d_ff=1024, vocab=320, group_size=32,
               max_batch=1, max_ctx=256, max_steps=64, rope_theta=10000.0, rms_eps=1e-5)
    if shape == "single_launch":
        cfg.update(d_model=1024, n_heads=8, n_kv_heads=2, d_ff=2048)
    dec = Decoder(**cfg)
    dec.init_random(seed=5)
    prompt = [7, 3, 11]
    assert dec.last_path() == -1
    got = dec.generate(prompt, max_tokens=12, top_k=1, top_p=1.0)
    assert dec.last_path() == (2 if shape == "single_launch" else 1)
    # the same through the device-side greedy loop: feed the prompt, then let the decoder run on its own picks
    dec.reset(np.array([prompt[0]], np.int32), 0)
    dec.run(1, auto=True)  # the path generate() takes: the fastest one the decoder has
    assert dec.last_path() == (2 if shape == "single_launch" else 1)
    for p, t in enumerate(prompt[1:], start=1):
        dec.reset(np.array([t], np.int32), p)
        dec.run(1, auto=True)
    first = int(dec.tokens(0, 1)[0, 0])
    dec.reset(np.array([first], np.int32), len(prompt))
    dec.run(11, auto=True)
    want = [first] + dec.tokens(0, 11)[:, 0].tolist()
    assert got.tolist() == want
    # EOS: the third generated token as EOS stops after two
    eos = int(got[2])
    if eos not in got[:2].tolist():
        short = dec.generate(prompt, max_tokens=12, top_k=1, top_p=1.0, eos_token_id=eos)
        assert short.tolist() == got[:2].tolist()
    # default configuration (top_k 50, top_p 0.9) with temperature and repetition penalty: valid tokens, reproducible
    a = dec.generate(prompt, max_tokens=8, temperature=0.8, repetition_penalty=1.3)
    b = dec.generate(prompt, max_tokens=8, temperature=0.8, repetition_penalty=1.3)
    assert a.tolist() == b.tolist() and len(a) == 8 and (a < cfg["vocab"]).all()
    dec.close()


# ---- the reference's own benchmark model, prompt pass, q / k / v bias ------------------------------------------------
# apps/llm-bench/COMPARISON.md:9-12: 24 layers, hidden 1024, 2 kv heads, head_dim 64 (16 query heads: eight per kv
# head), a 43-token prompt; the vocabulary and the FFN width are cut down to keep the numpy side short.
BENCH_MODEL = dict(n_layers=24, d_model=1024, n_heads=16, n_kv_heads=2, head_dim=64, d_ff=2816, vocab=2048, group_size=32,
                   max_batch=2, max_ctx=256, max_steps=16, rope_theta=1000000.0, rms_eps=1e-6)


def test_reference_benchmark_model_decodes_and_prefills():
    """head_dim 64 with eight query heads per kv head (the general attention kernel) at 24 layers: token-by-token feeding
    of a 43-token prompt against the checker, then the same prompt through yscv_hip_decoder_prefill: logits of the last
    prompt position, the cache rows of every position and the decode steps that follow agree with the fed run."""
    rng = np.random.default_rng(4800)
    cfg = dict(BENCH_MODEL)
    dec, ref = _build(rng, cfg, symmetric=True, qkv_bias=True)
    prompt = rng.integers(0, cfg["vocab"], 43).astype(np.int32)
    for p, t in enumerate(prompt):
        dec.reset(np.array([t], np.int32), p)
        dec.run(1, use_graph=bool(p & 1))
        exp = ref.step(np.array([t]), p)
        if p in (0, 1, 20, 42):
            err = np.abs(dec.logits() - exp).max() / np.abs(exp).max()
            assert err < LOGIT_TOL, (p, err)
    fed_logits = dec.logits().copy()
    fed_kv = [dec.get_kv(l, 1, 0, 43) for l in (0, 11, 23)]
    fed_tok = int(dec.tokens(0, 1)[0, 0])
    # continue for three steps on the device's own picks: the trajectory the prefilled decoder must repeat
    dec.run(3, use_graph=True)
    fed_next = dec.tokens(0, 4)[:, 0].tolist()
    fed_logits3 = dec.logits().copy()

    dec2, _ = _build(np.random.default_rng(4800), cfg, symmetric=True, qkv_bias=True)  # same seed: the same model
    dec2.prefill(prompt)
    got = dec2.logits()
    # The prompt pass runs the projections on the MFMA GEMM, which folds the group scale into an fp16 weight (relative
    # 2^-11 per weight, 2e-4 of a projection's output) where the decode kernel applies it in f32; through 24 layers of a
    # random model that comes to about 1e-2 of max|logit| at the last position, so this depth is held to twice the bar
    # (the two-layer prompt tests below hold the bar itself)
    assert np.abs(got - exp).max() / np.abs(exp).max() < 2 * LOGIT_TOL
    between = np.abs(got - fed_logits).max() / np.abs(fed_logits).max()
    assert between < 2 * LOGIT_TOL, between
    assert int(dec2.tokens(0, 1)[0, 0]) == fed_tok or between > 1e-3
    for (fk, fv), l in zip(fed_kv, (0, 11, 23)):
        gk, gv = dec2.get_kv(l, 1, 0, 43)
        assert np.abs(gk.astype(np.float32) - fk.astype(np.float32)).max() <= 2e-2 * np.abs(fk.astype(np.float32)).max(), l
        assert np.abs(gv.astype(np.float32) - fv.astype(np.float32)).max() <= 2e-2 * np.abs(fv.astype(np.float32)).max(), l
    dec2.run(3, use_graph=True)
    if dec2.tokens(0, 4)[:, 0].tolist() == fed_next:  # the same trajectory: the same inputs at every step
        assert np.abs(dec2.logits() - fed_logits3).max() / np.abs(fed_logits3).max() < 2 * LOGIT_TOL
    dec.close()
    dec2.close()


@pytest.mark.parametrize("n_prompt,start,kv_dtype", [(1, 0, "f16"), (5, 0, "f16"), (16, 3, "f16"), (17, 0, "f16"), (130, 9, "f16"),
                                                     (1, 0, "i8"), (5, 2, "i8"), (17, 0, "i8"), (130, 9, "i8")])
def test_prefill_equals_feeding_at_toy_widths(n_prompt, start, kv_dtype):
    """Prompt lengths on both sides of the skinny / GEMM switch (16 rows) and across a 128-position attention chunk, at a
    start position other than 0 (a prompt appended to a cache that already holds positions): prefill against the
    checker fed token by token, head_dim 128.  With the int8 cache the pass quantises every appended row (scales over
    all kv heads of the position) and attends over what the cache returns, earlier positions included."""
    rng = np.random.default_rng(4900 + n_prompt)
    cfg = dict(CFG, max_batch=1, max_ctx=256)
    dec, ref = _build(rng, cfg, kv_dtype=kv_dtype, symmetric=True)
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((1, start, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        v = rng.standard_normal((1, start, cfg["n_kv_heads"], cfg["head_dim"])).astype(np.float16)
        if start:
            dec.set_kv(l, k, v)
            ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    for i, t in enumerate(prompt):
        exp = ref.step(np.array([t]), start + i)
    dec.prefill(prompt, start_pos=start)
    got = dec.logits()
    assert np.abs(got - exp).max() / np.abs(exp).max() < LOGIT_TOL
    row = got[0]
    assert int(dec.tokens(0, 1)[0, 0]) == np.flatnonzero(row == row.max())[-1]
    # the step after the prompt continues from the cache the prompt pass wrote
    nxt = dec.tokens(0, 1)[0].copy()
    dec.run(1, use_graph=True)
    exp2 = ref.step(nxt, start + n_prompt)
    assert np.abs(dec.logits() - exp2).max() / np.abs(exp2).max() < LOGIT_TOL
    dec.close()


@pytest.mark.parametrize("hd,nh,nkv,n_prompt,start", [
    (128, 4, 1, 150, 0),   # four query heads per kv head: the four waves of a workgroup are the four heads
    (64, 8, 1, 97, 5),     # eight per kv head: two workgroups per kv head; the prompt ends inside a 32-query range
    (64, 4, 2, 200, 0),    # two per kv head: two heads x two query ranges per workgroup
    (32, 4, 4, 161, 30),   # one per kv head: four query ranges per workgroup, the last one past the prompt's end
    (96, 12, 4, 70, 0),    # three per kv head (neither four nor two divides it): one head per workgroup; 96-wide rows
])
def test_prefill_of_long_prompts_across_head_shapes(hd, nh, nkv, n_prompt, start):
    """Prompts of 64 rows and more go through the attention kernel that shares a stage of K / V between the four waves
    of a workgroup; how heads and query ranges are spread over the waves depends on the heads per kv head.  Logits of
    the last prompt position (which, through the second layer's K / V, depend on the first layer's attention output at
    every position) against the checker fed token by token, and the cache the pass leaves behind through one more
    decode step."""
    rng = np.random.default_rng(5000 + hd + nh)
    cfg = dict(CFG, n_heads=nh, n_kv_heads=nkv, head_dim=hd, d_model=256, max_batch=1, max_ctx=256)
    dec, ref = _build(rng, cfg, symmetric=True)
    if start:
        for l in range(cfg["n_layers"]):
            k = rng.standard_normal((1, start, nkv, hd)).astype(np.float16)
            v = rng.standard_normal((1, start, nkv, hd)).astype(np.float16)
            dec.set_kv(l, k, v)
            ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    prompt = rng.integers(0, cfg["vocab"], n_prompt).astype(np.int32)
    for i, t in enumerate(prompt):
        exp = ref.step(np.array([t]), start + i)
    dec.prefill(prompt, start_pos=start)
    got = dec.logits()
    assert np.abs(got - exp).max() / np.abs(exp).max() < LOGIT_TOL
    # every cache row the pass wrote, first and second layer
    for l in range(cfg["n_layers"]):
        gk, gv = dec.get_kv(l, 1, 0, start + n_prompt)
        ek, ev = ref.kc[l][0], ref.vc[l][0]
        assert np.abs(gk.astype(np.float32) - ek).max() <= 1e-2 * np.abs(ek).max(), l
        assert np.abs(gv.astype(np.float32) - ev).max() <= 1e-2 * np.abs(ev).max(), l
    nxt = dec.tokens(0, 1)[0].copy()
    dec.run(1, use_graph=True)
    exp2 = ref.step(nxt, start + n_prompt)
    assert np.abs(dec.logits() - exp2).max() / np.abs(exp2).max() < LOGIT_TOL
    dec.close()


@pytest.mark.parametrize("kv_dtype,chunk", [("f16", 64), ("f16", 17), ("i8", 64), ("i8", 40)])
def test_prefill_in_several_passes(kv_dtype, chunk):
    """A prompt longer than yscv_hip_decoder_set_prefill_rows runs as several passes; every pass after the first starts
    at a position other than 0 and attends over the cache rows the earlier passes wrote (with the int8 cache: over what
    the cache returns for them).  150 tokens in passes of 64 / 17 / 40 rows -- the row counts of the passes straddle the
    kernel switches at 16 and 32 rows -- against the checker fed token by token, and against the one-pass result."""
    rng = np.random.default_rng(5200)
    cfg = dict(CFG, max_batch=1, max_ctx=256)
    dec, ref = _build(rng, cfg, kv_dtype=kv_dtype, symmetric=True)
    prompt = rng.integers(0, cfg["vocab"], 150).astype(np.int32)
    for i, t in enumerate(prompt):
        exp = ref.step(np.array([t]), i)
    dec.prefill(prompt)
    one_pass = dec.logits().copy()
    dec.set_prefill_rows(chunk)
    dec.prefill(prompt)
    got = dec.logits()
    assert np.abs(got - exp).max() / np.abs(exp).max() < LOGIT_TOL
    assert np.abs(got - one_pass).max() / np.abs(one_pass).max() < LOGIT_TOL
    for l in range(cfg["n_layers"]):
        gk, gv = dec.get_kv(l, 1, 0, 150)
        ek, ev = ref.kc[l][0], ref.vc[l][0]
        assert np.abs(gk.astype(np.float32) - ek).max() <= 1e-2 * np.abs(ek).max(), l
        assert np.abs(gv.astype(np.float32) - ev).max() <= 1e-2 * np.abs(ev).max(), l
    with pytest.raises(Exception, match="rows per prompt pass"):
        dec.set_prefill_rows(0)
    dec.close()

"""Decode loop at the widths the benchmark times (BASELINE configs[3]: d_model 4096, 32 query / 8 kv heads of 128,
SwiGLU 14336, vocab 32000, int4 group 32 with fp16 scales, fp16 KV cache at context 2048).

* Two layers of those widths against the numpy checker (oracle/decoder_ref.py, pinned by tests/test_oracle_decoder.py):
  the single-launch kernel at batch 1 and the multi-kernel path at batch 16, both starting beyond 2048 cached positions,
  so per-wave k slices of 1024 and 3584, the grid K split of the down projection, 17 attention chunks per head and a
  125-block LM head per workgroup are all exercised against an independent result.
* All 32 layers: the single-launch kernel against the multi-kernel path (tokens and logits), step by step and as one
  launch, and row 0 of a batch-16 step against the batch-1 step.
Tolerances: the logits are held to 1e-2 of max|logit| (the float bar of the int4 path) against TWO results of the
checker: f32 from the embedding row to the logits, which is what the reference's CPU path computes, and the same with
every activation rounded to fp16 where the GPU's multi-launch path stores fp16.  The GPU paths round at slightly
different points (the single-launch kernel and the folded norms keep some values in f32 longer, or round before the
norm's row factor is applied instead of after), so they sit as far from the f32 result as the rounded checker does
(1e-3 .. 4e-3 here), not closer to one than to the other.  With the int8 cache a key or value whose scaled magnitude
lies next to a rounding boundary takes the neighbouring int8 code as soon as its input differs in the last fp16 bit,
a step of 1/127 of the row's maximum: there the rounded checker itself is up to 1.6e-2 from the f32 one, and the bar
for the logits is 3e-2 (every stage-level check keeps its own, tighter bound).

Weights of the two-layer model are uniform over the nibbles 1..15, i.e. symmetric about the zero point 8.  Uniform
0..15 (what the benchmark's random init draws) has mean -0.5 after the zero point: with positive RMSNorm gains every
projection then adds a common offset of about -25 to all its outputs, q / k / v sit at |x| > 32 where one fp16 ulp is
0.03, and a one-ulp difference between two correct implementations moves an attention score by 0.1 and a softmax
weight by percents -- the end-to-end comparison against an independent implementation would measure that model's
conditioning, not the kernels.  The stage-level checks below (each GPU stage against the checker applied to the
GPU's own inputs) do not depend on conditioning, and the full-depth test keeps the benchmark's init.
"""
import numpy as np
import pytest

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]  # building two 7B-width layers and their checker takes a while

W7B = dict(d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ff=14336, vocab=32000, group_size=32,
           rope_theta=10000.0, rms_eps=1e-5)
PREFILL = 2051  # beyond 2048, not a multiple of 8 or 128


def _build_two_layers():
    from oracle.decoder_ref import RefDecoder
    from yscv_amd.decoder import Decoder

    rng = np.random.default_rng(7000)
    cfg = dict(W7B, n_layers=2, max_batch=16, max_ctx=2304, max_steps=16)
    D, hd, g = cfg["d_model"], cfg["head_dim"], cfg["group_size"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    shapes = {"q": (hq, D), "k": (hkv, D), "v": (hkv, D), "o": (D, hq), "gate": (ff, D), "up": (ff, D), "down": (D, ff)}
    dec = Decoder(**cfg)
    linears, norms = {}, {}

    def weight(n, k):
        nib = rng.integers(1, 16, (n * k // 2, 2), dtype=np.uint8)
        return nib[:, 0] | (nib[:, 1] << 4), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)

    for l in range(cfg["n_layers"]):
        for kind, (n, k) in shapes.items():
            linears[(l, kind)] = weight(n, k)
            dec.set_linear(l, kind, *linears[(l, kind)], n, k)
        for kind in ("attn", "ffn"):
            norms[(l, kind)] = rng.uniform(0.5, 1.5, D).astype(np.float32)
            dec.set_norm(l, kind, norms[(l, kind)])
    linears[("lm_head",)] = weight(cfg["vocab"], D)
    dec.set_linear(0, "lm_head", *linears[("lm_head",)], cfg["vocab"], D)
    norms[("final",)] = rng.uniform(0.5, 1.5, D).astype(np.float32)
    dec.set_norm(0, "final", norms[("final",)])
    emb = rng.standard_normal((cfg["vocab"], D)).astype(np.float16)
    dec.set_embedding(emb)
    dec.finalize()
    ref = RefDecoder(cfg, linears, norms, emb)
    ref.f32 = RefDecoder(cfg, linears, norms, emb, round_f16=False)
    B = cfg["max_batch"]
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
        ref.f32.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    return cfg, dec, ref, linears


@pytest.fixture(scope="module")
def two_layers():
    import torch

    assert torch.cuda.is_available()
    cfg, dec, ref, linears = _build_two_layers()
    yield cfg, dec, ref, linears
    dec.close()


def _check_rows(got_logits, got_tok, exp_logits, exp_f32, what, tol=1e-2):
    """Logits against the rounded and the f32 result of the checker; returns the worst row of each."""
    from oracle.decoder_ref import greedy_pick

    worst = [0.0, 0.0]
    for b in range(exp_logits.shape[0]):
        for i, exp in enumerate((exp_logits, exp_f32)):
            err = np.abs(got_logits[b] - exp[b]).max() / np.abs(exp[b]).max()
            assert err < tol, (what, "rounded" if i == 0 else "f32", b, err)
            worst[i] = max(worst[i], float(err))
        assert got_tok[b] == greedy_pick(got_logits[b]), (what, b)  # the exact rule, on the GPU's own logits
    return worst


def test_single_launch_batch1_at_7b_widths_matches_numpy(two_layers):
    cfg, dec, ref, _ = two_layers
    tokens = np.array([4321], np.int32)
    dec.reset(tokens, PREFILL)
    cur = tokens.copy()
    seen = []
    for step in range(3):
        dec.run(1, persistent=True)
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp, exp32 = ref.step(cur, PREFILL + step), ref.f32.step(cur, PREFILL + step)
        worst = _check_rows(got_logits, got_tok, exp, exp32, f"persistent step {step}")
        print(f"[7b widths, single launch] step {step}: rel err {worst[0]:.2e} (f32 checker {worst[1]:.2e})", flush=True)
        seen.append(int(got_tok[0]))
        cur = got_tok.copy()
    last = dec.logits().copy()
    # the same three steps inside one launch, and through the multi-kernel path (graph replay and eager)
    dec.reset(tokens, PREFILL)
    dec.run(3, persistent=True)
    assert dec.tokens(0, 3)[:, 0].tolist() == seen
    assert np.abs(dec.logits() - last).max() <= 1e-5 * np.abs(last).max()
    for use_graph in (True, False):
        dec.reset(tokens, PREFILL)
        dec.run(3, use_graph=use_graph)
        assert dec.tokens(0, 3)[:, 0].tolist() == seen
        assert np.abs(dec.logits() - last).max() / np.abs(last).max() < 5e-3


def _stage_checks(oracle, cfg, dec, ref, linears, pos, B):
    """Each stage of the last layer against the checker applied to the GPU's OWN inputs of that stage."""
    import math

    from gpu_util import int4_tolerances
    from oracle import decoder_ref as R

    nh, nkv, hd, D = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"], cfg["d_model"]
    L = cfg["n_layers"] - 1
    qkv, ao = dec.activation("qkv"), dec.activation("attn_out")
    resid, normed, logits = dec.activation("residual"), dec.activation("normed"), dec.logits()
    # attention: float64 softmax over the cache as the GPU holds it (the uploaded prefill + the rows it appended)
    worst_att = 0.0
    gk, gv = dec.get_kv(L, B, PREFILL, pos + 1 - PREFILL)
    for b in range(B):
        q = qkv[b][: nh * hd].reshape(nh, hd).astype(np.float64)
        kc, vc = ref.kc[L][b].astype(np.float64), ref.vc[L][b].astype(np.float64)
        kc[PREFILL:], vc[PREFILL:] = gk[b], gv[b]
        # the rows appended in this step are the rotated k and the v of this step's projection
        k_new = R.f16(R.rope(qkv[b][nh * hd:(nh + nkv) * hd].reshape(nkv, hd), pos, cfg["rope_theta"]))
        assert np.abs(gk[b][-1] - k_new).max() <= 2.0 ** -9 * np.abs(k_new).max()  # sincosf vs numpy: an fp16 ulp
        assert np.array_equal(gv[b][-1], qkv[b][(nh + nkv) * hd:].reshape(nkv, hd).astype(np.float16))
        want = np.zeros((nh, hd))
        for h in range(nh):
            s = kc[:, h // (nh // nkv), :] @ q[h] / math.sqrt(hd)
            p = np.exp(s - s.max())
            want[h] = (p / p.sum()) @ vc[:, h // (nh // nkv), :]
        err = np.abs(ao[b].reshape(nh, hd) - want).max() / np.abs(want).max()
        worst_att = max(worst_att, err)
        assert err < 2e-3, ("attention", b, err)  # fp16 weights and fp16 output: a few 2^-11
    # final RMSNorm of the residual stream (fp16 output)
    want = R.rmsnorm(resid, ref.norms[("final",)], cfg["rms_eps"])
    assert np.abs(normed - want).max() <= 2.0 ** -10 * np.abs(want).max() + 1e-6
    # LM head: the int4 projection of the GPU's own input, held to the bar of the int4 kernels, on sampled rows of W
    p, s16 = linears[("lm_head",)]
    cols = np.sort(np.random.default_rng(pos).choice(cfg["vocab"], 64, replace=False))
    g = cfg["group_size"]
    bs = p.reshape(cfg["vocab"], D // 2)[cols]
    ss = s16.reshape(cfg["vocab"], D // g)[cols].astype(np.float32)
    want = oracle.packed_int4_gemm_scalar(bs ^ 0x88, ss, normed, B, len(cols), D, g).reshape(B, len(cols))
    _, rel = int4_tolerances(logits[:, cols], want, D, normed)
    return worst_att, rel


def test_multi_kernel_batch16_at_7b_widths_matches_numpy(two_layers, oracle):
    cfg, dec, ref, linears = two_layers
    B = 16
    tokens = (np.arange(B, dtype=np.int32) * 1999 + 17) % cfg["vocab"]
    dec.reset(tokens, PREFILL)
    cur = tokens.copy()
    for step in range(2):
        dec.run(1, use_graph=True)
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp, exp32 = ref.step(cur, PREFILL + step), ref.f32.step(cur, PREFILL + step)
        worst = _check_rows(got_logits, got_tok, exp, exp32, f"batch 16 step {step}")
        att, lm = _stage_checks(oracle, cfg, dec, ref, linears, PREFILL + step, B)
        print(f"[7b widths, batch 16] step {step}: worst row rel err {worst[0]:.2e} (f32 checker {worst[1]:.2e}); stage level: attention {att:.1e}, "
              f"lm_head {lm:.1e}", flush=True)
        cur = got_tok.copy()
    # eager launches give the same stream as the graph replays
    graph_tok, graph_logits = dec.tokens(0, 2).copy(), dec.logits().copy()
    dec.reset(tokens, PREFILL)
    dec.run(2, use_graph=False)
    assert np.array_equal(dec.tokens(0, 2), graph_tok)
    assert np.array_equal(dec.logits(), graph_logits)


def test_multi_kernel_int8_cache_at_7b_widths_matches_numpy(two_layers):
    """The int8 KV cache (--kv-dtype i8) at the 7B-shape widths, four sequences beyond 2048 cached positions, against
    the checker in its int8 mode; the weights are the fixture's."""
    from oracle.decoder_ref import RefDecoder
    from yscv_amd.decoder import Decoder

    cfg, _, ref16, linears = two_layers
    cfg = dict(cfg, max_batch=4)
    D, hd = cfg["d_model"], cfg["head_dim"]
    hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
    shapes = {"q": (hq, D), "k": (hkv, D), "v": (hkv, D), "o": (D, hq), "gate": (ff, D), "up": (ff, D), "down": (D, ff)}
    dec = Decoder(kv_dtype="i8", **cfg)
    for (key, (p, s)) in linears.items():
        if key == ("lm_head",):
            dec.set_linear(0, "lm_head", p, s, cfg["vocab"], D)
        else:
            dec.set_linear(key[0], key[1], p, s, *shapes[key[1]])
    for key, g in ref16.norms.items():
        dec.set_norm(0 if key == ("final",) else key[0], "final" if key == ("final",) else key[1], g)
    emb16 = ref16.emb.astype(np.float16)
    dec.set_embedding(emb16)
    dec.finalize()
    ref = RefDecoder(cfg, linears, ref16.norms, emb16, kv_i8=True)
    ref32 = RefDecoder(cfg, linears, ref16.norms, emb16, kv_i8=True, round_f16=False)
    rng = np.random.default_rng(7100)
    B = cfg["max_batch"]
    for l in range(cfg["n_layers"]):
        k = (rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32) * 1.5).astype(np.float16)
        v = rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
        ref32.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    tokens = np.array([11, 2222, 13333, 31999], np.int32)
    dec.reset(tokens, PREFILL)
    cur = tokens.copy()
    for step in range(3):
        dec.run(1, use_graph=True)
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp, exp32 = ref.step(cur, PREFILL + step), ref32.step(cur, PREFILL + step)
        worst = _check_rows(got_logits, got_tok, exp, exp32, f"int8 cache step {step}", tol=3e-2)
        print(f"[7b widths, int8 cache] step {step}: worst row rel err {worst[0]:.2e} (f32 checker {worst[1]:.2e})", flush=True)
        cur = got_tok.copy()
    dec.close()


@pytest.mark.parametrize("nibbles", [(0, 15), (1, 15)], ids=["benchmark-init", "symmetric-init"])
def test_full_depth_single_launch_agrees_with_multi_kernel_path(nibbles):
    """32 layers, random init, cache filled to beyond 2000 positions: 16 steps.  The benchmark's init (nibbles 0..15)
    yields a degenerate model that keeps picking one token; nibbles 1..15 give a token stream that varies."""
    import torch

    from oracle.decoder_ref import greedy_pick
    from yscv_amd.decoder import Decoder

    assert torch.cuda.is_available()
    cfg = dict(W7B, n_layers=32, max_batch=16, max_ctx=2176, max_steps=32)
    dec = Decoder(**cfg)
    dec.init_random(seed=11, nibbles=nibbles)
    dec.fill_kv_random(seed=12)
    start, first, steps = 2040, 777, 16  # crosses position 2048 (a new attention chunk) on the way
    cur = first
    toks, worst = [], 0.0
    # two implementations with different fp16 rounding points, 32 layers deep, as a fraction of max|logit|: observed
    # 1.5e-4 on the degenerate benchmark init and 1.7e-2 on the symmetric one, where rounding noise is amplified layer
    # by layer (the comparisons against the checker above run at two layers for that reason)
    bound = 2e-2 if nibbles == (0, 15) else 5e-2
    for s in range(steps):
        # the multi-kernel path first, then the single launch, so that the cache keeps the latter's k / v
        dec.reset(np.array([cur], np.int32), start + s)
        dec.run(1, use_graph=True)
        lg, tg = dec.logits()[0], int(dec.tokens(0, 1)[0, 0])
        dec.reset(np.array([cur], np.int32), start + s)
        dec.run(1, persistent=True)
        lp, tp = dec.logits()[0], int(dec.tokens(0, 1)[0, 0])
        assert np.isfinite(lp).all() and np.isfinite(lg).all()
        diff = np.abs(lp - lg).max()
        worst = max(worst, diff / np.abs(lg).max())
        assert diff / np.abs(lg).max() < bound, (s, diff / np.abs(lg).max())
        assert tp == greedy_pick(lp) and tg == greedy_pick(lg)
        if tp != tg:  # only a near tie may flip the pick
            assert abs(lg[tp] - lg[tg]) <= 2 * diff, (s, tp, tg)
        toks.append(tp)
        cur = tp
    print(f"[32 layers, nibbles {nibbles}] single launch vs multi-kernel: worst rel logit diff {worst:.2e}, tokens {toks}", flush=True)
    if nibbles == (1, 15):
        assert len(set(toks)) > 4
    last = dec.logits()[0].copy()
    # the same 16 steps as ONE launch reproduce the step-by-step stream exactly
    dec.reset(np.array([first], np.int32), start)
    dec.run(steps, persistent=True)
    assert dec.tokens(0, steps)[:, 0].tolist() == toks
    assert np.abs(dec.logits()[0] - last).max() <= 1e-5 * np.abs(last).max()
    # batch 16: row 0 shares token and cache with the batch-1 run, every row obeys the pick rule
    B = 16
    tokens = np.array([first] + [(first + 37 * b) % cfg["vocab"] for b in range(1, B)], np.int32)
    dec.reset(np.array([first], np.int32), start)
    dec.run(1, use_graph=True)
    one = dec.logits()[0].copy()
    dec.reset(tokens, start)
    dec.run(1, use_graph=True)
    many = dec.logits()
    assert np.isfinite(many).all()
    assert np.abs(many[0] - one).max() / np.abs(one).max() < bound
    picks = dec.tokens(0, 1)[0]
    for b in range(B):
        assert picks[b] == greedy_pick(many[b])
    assert len({int(p) for p in picks}) > 1  # different rows, different inputs
    # no path has a result that depends on timing (no atomics on shared sums, fixed merge orders): the same state gives
    # the same bits, three times over 24 steps
    for persistent, b in ((True, 1), (False, 1), (False, B)):
        want = None
        for rep in range(3):
            dec.reset(tokens[:b], start)
            dec.run(24, use_graph=True, persistent=persistent)
            got = (dec.tokens(0, 24).copy(), dec.logits().copy())
            if want is None:
                want = got
            else:
                assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), (persistent, b, rep)
    dec.close()


def test_graph_is_recaptured_after_weights_are_reloaded():
    """A captured step holds device addresses of the weights: reloading them must not replay the old graph."""
    from yscv_amd.decoder import Decoder

    cfg = dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=2, head_dim=128, d_ff=1024, vocab=320, group_size=32,
               max_batch=2, max_ctx=256, max_steps=16, rope_theta=10000.0, rms_eps=1e-5)
    dec = Decoder(**cfg)
    tokens = np.array([3, 9], np.int32)
    streams = {}
    for seed in (21, 22, 21):
        dec.init_random(seed=seed)  # frees and recreates every weight
        dec.reset(tokens, 0)
        dec.run(6, use_graph=True)
        g_tok, g_logits = dec.tokens(0, 6).copy(), dec.logits().copy()
        dec.reset(tokens, 0)
        dec.run(6, use_graph=False)
        assert np.array_equal(dec.tokens(0, 6), g_tok), seed
        assert np.array_equal(dec.logits(), g_logits), seed
        if seed in streams:
            assert np.array_equal(streams[seed], g_logits)
        streams[seed] = g_logits
    assert not np.array_equal(streams[21], streams[22])
    dec.close()


def test_prefill_of_2048_tokens_equals_feeding_at_7b_widths(two_layers):
    """yscv_hip_decoder_prefill at the true widths: 2048 prompt tokens in one pass (every projection as an M = 2048 MFMA
    GEMM, causal attention over 2048 positions) against the same prompt fed through the decode step position by
    position: logits of the last position, the greedy pick, cache rows at the start, middle and end of the prompt, and
    the decode steps that follow.  The two differ where the GEMM folds the group scale into fp16 weights and the decode
    kernel applies it in fp32 (relative 2^-11 per weight), inside the decoder bar of 1e-2."""
    import time

    import torch

    cfg, dec, _, _ = two_layers
    L, n = cfg["n_layers"], 2048
    saved = [dec.get_kv(l, 1, 0, n + 8) for l in range(L)]  # batch row 0 is overwritten: put it back afterwards
    rng = np.random.default_rng(7100)
    prompt = rng.integers(0, cfg["vocab"], n).astype(np.int32)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for p, t in enumerate(prompt):
        dec.reset(np.array([t], np.int32), p)
        dec.run(1, use_graph=True)
    fed_logits = dec.logits().copy()
    t_fed = time.perf_counter() - t0
    fed_tok = int(dec.tokens(0, 1)[0, 0])
    fed_kv = [dec.get_kv(l, 1, 0, n) for l in range(L)]
    dec.run(2, use_graph=True)
    fed_after = dec.logits().copy()
    for l in range(L):  # scrub the rows, so that the prompt pass must write them itself
        z = np.zeros((1, n + 8, cfg["n_kv_heads"], cfg["head_dim"]), np.float16)
        dec.set_kv(l, z, z)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.prefill(prompt)
    got = dec.logits()
    t_pre = time.perf_counter() - t0
    print(f"[7b widths, 2 layers] 2048-token prompt: fed {t_fed * 1e3:.0f} ms, one pass {t_pre * 1e3:.1f} ms", flush=True)
    err = np.abs(got - fed_logits).max() / np.abs(fed_logits).max()
    assert err < 1e-2, err
    assert int(dec.tokens(0, 1)[0, 0]) == fed_tok or err < 2e-3
    for l in range(L):
        gk, gv = dec.get_kv(l, 1, 0, n)
        for a, b_ in ((gk, fed_kv[l][0]), (gv, fed_kv[l][1])):
            for pos in (0, 1, 1023, 2047):
                x, y = a[0, pos].astype(np.float32), b_[0, pos].astype(np.float32)
                assert np.abs(x - y).max() <= 1e-2 * np.abs(y).max(), (l, pos)
    dec.run(2, use_graph=True)
    assert np.abs(dec.logits() - fed_after).max() / np.abs(fed_after).max() < 1e-2
    for l in range(L):
        dec.set_kv(l, *saved[l])

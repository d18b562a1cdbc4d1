"""Decode loop at the widths the benchmark times (BASELINE configs[3]: d_model 4096, 32 query / 8 kv heads of 128,
SwiGLU 14336, vocab 32000, int4 group 32 with fp16 scales, fp16 KV cache at context 2048).

* Two layers of those widths against the numpy checker (oracle/decoder_ref.py, pinned by tests/test_oracle_decoder.py):
  the single-launch kernel at batch 1 and the multi-kernel path at batch 16, both starting beyond 2048 cached positions,
  so per-wave k slices of 1024 and 3584, the grid K split of the down projection, 17 attention chunks per head and a
  125-block LM head per workgroup are all exercised against an independent result.
* All 32 layers: the single-launch kernel against the multi-kernel path (tokens and logits), step by step and as one
  launch, and row 0 of a batch-16 step against the batch-1 step.
Tolerances: the activations between stages are fp16 on the GPU and in the checker (same rounding points), the
projections sum in another order than numpy: 1e-2 of max|logit| is the float bar of the int4 path.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

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
        return rng.integers(0, 256, n * k // 2, dtype=np.uint8), rng.uniform(0.005, 0.02, n * (k // g)).astype(np.float16)

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
    B = cfg["max_batch"]
    for l in range(cfg["n_layers"]):
        k = rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32).astype(np.float16)
        v = rng.standard_normal((B, PREFILL, cfg["n_kv_heads"], hd), dtype=np.float32).astype(np.float16)
        dec.set_kv(l, k, v)
        ref.set_kv(l, k.astype(np.float32), v.astype(np.float32))
    return cfg, dec, ref


@pytest.fixture(scope="module")
def two_layers():
    import torch

    assert torch.cuda.is_available()
    cfg, dec, ref = _build_two_layers()
    yield cfg, dec, ref
    dec.close()


def _check_rows(got_logits, got_tok, exp_logits, what):
    from oracle.decoder_ref import greedy_pick

    for b in range(exp_logits.shape[0]):
        err = np.abs(got_logits[b] - exp_logits[b]).max() / np.abs(exp_logits[b]).max()
        assert err < 1e-2, (what, b, err)
        assert got_tok[b] == greedy_pick(got_logits[b]), (what, b)  # the exact rule, on the GPU's own logits
    return max(np.abs(got_logits[b] - exp_logits[b]).max() / np.abs(exp_logits[b]).max() for b in range(exp_logits.shape[0]))


def test_single_launch_batch1_at_7b_widths_matches_numpy(two_layers):
    cfg, dec, ref = two_layers
    tokens = np.array([4321], np.int32)
    dec.reset(tokens, PREFILL)
    cur = tokens.copy()
    seen = []
    for step in range(3):
        dec.run(1, persistent=True)
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp = ref.step(cur, PREFILL + step)
        worst = _check_rows(got_logits, got_tok, exp, f"persistent step {step}")
        print(f"[7b widths, single launch] step {step}: rel err {worst:.2e}", flush=True)
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


def test_multi_kernel_batch16_at_7b_widths_matches_numpy(two_layers):
    cfg, dec, ref = two_layers
    B = 16
    tokens = (np.arange(B, dtype=np.int32) * 1999 + 17) % cfg["vocab"]
    dec.reset(tokens, PREFILL)
    cur = tokens.copy()
    for step in range(2):
        dec.run(1, use_graph=True)
        got_logits, got_tok = dec.logits(), dec.tokens(step, 1)[0]
        exp = ref.step(cur, PREFILL + step)
        worst = _check_rows(got_logits, got_tok, exp, f"batch 16 step {step}")
        print(f"[7b widths, batch 16] step {step}: worst row rel err {worst:.2e}", flush=True)
        cur = got_tok.copy()
    # eager launches give the same stream as the graph replays
    graph_tok, graph_logits = dec.tokens(0, 2).copy(), dec.logits().copy()
    dec.reset(tokens, PREFILL)
    dec.run(2, use_graph=False)
    assert np.array_equal(dec.tokens(0, 2), graph_tok)
    assert np.array_equal(dec.logits(), graph_logits)


def test_full_depth_single_launch_agrees_with_multi_kernel_path():
    """32 layers, random init, cache filled to beyond 2000 positions: 16 steps."""
    import torch

    from oracle.decoder_ref import greedy_pick
    from yscv_amd.decoder import Decoder

    assert torch.cuda.is_available()
    cfg = dict(W7B, n_layers=32, max_batch=16, max_ctx=2176, max_steps=32)
    dec = Decoder(**cfg)
    dec.init_random(seed=11)
    dec.fill_kv_random(seed=12)
    start, first, steps = 2040, 777, 16  # crosses position 2048 (a new attention chunk) on the way
    cur = first
    toks, worst = [], 0.0
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
        assert diff / np.abs(lg).max() < 5e-3, (s, diff / np.abs(lg).max())
        assert tp == greedy_pick(lp) and tg == greedy_pick(lg)
        if tp != tg:  # only a near tie may flip the pick
            assert abs(lg[tp] - lg[tg]) <= 2 * diff, (s, tp, tg)
        toks.append(tp)
        cur = tp
    print(f"[32 layers] single launch vs multi-kernel: worst rel logit diff {worst:.2e}, tokens {toks}", flush=True)
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
    assert np.abs(many[0] - one).max() / np.abs(one).max() < 5e-3
    picks = dec.tokens(0, 1)[0]
    for b in range(B):
        assert picks[b] == greedy_pick(many[b])
    assert len({int(p) for p in picks}) > 1  # different rows, different inputs
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

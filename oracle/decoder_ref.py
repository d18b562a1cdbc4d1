"""TEST INFRASTRUCTURE ONLY -- numpy restatement of one Llama-style decode step.

Tolerance-checked glue (libm-dependent, not bit-pinned), following the reference semantics of
  RMSNorm   crates/yscv-kernels/src/ops/norm.rs:1497-1518
  RoPE      crates/yscv-kernels/src/ops/rope.rs:24-117   (rotate-half pairs (i, i + d/2))
  GQA       crates/yscv-onnx/src/runner/linear.rs:552-646 (kv_h = q_h / groups, scale 1/sqrt(d),
            max-subtracted softmax) applied to every cached position up to the current token
  greedy    apps/llm-bench/src/main.rs:538-543 (last index among equal maxima)
and the int4 projection definition of packed_int4_gemm_scalar (int4_matmul.rs:387-435) through
dequantised weights.  Activations are rounded to fp16 where the GPU decoder stores fp16.

The glue functions (rmsnorm, rope, gqa_attend, swiglu, greedy_pick) are module-level and work in f32, so
that tests/test_oracle_decoder.py can pin each of them to the reference's own unit-test vectors and to
closed forms; RefDecoder only strings them together and adds the fp16 roundings.
"""
from __future__ import annotations

import numpy as np


def f16(x):
    return np.asarray(x, np.float32).astype(np.float16).astype(np.float32)


def dequant_uint4(packed, scales16, n, k, g):
    """[n][k/2] uint4 nibbles (zero point 8) + fp16 scales -> f32 [n][k]."""
    pb = np.asarray(packed, np.uint8).reshape(n, k // 2)
    q = np.empty((n, k), np.float32)
    q[:, 0::2] = (pb & 15).astype(np.float32) - 8.0
    q[:, 1::2] = (pb >> 4).astype(np.float32) - 8.0
    s = np.asarray(scales16).reshape(n, k // g).astype(np.float32)
    return q * np.repeat(s, g, axis=1)


def rmsnorm(h, gamma, eps):
    """y = x * (1 / sqrt(mean(x^2) + eps)) * gamma over the last axis (ops/norm.rs:1497-1518)."""
    h = np.asarray(h, np.float32)
    inv = np.float32(1.0) / np.sqrt((h * h).mean(-1, keepdims=True, dtype=np.float32) + np.float32(eps))
    return (h * inv.astype(np.float32) * np.asarray(gamma, np.float32)).astype(np.float32)


def rope(x, pos, theta):
    """Rotate-half RoPE of x [..., d] at absolute position pos (ops/rope.rs:24-117): inv_freq[i] = 1/theta^(2i/d),
    pair (x[i], x[i + d/2]), x0' = x0 cos - x1 sin, x1' = x0 sin + x1 cos, angle = inv_freq[i] * pos in f32."""
    x = np.asarray(x, np.float32)
    d = x.shape[-1]
    i = np.arange(d // 2, dtype=np.float32)
    inv_freq = (np.float32(1.0) / np.power(np.float32(theta), np.float32(2.0) * i / np.float32(d))).astype(np.float32)
    ang = (inv_freq * np.float32(pos)).astype(np.float32)
    cs, sn = np.cos(ang), np.sin(ang)
    x0, x1 = x[..., : d // 2], x[..., d // 2:]
    return np.concatenate([x0 * cs - x1 * sn, x0 * sn + x1 * cs], -1).astype(np.float32)


def gqa_attend(q, kc, vc, groups):
    """One query position against a cache: q [heads][d], kc / vc [positions][kv_heads][d] ->
    [heads][d] (runner/linear.rs:552-646: kv_h = qh / groups, scores * 1/sqrt(d), max-subtracted softmax)."""
    q = np.asarray(q, np.float32)
    nh, hd = q.shape
    out = np.zeros((nh, hd), np.float32)
    scale = np.float32(1.0 / np.sqrt(hd))
    for qh in range(nh):
        kvh = qh // groups
        s = (kc[:, kvh, :] @ q[qh]) * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        out[qh] = p @ vc[:, kvh, :]
    return out


def swiglu(gate, up):
    gate = np.asarray(gate, np.float32)
    return (gate / (np.float32(1.0) + np.exp(-gate)) * np.asarray(up, np.float32)).astype(np.float32)


def greedy_pick(row):
    """Last index among equal maxima (Iterator::max_by, apps/llm-bench/src/main.rs:538-543)."""
    row = np.asarray(row)
    return int(np.flatnonzero(row == row.max())[-1])


def kv_i8_roundtrip(rows):
    """rows [n][kv_dim] f32 -> what an int8 cache returns for them: per-row scale = absmax / 127, q = round half away
    of v / scale clamped to +-127, value q * scale (LayerStorage::append / dequantise_to_vec,
    crates/yscv-onnx/src/runner/kv_cache.rs:45-79), through the C restatement."""
    from . import oracle as orc

    rows = np.ascontiguousarray(rows, np.float32)
    data, scales = orc.kv_i8_quantize_rows(rows, rows.shape[0], rows.shape[1])
    return (data.reshape(rows.shape).astype(np.float32) * scales.reshape(-1, 1).astype(np.float32)).astype(np.float32)


class RefDecoder:
    def __init__(self, cfg: dict, linears: dict, norms: dict, emb16, kv_i8: bool = False, round_f16: bool = True,
                 biases: dict | None = None):
        """linears[(layer, kind)] = (packed, scales16) with kind in q k v o gate up down, and
        linears[('lm_head',)]; norms[(layer, 'attn'|'ffn')], norms[('final',)] f32 gamma.
        kv_i8: the cache stores per-row int8 (KvDtype::I8); the rotated key of a new token is then quantised from its f32
        value, not from an fp16 rounding of it.
        round_f16=False drops every fp16 rounding of an activation: f32 from the embedding row to the logits, which
        is what the reference's CPU path computes (its activations are f32 tensors); the default rounds where the
        GPU decoder's multi-launch path without folded norms stores fp16."""
        self.c = cfg
        self._r = f16 if round_f16 else (lambda x: np.asarray(x, np.float32))
        self.kv_i8 = kv_i8
        g = cfg["group_size"]
        D, hd = cfg["d_model"], cfg["head_dim"]
        hq, hkv, ff = cfg["n_heads"] * hd, cfg["n_kv_heads"] * hd, cfg["d_ff"]
        shapes = {"q": (hq, D), "k": (hkv, D), "v": (hkv, D), "o": (D, hq), "gate": (ff, D), "up": (ff, D), "down": (D, ff)}
        self.w = {}
        for key, (p, s) in linears.items():
            n, k = (cfg["vocab"], D) if key == ("lm_head",) else shapes[key[1]]
            self.w[key] = dequant_uint4(p, s, n, k, g)
        self.norms = norms
        # biases[layer] = f32 [(n_heads + 2 n_kv_heads) * head_dim] in q, k, v order, added to the projections' outputs
        # (the Add node an exporter places behind the q / k / v MatMuls of a Qwen-style attention block)
        self.biases = biases or {}
        self.emb = np.asarray(emb16).view(np.float16).astype(np.float32).reshape(cfg["vocab"], D)
        L, B = cfg["n_layers"], cfg["max_batch"]
        self.kc = [[np.zeros((0, cfg["n_kv_heads"], hd), np.float32) for _ in range(B)] for _ in range(L)]
        self.vc = [[np.zeros((0, cfg["n_kv_heads"], hd), np.float32) for _ in range(B)] for _ in range(L)]

    def set_kv(self, layer, k_nat, v_nat):
        """k_nat / v_nat: f32 [batch][pos][kv_head][d] (keys already rotated)."""
        for b in range(k_nat.shape[0]):
            kb, vb = np.array(k_nat[b], np.float32), np.array(v_nat[b], np.float32)
            if self.kv_i8:
                kb = kv_i8_roundtrip(kb.reshape(kb.shape[0], -1)).reshape(kb.shape)
                vb = kv_i8_roundtrip(vb.reshape(vb.shape[0], -1)).reshape(vb.shape)
            self.kc[layer][b], self.vc[layer][b] = kb, vb

    def _rmsnorm(self, h, gamma):
        return self._r(rmsnorm(h, gamma, self.c["rms_eps"]))

    def _rope(self, x, pos):
        """x: [heads][d]."""
        return self._r(rope(x, pos, self.c["rope_theta"]))

    def step(self, tokens, pos):
        """tokens: int [batch]; pos: position the new token is written at.  Returns logits f32 [batch][vocab].
        self.trace keeps the last layer's intermediates (q|k|v with q and k rotated, attention output, SwiGLU
        output), the residual stream after the last layer and the LM head's input, each [batch][width]."""
        c = self.c
        hd, nh, nkv = c["head_dim"], c["n_heads"], c["n_kv_heads"]
        groups = nh // nkv
        B = len(tokens)
        h = self.emb[np.asarray(tokens)].astype(np.float32)
        for l in range(c["n_layers"]):
            xn = self._rmsnorm(h, self.norms[(l, "attn")])
            q = self._r(xn @ self.w[(l, "q")].T)
            k = self._r(xn @ self.w[(l, "k")].T)
            v = self._r(xn @ self.w[(l, "v")].T)
            if l in self.biases:
                bias = np.asarray(self.biases[l], np.float32)
                q = self._r(q + bias[: nh * hd])
                k = self._r(k + bias[nh * hd: (nh + nkv) * hd])
                v = self._r(v + bias[(nh + nkv) * hd:])
            q, k, v = q.reshape(B, nh, hd), k.reshape(B, nkv, hd), v.reshape(B, nkv, hd)
            ao = np.zeros((B, nh, hd), np.float32)
            qkv = np.zeros((B, (nh + 2 * nkv) * hd), np.float32)
            for b in range(B):
                qr, kr = self._rope(q[b], pos), self._rope(k[b], pos)
                k_row, v_row = kr, v[b]
                if self.kv_i8:
                    k_row = kv_i8_roundtrip(rope(k[b], pos, self.c["rope_theta"]).reshape(1, -1)).reshape(kr.shape)
                    v_row = kv_i8_roundtrip(v[b].reshape(1, -1)).reshape(v[b].shape)
                qkv[b] = np.concatenate([qr.reshape(-1), k_row.reshape(-1), v_row.reshape(-1)])
                self.kc[l][b] = np.concatenate([self.kc[l][b][:pos], k_row[None]], 0)
                self.vc[l][b] = np.concatenate([self.vc[l][b][:pos], v_row[None]], 0)
                ao[b] = gqa_attend(qr, self.kc[l][b], self.vc[l][b], groups)
            ao = self._r(ao.reshape(B, nh * hd))
            h = h + ao @ self.w[(l, "o")].T
            xn = self._rmsnorm(h, self.norms[(l, "ffn")])
            gt = xn @ self.w[(l, "gate")].T
            up = xn @ self.w[(l, "up")].T
            act = self._r(swiglu(gt, up))
            h = h + act @ self.w[(l, "down")].T
        xn = self._rmsnorm(h, self.norms[("final",)])
        self.trace = {"qkv": qkv, "attn_out": ao, "ffn": act, "residual": h.astype(np.float32), "normed": xn}
        return (xn @ self.w[("lm_head",)].T).astype(np.float32)

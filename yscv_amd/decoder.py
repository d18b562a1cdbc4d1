"""Thin binding of the GPU-resident decoder (yscv_hip_decoder_* in include/yscv_hip.h)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .capi import DecoderConfig, lib

KINDS = {"q": 0, "k": 1, "v": 2, "o": 3, "gate": 4, "up": 5, "down": 6, "lm_head": 7}
NORMS = {"attn": 0, "ffn": 1, "final": 2}


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class Decoder:
    def __init__(self, kv_dtype="f16", **cfg):
        """kv_dtype: 'f16' or 'i8' (per-row int8 cache, KvDtype::I8 of the reference's KvCache)."""
        self.cfg = dict(cfg)
        self.kv_dtype = kv_dtype
        c = DecoderConfig(**cfg)
        h = C.c_void_p()
        lib().decoder_create_kv(C.byref(c), {"f16": 0, "i8": 1}[kv_dtype], C.byref(h))
        self._h = h
        self.batch = 0

    def set_linear(self, layer, kind, packed, scales16, n, k):
        p = np.ascontiguousarray(packed, np.uint8)
        s = np.ascontiguousarray(scales16)
        assert s.dtype == np.float16
        lib().decoder_set_linear(self._h, int(layer), KINDS[kind], _p(p), _p(s), C.c_size_t(n), C.c_size_t(k))

    def set_norm(self, layer, kind, gamma):
        g = np.ascontiguousarray(gamma, np.float32)
        lib().decoder_set_norm(self._h, int(layer), NORMS[kind], _p(g))

    def set_qkv_bias(self, layer, bias16):
        """Bias of the fused q / k / v projection of one layer: fp16 [(n_heads + 2 n_kv_heads) * head_dim], or None."""
        if bias16 is None:
            lib().decoder_set_qkv_bias(self._h, int(layer), None)
            return
        b = np.ascontiguousarray(bias16)
        c = self.cfg
        assert b.dtype == np.float16 and b.size == (c["n_heads"] + 2 * c["n_kv_heads"]) * c["head_dim"]
        lib().decoder_set_qkv_bias(self._h, int(layer), _p(b))

    def set_embedding(self, table16):
        t = np.ascontiguousarray(table16)
        assert t.dtype == np.float16
        lib().decoder_set_embedding(self._h, _p(t))

    def finalize(self):
        lib().decoder_finalize(self._h)

    def init_random(self, seed=0, nibbles=(0, 15)):
        lib().decoder_init_random_range(self._h, C.c_uint64(seed), int(nibbles[0]), int(nibbles[1]))

    def fill_kv_random(self, seed=0):
        lib().decoder_fill_kv_random(self._h, C.c_uint64(seed))

    def set_kv(self, layer, k16, v16):
        k = np.ascontiguousarray(k16)
        v = np.ascontiguousarray(v16)
        assert k.dtype == np.float16 and v.dtype == np.float16 and k.shape == v.shape and k.ndim == 4
        lib().decoder_set_kv(self._h, int(layer), _p(k), _p(v), int(k.shape[0]), int(k.shape[1]))

    def get_kv(self, layer, batch, first_pos, n_positions):
        """(k, v) fp16 arrays [batch][n_positions][kv_head][head_dim] of cache positions first_pos .. (keys rotated)."""
        shape = (batch, n_positions, self.cfg["n_kv_heads"], self.cfg["head_dim"])
        k, v = np.empty(shape, np.float16), np.empty(shape, np.float16)
        lib().decoder_get_kv(self._h, int(layer), _p(k), _p(v), int(batch), int(first_pos), int(n_positions))
        return k, v

    def reset(self, tokens, start_pos):
        t = np.ascontiguousarray(tokens, np.int32)
        self.batch = t.size
        lib().decoder_reset(self._h, int(t.size), int(start_pos), _p(t))

    def prefill(self, tokens, start_pos=0, stream=None):
        """yscv_hip_decoder_prefill: the prompt in one pass; afterwards batch 1, the pick of the last position is the
        next input token and token 0 of the history, position start_pos + len(tokens)."""
        t = np.ascontiguousarray(tokens, np.int32)
        self.batch = 1
        lib().decoder_prefill(self._h, _p(t), int(t.size), int(start_pos), C.c_void_p(stream) if stream else None)

    def set_prefill_rows(self, rows):
        """yscv_hip_decoder_set_prefill_rows: prompt rows per pass of prefill() (default 4096)."""
        lib().decoder_set_prefill_rows(self._h, int(rows))

    def run(self, n_steps, use_graph=True, stream=None, persistent=False, auto=False):
        """use_graph: replay one captured HIP graph per step; persistent: run all steps inside one
        cooperative launch (batch 1, shapes the single-launch kernel supports); auto: the fastest of the two
        that applies (YSCV_HIP_DECODE_AUTO, what generate() uses)."""
        mode = 3 if auto else (2 if persistent else int(bool(use_graph)))
        lib().decoder_run(self._h, int(n_steps), mode, C.c_void_p(stream) if stream else None)

    def last_path(self):
        """yscv_hip_decoder_last_path: 0 kernel launches, 1 graph replays, 2 the single-launch kernel, -1 before any run."""
        v = C.c_int32(-1)
        lib().decoder_last_path(self._h, C.byref(v))
        return int(v.value)

    def run_projections(self, n_steps, stream=None):
        lib().decoder_run_projections(self._h, int(n_steps), C.c_void_p(stream) if stream else None)

    def tokens(self, first_step, n_steps):
        out = np.empty((n_steps, self.batch), np.int32)
        lib().decoder_read_tokens(self._h, int(first_step), int(n_steps), _p(out))
        return out

    def logits(self):
        out = np.empty((self.batch, self.cfg["vocab"]), np.float32)
        lib().decoder_read_logits(self._h, _p(out))
        return out

    def activation(self, which):
        """yscv_hip_decoder_read_activation: 'residual' | 'normed' | 'qkv' | 'attn_out' | 'ffn' of the last multi-kernel step."""
        c = self.cfg
        width = {"residual": c["d_model"], "normed": c["d_model"], "qkv": (c["n_heads"] + 2 * c["n_kv_heads"]) * c["head_dim"],
                 "attn_out": c["n_heads"] * c["head_dim"], "ffn": c["d_ff"]}[which]
        code = ["residual", "normed", "qkv", "attn_out", "ffn"].index(which)
        out = np.empty((self.batch, width), np.float32)
        lib().decoder_read_activation(self._h, code, _p(out), C.c_size_t(out.size))
        return out

    def generate(self, input_ids, max_tokens=256, temperature=1.0, top_k=50, top_p=0.9, eos_token_id=None,
                 repetition_penalty=1.0):
        """generate() of crates/yscv-onnx/src/generate.rs:58-118 with this decoder as the model (defaults = GenerateConfig
        ::default()).  Returns the generated token ids (prompt not included)."""
        ids = np.ascontiguousarray(input_ids, dtype=np.uint32)
        cfg = capi.GenerateConfig(max_tokens, temperature, top_k, top_p, 0 if eos_token_id is None else 1,
                                  0 if eos_token_id is None else int(eos_token_id), repetition_penalty)
        out = np.zeros(max(max_tokens, 1), np.uint32)
        n = C.c_size_t(0)
        lib().decoder_generate(self._h, _p(ids), C.c_size_t(ids.size), C.byref(cfg), _p(out), C.byref(n))
        return out[: n.value].copy()

    def weight_bytes(self) -> int:
        b = C.c_size_t()
        lib().decoder_weight_bytes(self._h, C.byref(b))
        return b.value

    def close(self):
        if self._h:
            lib().decoder_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

"""A BitNet-b1.58-style decoder assembled from the library's kernels.

Every linear layer is a ternary BitLinear: RMSNorm, per-token int8 quantisation (one fused
kernel), ternary matmul with the fused dequantisation.  Attention keeps K and V in f16.  The
reference has no decoder (its BitNet provider stops at the matmul,
crates/ronn-providers/src/bitnet/kernels.rs:134-178), so the layer formulas are the usual
LLaMA / BitNet-b1.58 ones; tests/decoder_model.py restates them in numpy.

A decode step is 122 kernel launches; it reads the position and the previous token from
device memory, so it is captured once in a HIP graph and replayed per token.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import time

import numpy as np

from . import _lib
from ._lib import check
from .device import Context, DeviceBuffer


@dataclasses.dataclass
class DecoderConfig:
    layers: int = 24
    hidden: int = 2560
    heads: int = 20
    head_dim: int = 128
    ffn: int = 6912
    vocab: int = 32000
    max_seq: int = 1024
    eps: float = 1e-5
    rope_theta: float = 10000.0

    @property
    def attn_dim(self) -> int:
        return self.heads * self.head_dim

    def linear_shapes(self):
        """(name, K, N) of the four BitLinear layers of a block."""
        return (("wqkv", self.hidden, 3 * self.attn_dim), ("wo", self.attn_dim, self.hidden),
                ("wgu", self.hidden, 2 * self.ffn), ("wdown", self.ffn, self.hidden))

    def packed_weight_bytes_per_token(self) -> int:
        per_layer = sum(k * n for _, k, n in self.linear_shapes())
        return (self.layers * per_layer + self.hidden * self.vocab) // 4


class _Linear:
    def __init__(self, tiled: DeviceBuffer, scale: float, K: int, N: int):
        self.tiled, self.scale, self.K, self.N = tiled, float(scale), K, N


class BitNetDecoder:
    """Weights, caches and scratch buffers of one decoder on one GPU."""

    def __init__(self, ctx: Context, cfg: DecoderConfig, max_batch_tokens: int = 512):
        if cfg.head_dim != 128:
            raise ValueError("head_dim must be 128")
        self.ctx, self.cfg, self.lib = ctx, cfg, ctx.lib
        self.max_tokens = max_batch_tokens
        H, A, F, V, T = cfg.hidden, cfg.attn_dim, cfg.ffn, cfg.vocab, max_batch_tokens
        a = ctx.alloc
        self.x = a(4 * T * H)
        self.o = a(4 * T * H)
        self.d = a(4 * T * H)
        self.qkv = a(4 * T * 3 * A)
        self.att = a(4 * T * A)
        self.gu = a(4 * T * 2 * F)
        self.logits = a(4 * V)
        pitch = ctx.act_pitch(max(H, A, F))
        self.acts = (a(T * pitch), a(4 * T), a(4 * T))
        self.tokens = a(4 * T)
        self.pos = a(4)
        self.history = a(4 * cfg.max_seq)
        cache = 2 * cfg.heads * cfg.max_seq * cfg.head_dim
        self.kcache = [a(cache) for _ in range(cfg.layers)]
        self.vcache = [a(cache) for _ in range(cfg.layers)]
        self.blocks = []
        self.embed = self.g_final = self.lm_head = None
        self._graph = None
        self._pos = 0   # host copy of the device position counter

    # -- weights ---------------------------------------------------------------------------
    def _linear_from_device_f32(self, d_w: DeviceBuffer, K: int, N: int) -> _Linear:
        d_p, scale, _, _ = self.ctx.quantize_ternary(d_w, K * N, _lib.SUM_STRICT_SEQ)
        tiled = self.ctx.tile_weights(d_p, K, N)
        self.ctx.sync()
        d_p.free()
        return _Linear(tiled, scale, K, N)

    def _vector(self, v: np.ndarray) -> DeviceBuffer:
        return self.ctx.to_device(np.ascontiguousarray(v, dtype=np.float32))

    def load_weights(self, w: dict):
        """w: numpy arrays 'embed' [V,H], 'g_final' [H], 'lm_head' [H,V], and per layer i
        'L{i}.g_attn' [H], 'L{i}.wqkv' [H,3A], 'L{i}.g_attn_sub' [A], 'L{i}.wo' [A,H],
        'L{i}.g_ffn' [H], 'L{i}.wgu' [H,2F], 'L{i}.g_ffn_sub' [F], 'L{i}.wdown' [F,H]."""
        cfg = self.cfg

        def lin(name, K, N):
            arr = np.ascontiguousarray(w[name], dtype=np.float32)
            assert arr.shape == (K, N), (name, arr.shape)
            d_w = self.ctx.to_device(arr)
            out = self._linear_from_device_f32(d_w, K, N)
            d_w.free()
            return out

        self.embed = self._vector(w["embed"])
        self.g_final = self._vector(w["g_final"])
        self.lm_head = lin("lm_head", cfg.hidden, cfg.vocab)
        self.blocks = []
        for i in range(cfg.layers):
            b = {"g_attn": self._vector(w["L%d.g_attn" % i]),
                 "g_attn_sub": self._vector(w["L%d.g_attn_sub" % i]),
                 "g_ffn": self._vector(w["L%d.g_ffn" % i]),
                 "g_ffn_sub": self._vector(w["L%d.g_ffn_sub" % i])}
            for name, K, N in cfg.linear_shapes():
                b[name] = lin("L%d.%s" % (i, name), K, N)
            self.blocks.append(b)

    def init_random(self, seed: int = 1, sigma: float = 0.02):
        """Random-initialised weights generated on the device (N(0, sigma) linears and
        embedding, unit norm gains)."""
        cfg, ctx = self.cfg, self.ctx
        counter = [seed * 1000]

        def normal(n, s):
            buf = ctx.alloc(4 * n)
            counter[0] += 1
            check(self.lib.rbn_synth_normal_device_f32(ctx.handle, counter[0], s, buf.ptr, n))
            return buf

        def lin(K, N):
            d_w = normal(K * N, sigma)
            out = self._linear_from_device_f32(d_w, K, N)
            d_w.free()
            return out

        ones = lambda n: self._vector(np.ones(n, dtype=np.float32))
        self.embed = normal(cfg.vocab * cfg.hidden, sigma)
        self.g_final = ones(cfg.hidden)
        self.lm_head = lin(cfg.hidden, cfg.vocab)
        self.blocks = []
        for _ in range(cfg.layers):
            b = {"g_attn": ones(cfg.hidden), "g_attn_sub": ones(cfg.attn_dim),
                 "g_ffn": ones(cfg.hidden), "g_ffn_sub": ones(cfg.ffn)}
            for name, K, N in cfg.linear_shapes():
                b[name] = lin(K, N)
            self.blocks.append(b)
        ctx.sync()

    # -- one forward pass over M tokens starting at the position in self.pos -----------------
    def _norm_quant(self, x, delta, gamma: DeviceBuffer, M: int, H: int, row0: int = 0, gate_up=None):
        off = 4 * row0 * H
        check(self.lib.rbn_rmsnorm_quant_i8(
            self.ctx.handle, (x.ptr + off) if x is not None else None,
            (delta.ptr + off) if delta is not None else None,
            gate_up.ptr if gate_up is not None else None, gamma.ptr,
            self.cfg.eps, M, H, self.acts[0].ptr, self.acts[1].ptr, self.acts[2].ptr))

    def _linear(self, lin: _Linear, M: int, out: DeviceBuffer):
        self.ctx.matmul(self.acts, lin.tiled, lin.scale, M, lin.K, lin.N, d_out=out)

    def _bitlinear1(self, lin: _Linear, gamma: DeviceBuffer, out: DeviceBuffer, x=None, gate_up=None,
                    residual=None, row0: int = 0):
        """One token: norm + quant + GEMV (+ residual) in one launch."""
        off = 4 * row0 * lin.K
        check(self.lib.rbn_bitlinear_gemv_f32(
            self.ctx.handle, (x.ptr + off) if x is not None else None,
            gate_up.ptr if gate_up is not None else None, gamma.ptr, self.cfg.eps, lin.tiled.ptr, lin.scale,
            lin.K, lin.N, residual.ptr if residual is not None else None, out.ptr))

    def forward_one(self):
        """forward(1) with five launches per layer: every BitLinear is one kernel, the
        residual additions ride on the o and down projections."""
        cfg, lib, hnd = self.cfg, self.lib, self.ctx.handle
        for i, b in enumerate(self.blocks):
            self._bitlinear1(b["wqkv"], b["g_attn"], self.qkv, x=self.x)
            check(lib.rbn_attention_decode_f16kv(hnd, self.qkv.ptr, self.pos.ptr, cfg.heads, cfg.head_dim,
                                                 cfg.rope_theta, self.kcache[i].ptr, self.vcache[i].ptr,
                                                 cfg.max_seq, self.att.ptr))
            self._bitlinear1(b["wo"], b["g_attn_sub"], self.x, x=self.att, residual=self.x)
            self._bitlinear1(b["wgu"], b["g_ffn"], self.gu, x=self.x)
            self._bitlinear1(b["wdown"], b["g_ffn_sub"], self.x, gate_up=self.gu, residual=self.x)
        self._bitlinear1(self.lm_head, self.g_final, self.logits, x=self.x)
        # position + 1, arg-max, history, and the next step's embedding in one launch
        check(lib.rbn_greedy_next_f32(hnd, self.logits.ptr, cfg.vocab, self.tokens.ptr, self.history.ptr,
                                      self.pos.ptr, cfg.max_seq, self.embed.ptr, cfg.hidden, self.x.ptr))

    def launches_per_token(self) -> int:
        """Kernel launches of one decode step (forward_one)."""
        return 5 * self.cfg.layers + 2

    def forward(self, M: int):
        """Tokens self.tokens[0:M] at positions *pos .. *pos+M-1; leaves the logits of the
        last token in self.logits and its arg-max in self.tokens[0] and the history."""
        cfg, lib, hnd = self.cfg, self.lib, self.ctx.handle
        H, A, F = cfg.hidden, cfg.attn_dim, cfg.ffn
        if M > self.max_tokens:
            raise ValueError("M exceeds max_batch_tokens")
        check(lib.rbn_embed_f32(hnd, self.embed.ptr, self.tokens.ptr, M, H, cfg.vocab, self.x.ptr))
        pending = None
        for i, b in enumerate(self.blocks):
            self._norm_quant(self.x, pending, b["g_attn"], M, H)
            self._linear(b["wqkv"], M, self.qkv)
            if M == 1:
                check(lib.rbn_attention_decode_f16kv(hnd, self.qkv.ptr, self.pos.ptr, cfg.heads, cfg.head_dim,
                                                     cfg.rope_theta, self.kcache[i].ptr, self.vcache[i].ptr,
                                                     cfg.max_seq, self.att.ptr))
            else:
                check(lib.rbn_rope_kv_store_f16(hnd, self.qkv.ptr, self.pos.ptr, M, cfg.heads, cfg.head_dim,
                                                cfg.rope_theta, self.kcache[i].ptr, self.vcache[i].ptr,
                                                cfg.max_seq))
                check(lib.rbn_attention_f16kv(hnd, self.qkv.ptr, self.pos.ptr, M, cfg.heads, cfg.head_dim,
                                              self.kcache[i].ptr, self.vcache[i].ptr, cfg.max_seq,
                                              self.att.ptr))
            self._norm_quant(self.att, None, b["g_attn_sub"], M, A)
            self._linear(b["wo"], M, self.o)
            self._norm_quant(self.x, self.o, b["g_ffn"], M, H)
            self._linear(b["wgu"], M, self.gu)
            self._norm_quant(None, None, b["g_ffn_sub"], M, F, gate_up=self.gu)   # SwiGLU fused in
            self._linear(b["wdown"], M, self.d)
            pending = self.d
        # only the last token needs logits; the pending residual is added for every row, so
        # that self.x is the complete residual stream
        if M > 1:
            self._norm_quant(self.x, pending, self.g_final, M - 1, H)
        self._norm_quant(self.x, pending, self.g_final, 1, H, row0=M - 1)
        self._linear(self.lm_head, 1, self.logits)
        check(lib.rbn_add_i32(hnd, self.pos.ptr, M))
        check(lib.rbn_argmax_f32(hnd, self.logits.ptr, cfg.vocab, self.tokens.ptr, self.history.ptr,
                                 self.pos.ptr, cfg.max_seq))

    # -- generation ------------------------------------------------------------------------
    def reset(self):
        check(self.lib.rbn_fill_u8(self.ctx.handle, self.pos.ptr, 0, 4))
        self._pos = 0

    def prefill(self, prompt: np.ndarray):
        """Runs the prompt from position 0.  The token predicted after it goes to history slot
        len(prompt), so the prompt has to be shorter than max_seq."""
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        if prompt.ndim != 1 or len(prompt) == 0:
            raise ValueError("the prompt must be a non-empty vector of token ids")
        if len(prompt) >= self.cfg.max_seq:
            raise ValueError("a prompt of %d tokens does not fit max_seq = %d (history slot %d is needed)"
                             % (len(prompt), self.cfg.max_seq, len(prompt)))
        self.reset()
        check(self.lib.rbn_h2d(self.ctx.handle, self.tokens.ptr, prompt.ctypes.data, prompt.nbytes))
        self.forward(len(prompt))
        self._pos = len(prompt)

    def capture_decode_step(self):
        if self._graph is None:
            self.ctx.graph_begin()
            self.forward_one()
            self._graph = self.ctx.graph_end()
        return self._graph

    def decode(self, n_tokens: int, use_graph: bool = True):
        """Greedy decoding of n_tokens more tokens; returns (tokens, seconds)."""
        if n_tokens < 0 or self._pos + n_tokens >= self.cfg.max_seq:
            raise ValueError("decoding %d tokens from position %d would pass max_seq = %d"
                             % (n_tokens, self._pos, self.cfg.max_seq))
        g = self.capture_decode_step() if use_graph else None
        # a step expects the embedding of the previous token in self.x (each step leaves the
        # next one's there; after a prompt it has to be looked up once)
        check(self.lib.rbn_embed_f32(self.ctx.handle, self.embed.ptr, self.tokens.ptr, 1, self.cfg.hidden,
                                     self.cfg.vocab, self.x.ptr))
        self.ctx.sync()
        t0 = time.perf_counter()
        for _ in range(n_tokens):
            if g is not None:
                self.ctx.graph_launch(g)
            else:
                self.forward_one()
        self.ctx.sync()
        dt = time.perf_counter() - t0
        self._pos += n_tokens
        return self.generated(n_tokens + 1)[1:], dt

    def generated(self, n: int) -> np.ndarray:
        """The last n generated tokens (history[p] = token predicted for position p)."""
        pos = int(self.pos.download(np.int32, 1)[0])
        hist = self.history.download(np.int32, self.cfg.max_seq)
        return hist[pos - n + 1:pos + 1].copy()

    def last_logits(self) -> np.ndarray:
        return self.logits.download(np.float32, self.cfg.vocab)

"""numpy restatement of the decoder that ronn_amd/decoder.py assembles on the device.

Test infrastructure only.  The reference has no decoder, so this file is what pins the
decoder kernels (the BitLinear inside it goes through the CPU oracle).  float32 throughout;
K and V pass through float16 as on the device.
"""
import numpy as np

from oracle import oracle as O
from util import epilogue, exact_int_matmul, oracle_weights


def rmsnorm_quant(x, gamma, eps):
    """y = (x * gamma) * rsqrt(mean(x^2) + eps), then per-token int8 quantisation."""
    x = x.astype(np.float32)
    ss = (x.astype(np.float64) ** 2).sum(axis=1) / x.shape[1]
    inv = (1.0 / np.sqrt(ss.astype(np.float32) + np.float32(eps))).astype(np.float32)
    y = (x * gamma.astype(np.float32)[None, :]).astype(np.float32) * inv[:, None]
    q, s, rs = O.act_quant_i8(y.astype(np.float32))
    return y.astype(np.float32), q, s, rs


class Linear:
    def __init__(self, w):
        self.t, self.vals = oracle_weights(np.ascontiguousarray(w, dtype=np.float32))

    def __call__(self, q, s):
        acc = exact_int_matmul(q, self.vals)
        return epilogue(acc, s, self.t.scale)


def rope(v, pos, theta):
    """v [M, heads, hd]; pairs (i, i + hd/2); angle pos * theta^(-2i/hd)."""
    M, heads, hd = v.shape
    half = hd // 2
    i = np.arange(half, dtype=np.float32)
    freq = np.power(np.float32(theta), (-2.0 * i / np.float32(hd)).astype(np.float32)).astype(np.float32)
    ang = (pos.astype(np.float32)[:, None] * freq[None, :]).astype(np.float32)
    cs, sn = np.cos(ang).astype(np.float32)[:, None, :], np.sin(ang).astype(np.float32)[:, None, :]
    a, b = v[..., :half], v[..., half:]
    return np.concatenate([a * cs - b * sn, b * cs + a * sn], axis=-1).astype(np.float32)


class Model:
    def __init__(self, cfg, w):
        self.cfg, self.w = cfg, w
        self.lin = {k: Linear(v) for k, v in w.items() if v.ndim == 2 and k != "embed"}
        self.k = [np.zeros((cfg.heads, cfg.max_seq, cfg.head_dim), np.float16) for _ in range(cfg.layers)]
        self.v = [np.zeros((cfg.heads, cfg.max_seq, cfg.head_dim), np.float16) for _ in range(cfg.layers)]
        self.pos = 0

    def forward(self, tokens):
        cfg, w = self.cfg, self.w
        M = len(tokens)
        pos = np.arange(self.pos, self.pos + M)
        x = w["embed"][np.asarray(tokens)].astype(np.float32)
        for i in range(cfg.layers):
            p = "L%d." % i
            _, q, s, _ = rmsnorm_quant(x, w[p + "g_attn"], cfg.eps)
            qkv = self.lin[p + "wqkv"](q, s).reshape(M, 3, cfg.heads, cfg.head_dim)
            qr = rope(qkv[:, 0], pos, cfg.rope_theta)
            kr = rope(qkv[:, 1], pos, cfg.rope_theta)
            self.k[i][:, pos, :] = kr.transpose(1, 0, 2).astype(np.float16)
            self.v[i][:, pos, :] = qkv[:, 2].transpose(1, 0, 2).astype(np.float16)
            att = np.zeros((M, cfg.heads, cfg.head_dim), np.float32)
            scale = np.float32(1.0 / np.sqrt(cfg.head_dim))
            for m in range(M):
                n = pos[m] + 1
                kk = self.k[i][:, :n, :].astype(np.float32)      # [heads, n, hd]
                vv = self.v[i][:, :n, :].astype(np.float32)
                sc = np.einsum("hd,hnd->hn", qr[m] * scale, kk)
                sc = sc - sc.max(axis=1, keepdims=True)
                pr = np.exp(sc)
                pr = pr / pr.sum(axis=1, keepdims=True)
                att[m] = np.einsum("hn,hnd->hd", pr, vv)
            _, q, s, _ = rmsnorm_quant(att.reshape(M, -1), w[p + "g_attn_sub"], cfg.eps)
            x = (x + self.lin[p + "wo"](q, s)).astype(np.float32)
            _, q, s, _ = rmsnorm_quant(x, w[p + "g_ffn"], cfg.eps)
            gu = self.lin[p + "wgu"](q, s)
            g, u = gu[:, :cfg.ffn], gu[:, cfg.ffn:]
            h = ((g / (1.0 + np.exp(-g))) * u).astype(np.float32)
            _, q, s, _ = rmsnorm_quant(h, w[p + "g_ffn_sub"], cfg.eps)
            x = (x + self.lin[p + "wdown"](q, s)).astype(np.float32)
        _, q, s, _ = rmsnorm_quant(x[-1:], w["g_final"], cfg.eps)
        logits = self.lin["lm_head"](q, s)[0]
        self.pos += M
        return logits


def random_weights(cfg, seed):
    from ronn_amd.device import synth_normal
    w = {}
    c = [seed * 100]

    def normal(shape, sigma):
        c[0] += 1
        return synth_normal(c[0], sigma, shape)

    def gain(n):
        return (1.0 + normal((n,), 0.1)).astype(np.float32)

    w["embed"] = normal((cfg.vocab, cfg.hidden), 1.0)
    w["g_final"] = gain(cfg.hidden)
    w["lm_head"] = normal((cfg.hidden, cfg.vocab), 0.02)
    for i in range(cfg.layers):
        p = "L%d." % i
        w[p + "g_attn"], w[p + "g_attn_sub"] = gain(cfg.hidden), gain(cfg.attn_dim)
        w[p + "g_ffn"], w[p + "g_ffn_sub"] = gain(cfg.hidden), gain(cfg.ffn)
        for name, K, N in cfg.linear_shapes():
            w[p + name] = normal((K, N), 0.02)
    return w

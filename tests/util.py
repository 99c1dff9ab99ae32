"""Helpers shared by the parity tests."""
import struct

import numpy as np

from oracle import oracle as O


def bits(x):
    return "0x%08x" % struct.unpack("<I", struct.pack("<f", float(x)))[0]


def same_bits(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and bool((a.view(np.uint32) == b.view(np.uint32)).all())


def exact_int_matmul(q, w_values):
    """int32 product of small-integer matrices through BLAS.

    |q| <= 128 and |w| <= 1, so every partial sum is bounded by 128*K; below 2^24 every
    f32 operation in any order is exact, and f64 covers the rest.  This is the library
    routine the literal oracle loop is cross-checked with (tests/test_oracle.py,
    tests/test_host_logic.py) and what stands in for it at sizes where the literal
    per-element loop would take minutes.
    """
    q = np.asarray(q)
    w_values = np.asarray(w_values)
    k = q.shape[1]
    dt = np.float32 if 128 * k < 2 ** 24 else np.float64
    return np.rint(q.astype(dt) @ w_values.astype(dt)).astype(np.int32)


def epilogue(acc, act_scale, w_scale):
    """kernels.rs:168: (acc as f32 * a.scale) * b.scale, left to right, in f32."""
    r = acc.astype(np.float32) * np.asarray(act_scale, dtype=np.float32).reshape(-1, 1)
    return (r.astype(np.float32) * np.float32(w_scale)).astype(np.float32)


def decode_tiled(tiled_words, K, N):
    """Inverse of the device's weight tiling: u32 words -> int8 values [K, N].

    Word ((q * KB + kb) * 4 + c) belongs to column 4q+c and k-block kb; inside a word the
    weight k = 16*kb + 4*s + b sits at bit 8*b + 2*s as code = value + 1.
    """
    kpad = (K + 127) // 128 * 128
    npad = (N + 63) // 64 * 64
    kb_n = kpad // 16
    t = np.asarray(tiled_words, dtype=np.uint32).reshape(npad // 4, kb_n, 4)
    t = t.transpose(1, 0, 2).reshape(kb_n, npad)          # [kb][column]
    out = np.zeros((kpad, npad), dtype=np.int8)
    for s in range(4):
        for b in range(4):
            code = (t >> np.uint32(8 * b + 2 * s)) & np.uint32(3)
            out[4 * s + b::16, :] = code.astype(np.int8) - 1
    assert (out[K:, :] == 0).all() and (out[:, N:] == 0).all(), "padding must be zero weights"
    return out[:K, :N]


def oracle_weights(w):
    """Oracle ternarisation of a weight matrix: (TernaryTensor, int8 values [K,N])."""
    t = O.quantize_ternary(w)
    return t, t.values().reshape(w.shape)

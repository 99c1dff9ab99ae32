"""Pins the CPU oracle (oracle/bitnet_oracle.c) before anything is compared with it.

Checks, in order: the reference's own known-answer test and hand-derived vectors for
its other test inputs (tests/golden/ternary_kats.json), closed forms, brute force on
tiny inputs with independent arithmetic, invariants, and regression figures that a
non-sequential sum would miss.
"""
import json
import os
import struct

import numpy as np
import pytest

from oracle import oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "ternary_kats.json")))


def bits(x):
    return "0x%08x" % struct.unpack("<I", struct.pack("<f", float(x)))[0]


@pytest.mark.parametrize("kat", KATS["quantize"], ids=lambda k: k["name"])
def test_quantize_known_answers(kat):
    t = O.quantize_ternary(np.array(kat["data"], dtype=np.float32).reshape(kat["shape"]))
    assert [t.get_value(i) for i in range(t.element_count)] == kat["values"]
    assert bytes(t.packed_data).hex() == kat["packed_hex"]
    assert bits(t.threshold) == kat["threshold_bits"]
    assert bits(t.scale) == kat["scale_bits"]
    assert t.shape == kat["shape"]


def test_reference_roundtrip_and_ratio():
    # quantization.rs:315-328: shape preserved, compression ratio > 15 (16.0 for n % 4 == 0)
    d = np.array(KATS["quantize"][1]["data"], dtype=np.float32).reshape(2, 4)
    t = O.quantize_ternary(d)
    back = O.dequantize_ternary(t)
    assert back.shape == d.shape
    assert t.compression_ratio() == np.float32(16.0)
    assert set(np.unique(back)).issubset({-t.scale, np.float32(0), t.scale})


@pytest.mark.parametrize("kat", KATS["matmul"], ids=lambda k: k["name"])
def test_matmul_known_answers(kat):
    a = np.array(kat["a"], dtype=np.float32).reshape(kat["m"], kat["k"])
    b = np.array(kat["b"], dtype=np.float32).reshape(kat["k"], kat["n"])
    out, acc = O.execute_ternary(a, b)
    assert acc.ravel().tolist() == kat["acc"]
    assert [bits(v) for v in out.ravel()] == kat["out_bits"]


@pytest.mark.parametrize("kat", KATS["allocator"], ids=str)
def test_allocator_sizes(kat):
    # allocator.rs:231-235, :257-261, :285-288
    assert O.packed_size(kat["shape"], kat["dtype"]) == kat["bytes"]
    assert O.alignment(kat["dtype"]) == kat["alignment"]
    assert O.packed_size([4], 3) == -1  # I8 is rejected (allocator.rs:60-63)


def test_get_value_table_and_out_of_range():
    # 0b11_10_01_00 = codes 0,1,2,3 for elements 0..3  (quantization.rs:285-290)
    t = O.TernaryTensor(np.array([0xE4], dtype=np.uint8), [4], 1.0, 0.0, 4)
    assert [t.get_value(i) for i in range(4)] == [-1, 0, 1, 0]
    assert t.get_value(4) == 0 and t.get_value(10**9) == 0  # :276-278
    assert O.dequantize_ternary(O.TernaryTensor(np.array([0xE4], dtype=np.uint8), [4], 2.5, 0.0, 4)
                                ).tolist() == [-2.5, 0.0, 2.5, 0.0]


def test_closed_forms():
    # constant c > 0: threshold 0.7c, everything survives, scale c, all codes 10
    for c, n in ((0.5, 8), (3.0, 37), (0.015625, 1024)):
        x = np.full(n, c, dtype=np.float32)
        x[::2] *= -1
        t = O.quantize_ternary(x)
        assert t.threshold == np.float32(np.float32(c) * np.float32(0.7))
        assert t.scale == np.float32(c) and t.survivors == n
        assert t.values().tolist() == [-1 if i % 2 == 0 else 1 for i in range(n)]
    # all zeros: threshold 0, every code 01, no survivors, scale 1.0 (quantization.rs:93-94)
    t = O.quantize_ternary(np.zeros(10, dtype=np.float32))
    assert t.threshold == 0 and t.scale == 1 and t.survivors == 0
    assert bytes(t.packed_data).hex() == "555505"  # tail bits of the last byte stay 0
    # signed zero and NaN: -0.0 is zero; NaN packs as 00 (-1) but is not a survivor
    x = np.array([-0.0, np.nan, 1.0, -1.0], dtype=np.float32)
    p = O.pack_ternary_bits(x, 0.5)
    assert p.tolist() == [0b00_10_00_01]


def test_bruteforce_small_dyadic():
    # dyadic values: every f32 operation is exact, so plain Python floats/ints give the answer
    rng = np.random.default_rng(7)
    for _ in range(50):
        n = int(rng.integers(1, 40))
        x = (rng.integers(-64, 65, n) / 16.0).astype(np.float32)
        t = O.quantize_ternary(x)
        mean = sum(abs(float(v)) for v in x) / n
        thr = np.float32(np.float32(mean) * np.float32(0.7))
        assert t.threshold == thr
        surv = [abs(float(v)) for v in x if abs(float(v)) > float(thr)]
        assert t.survivors == len(surv)
        want_scale = np.float32(1.0) if not surv else np.float32(np.float32(sum(surv)) / np.float32(len(surv)))
        assert t.scale == want_scale
        want = [0 if abs(float(v)) <= float(thr) else (1 if v > 0 else -1) for v in x]
        assert t.values().tolist() == want


def test_matmul_bruteforce_and_structure():
    rng = np.random.default_rng(11)
    for m, k, n in ((1, 5, 3), (3, 17, 9), (4, 64, 64), (2, 33, 7)):
        a = rng.normal(0, 1, (m, k)).astype(np.float32)
        b = rng.normal(0, 0.02, (k, n)).astype(np.float32)
        ta, tb = O.quantize_ternary(a), O.quantize_ternary(b)
        out, acc = O.ternary_matmul(ta, tb, m, n, k)
        va = ta.values().reshape(m, k).astype(np.int64)
        vb = tb.values().reshape(k, n).astype(np.int64)
        want = va @ vb
        assert (acc == want).all()
        want_f = (want.astype(np.float32) * ta.scale) * tb.scale
        assert (out.view(np.uint32) == want_f.astype(np.float32).view(np.uint32)).all()
    # transposed operands must NOT give the same answer (catches an index swap)
    a = rng.normal(0, 1, (3, 3)).astype(np.float32)
    b = rng.normal(0, 1, (3, 3)).astype(np.float32)
    _, acc_ab = O.execute_ternary(a, b)
    va = O.quantize_ternary(a).values().reshape(3, 3).astype(int)
    vb = O.quantize_ternary(b).values().reshape(3, 3).astype(int)
    assert (acc_ab == va @ vb).all()
    # identity-like weights reduce to a gather of the ternarised activations
    k = 8
    w = np.zeros((k, k), dtype=np.float32)
    perm = rng.permutation(k)
    w[np.arange(k), perm] = 1.0
    x = rng.normal(0, 1, (2, k)).astype(np.float32)
    _, acc = O.execute_ternary(x, w)
    vx = O.quantize_ternary(x).values().reshape(2, k)
    assert (acc[:, perm] == vx).all()


def test_dimension_mismatch_message():
    ta = O.quantize_ternary(np.ones((2, 3), dtype=np.float32))
    tb = O.quantize_ternary(np.ones((3, 2), dtype=np.float32))
    with pytest.raises(ValueError, match="Matrix dimension mismatch"):
        O.ternary_matmul(ta, tb, 2, 2, 4)


def test_sequential_sum_semantics_regression():
    # A sequential f32 fold drifts from the true sum; a tree or f64 sum would not.
    # 2^24 ones then more ones: the fold sticks at 16777216.
    x = np.ones(2**24 + 1000, dtype=np.float32)
    t = O.quantize_ternary(x)
    assert t.threshold == np.float32(np.float32(np.float32(16777216.0) / np.float32(x.size)) * np.float32(0.7))
    # numpy's cumsum in f32 is the same left fold: cross-check on random data
    rng = np.random.default_rng(3)
    x = rng.normal(0, 0.02, 300_000).astype(np.float32)
    seq = np.cumsum(np.abs(x), dtype=np.float32)[-1]
    t = O.quantize_ternary(x)
    assert t.threshold == np.float32(np.float32(seq / np.float32(x.size)) * np.float32(0.7))
    surv = np.abs(x)[np.abs(x) > t.threshold]
    assert t.survivors == surv.size
    assert t.scale == np.float32(np.cumsum(surv, dtype=np.float32)[-1] / np.float32(surv.size))


def test_empty_tensor():
    t = O.quantize_ternary(np.zeros(0, dtype=np.float32))
    assert np.isnan(t.threshold) and t.scale == 1 and t.packed_data.size == 0


# ---- build-defined int8 activation path (no reference counterpart) -------------------

def test_act_quant_closed_forms():
    k = 16
    x = np.zeros((3, k), dtype=np.float32)
    x[0, :] = np.linspace(-2, 2, k)          # row hits +-amax -> +-127
    x[2, :] = 1e-8                            # far below the 1e-5 guard: 1e-8*127/1e-5 = 0.127 -> 0
    x[2, 3] = 1e-7                            # 1.27 -> 1 (the guard fixes the scale, not the values)
    q, s, rs = O.act_quant_i8(x)
    assert q[0, 0] == -127 and q[0, -1] == 127 and s[0] == np.float32(2.0) / np.float32(127.0)
    assert (q[1] == 0).all() and s[1] == np.float32(1e-5) / np.float32(127.0)
    assert q[2].tolist() == [0, 0, 0, 1] + [0] * 12 and s[2] == s[1]
    assert (rs == q.astype(np.int64).sum(1)).all()
    # ties round half to even: amax = 127 -> inv = 1 -> q = rne(x)
    x = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49]], dtype=np.float32)
    q, s, _ = O.act_quant_i8(x)
    assert q[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 3] and s[0] == 1.0


def test_i8_matmul_against_integer_library_routine():
    rng = np.random.default_rng(5)
    for m, k, n in ((1, 64, 32), (4, 100, 19), (16, 256, 48)):
        x = rng.normal(0, 1, (m, k)).astype(np.float32)
        w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
        q, s, _ = O.act_quant_i8(x)
        tb = O.quantize_ternary(w)
        out, acc = O.matmul_i8_ternary(q, s, tb)
        want = q.astype(np.int64) @ tb.values().reshape(k, n).astype(np.int64)
        assert (acc == want).all()
        want_f = ((want.astype(np.float32) * s[:, None]).astype(np.float32) * tb.scale).astype(np.float32)
        assert (out.view(np.uint32) == want_f.view(np.uint32)).all()

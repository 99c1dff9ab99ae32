"""HIP kernels against the CPU oracle, through the C ABI, on a real MI355X.

Bar: packed bytes, thresholds, scales, int8 activations and int32 accumulators are
bit-exact; f32 outputs are bit-exact too (stricter than the 1e-6 relative the
target asks for), because |acc| < 2^24 and the epilogue keeps the reference's
multiplication order.
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from ronn_amd import _lib
from ronn_amd.device import synth_normal
from util import bits, decode_tiled, epilogue, exact_int_matmul, oracle_weights, same_bits

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "ternary_kats.json")))
STRICT, TREE = _lib.SUM_STRICT_SEQ, _lib.SUM_TREE


def say(*a):
    print(*a, flush=True)


def device_quantize(ctx, x, mode=STRICT):
    x = np.ascontiguousarray(x, dtype=np.float32)
    d_x = ctx.to_device(x)
    d_p, scale, thr, cnt = ctx.quantize_ternary(d_x, x.size, mode)
    packed = d_p.download(np.uint8, (x.size + 3) // 4)
    return d_p, packed, scale, thr, cnt


# ---- golden vectors -------------------------------------------------------------------

@pytest.mark.parametrize("kat", KATS["quantize"], ids=lambda k: k["name"])
def test_kat_quantize(ctx, kat):
    x = np.array(kat["data"], dtype=np.float32)
    _, packed, scale, thr, _ = device_quantize(ctx, x)
    assert bytes(packed).hex() == kat["packed_hex"]
    assert bits(thr) == kat["threshold_bits"] and bits(scale) == kat["scale_bits"]


@pytest.mark.parametrize("kat", KATS["matmul"], ids=lambda k: k["name"])
def test_kat_execute(ctx, kat):
    a = np.array(kat["a"], dtype=np.float32).reshape(kat["m"], kat["k"])
    b = np.array(kat["b"], dtype=np.float32).reshape(kat["k"], kat["n"])
    out, acc = ctx.execute_ternary_matmul(a, b)
    assert acc.ravel().tolist() == kat["acc"]
    assert [bits(v) for v in out.ravel()] == kat["out_bits"]


# ---- (1) ternarize + pack ----------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 3, 4, 5, 15, 16, 17, 63, 64, 65, 4095, 4096, 4097, 100003])
def test_pack_ragged_sizes(ctx, n):
    x = synth_normal(100 + n, 1.0, (n,))
    thr = np.float32(0.6)
    d_p = ctx.pack_ternary(ctx.to_device(x), n, thr)
    got = d_p.download(np.uint8, (n + 3) // 4)
    assert (got == O.pack_ternary_bits(x, thr)).all()


def test_pack_special_values(ctx):
    x = np.array([-0.0, 0.0, np.nan, -np.nan, np.inf, -np.inf, 0.5, -0.5, 0.5000001, 1e-45] * 13,
                 dtype=np.float32)
    for thr in (np.float32(0.5), np.float32(0.0), np.float32(np.nan), np.float32(np.inf)):
        got = ctx.pack_ternary(ctx.to_device(x), x.size, thr).download(np.uint8, (x.size + 3) // 4)
        assert (got == O.pack_ternary_bits(x, thr)).all()


DISTS = {
    "weights_0.02": lambda n, s: synth_normal(s, 0.02, (n,)),
    "acts_1.0": lambda n, s: synth_normal(s, 1.0, (n,)),
    "ones": lambda n, s: np.ones(n, dtype=np.float32),
    "zeros": lambda n, s: np.zeros(n, dtype=np.float32),
    "denormal": lambda n, s: synth_normal(s, 1e-40, (n,)),
    "huge": lambda n, s: synth_normal(s, 1e30, (n,)),
    "wide": lambda n, s: (synth_normal(s, 1.0, (n,)) * np.exp(6 * synth_normal(s + 1, 1.0, (n,)))).astype(np.float32),
}


@pytest.mark.parametrize("dist", sorted(DISTS))
@pytest.mark.parametrize("n", [1, 17, 4096, 4097, 70001, 1 << 20])
def test_strict_abs_sum_matches_sequential_fold(ctx, dist, n):
    x = DISTS[dist](n, 7)
    want = np.cumsum(np.abs(x), dtype=np.float32)[-1]   # numpy's f32 cumsum is the same left fold
    got, cnt = ctx.abs_sum(ctx.to_device(x), n, STRICT)
    assert bits(got) == bits(want) and cnt == n
    thr = np.float32(np.median(np.abs(x)))
    surv = np.abs(x)[np.abs(x) > thr]
    want_m = np.cumsum(surv, dtype=np.float32)[-1] if surv.size else np.float32(0)
    got_m, cnt_m = ctx.abs_sum(ctx.to_device(x), n, STRICT, mask_threshold=thr)
    assert cnt_m == surv.size
    if surv.size:
        assert bits(got_m) == bits(want_m)


def _steps(n, seed):
    """Growth that changes by orders of magnitude along the tensor: the windows that predict the
    exponent of S per block lose it in both directions and must end early, not go wrong."""
    x = synth_normal(seed, 1.0, (n,))
    scale = np.ones(n, dtype=np.float32)
    cuts = [0, n // 16, n // 7, n // 3, n // 2, (3 * n) // 4, n]
    for i, f in enumerate((1e-6, 1.0, 1e-3, 300.0, 0.0, 2e-2)):
        scale[cuts[i]:cuts[i + 1]] = f
    return (x * scale).astype(np.float32)


@pytest.mark.parametrize("n", [300_001, 3_000_000])
def test_strict_abs_sum_when_the_growth_prediction_fails(ctx, n):
    x = _steps(n, 21)
    want = np.cumsum(np.abs(x), dtype=np.float32)[-1]
    got, cnt = ctx.abs_sum(ctx.to_device(x), n, STRICT)
    assert bits(got) == bits(want) and cnt == n
    thr = np.float32(1e-3)
    surv = np.abs(x)[np.abs(x) > thr]
    got_m, cnt_m = ctx.abs_sum(ctx.to_device(x), n, STRICT, mask_threshold=thr)
    assert cnt_m == surv.size and bits(got_m) == bits(np.cumsum(surv, dtype=np.float32)[-1])


def test_strict_abs_sum_with_a_crossing_deep_inside_a_long_window(ctx):
    """One term of 1.0 per block of 4096 behind a first term of 2^16: S climbs one unit per block, the
    window that follows block 8192 is some 63,000 blocks long, and S leaves its binade (at 2^17) beyond
    block 57,000 of that window - in the second of the stretches of 32,768 maps the window-end kernel
    walks.  Every partial sum is an integer below 2^24, so the fold is exact and its value known."""
    blocks = 72_000
    n = blocks * 4096
    x = np.zeros(n, dtype=np.float32)
    x[5::4096] = -1.0
    x[0] = 65536.0
    want = np.float32(65536 + blocks)
    d_x = ctx.to_device(x)
    got, cnt = ctx.abs_sum(d_x, n, STRICT)
    assert bits(got) == bits(want) and cnt == n
    got_m, cnt_m = ctx.abs_sum(d_x, n, STRICT, mask_threshold=np.float32(0.75))
    assert bits(got_m) == bits(want) and cnt_m == blocks + 1
    got_1, cnt_1 = ctx.abs_sum(d_x, n, STRICT, mask_threshold=np.float32(2.0))
    assert bits(got_1) == bits(np.float32(65536)) and cnt_1 == 1
    d_x.free()


@pytest.mark.parametrize("case", range(8))
def test_quantize_strict_on_random_piecewise_tensors(ctx, case):
    """Threshold, scale, survivor count and every packed byte of the strict quantiser against numpy's
    own f32 left folds, on tensors whose scale jumps by orders of magnitude at random places (zero
    stretches and short mantissas - exact ties - among them)."""
    rng = np.random.default_rng(1000 + case)
    n = int(rng.integers(1, 9_000_000)) if case % 2 else int(rng.integers(1, 600_000))
    x = rng.standard_normal(n).astype(np.float32)
    cuts = np.concatenate([[0], np.sort(rng.integers(0, n + 1, size=int(rng.integers(0, 9)))), [n]])
    for a, b in zip(cuts[:-1], cuts[1:]):
        x[a:b] *= np.float32(0.0 if rng.random() < 0.15 else 10.0 ** rng.uniform(-7, 4))
    if case % 4 == 0:
        x = (np.round(x * 64) / 64).astype(np.float32)
    d_p, packed, scale, thr, survivors = device_quantize(ctx, x)
    ax = np.abs(x)
    total = np.cumsum(ax, dtype=np.float32)[-1]
    thr_want = np.float32(np.float32(total / np.float32(n)) * np.float32(0.7))   # quantization.rs:79
    assert bits(thr) == bits(thr_want)
    sv = ax[ax > thr_want]
    assert survivors == sv.size
    if sv.size:
        assert bits(scale) == bits(np.float32(np.cumsum(sv, dtype=np.float32)[-1] / np.float32(sv.size)))
    codes = np.where(ax <= thr_want, 1, np.where(x > 0, 2, 0)).astype(np.uint8)
    codes = np.concatenate([codes, np.zeros((-n) % 4, np.uint8)]).reshape(-1, 4)
    want = (codes[:, 0] | (codes[:, 1] << 2) | (codes[:, 2] << 4) | (codes[:, 3] << 6)).astype(np.uint8)
    assert (packed == want).all()


def test_strict_abs_sum_nonfinite(ctx):
    x = synth_normal(9, 1.0, (100000,))
    for edit, want in (({5000: np.inf}, np.inf), ({5000: np.inf, 90000: np.nan}, np.nan),
                       ({70000: np.nan}, np.nan), ({}, None)):
        y = x.copy()
        for i, v in edit.items():
            y[i] = v
        got, _ = ctx.abs_sum(ctx.to_device(y), y.size, STRICT)
        ref = np.cumsum(np.abs(y), dtype=np.float32)[-1]
        assert bits(got) == bits(ref) or (np.isnan(got) and np.isnan(ref))
    y = synth_normal(10, 3e37, (100000,))   # the fold overflows to +Inf
    got, _ = ctx.abs_sum(ctx.to_device(y), y.size, STRICT)
    assert np.isinf(got)


def test_stall_at_two_pow_24(ctx):
    n = (1 << 24) + 5000
    got, _ = ctx.abs_sum(ctx.to_device(np.ones(n, dtype=np.float32)), n, STRICT)
    assert got == np.float32(16777216.0)
    tree, _ = ctx.abs_sum(ctx.to_device(np.ones(n, dtype=np.float32)), n, TREE)
    assert tree == np.float32(n)


@pytest.mark.parametrize("shape,sigma", [((64, 64), 0.02), ((2048, 2048), 0.02), ((1000, 777), 0.02),
                                         ((4096, 4096), 0.02)])
def test_quantize_ternary_bit_exact(ctx, shape, sigma):
    w = synth_normal(0x5EED1001, sigma, shape)
    say("quantize", shape)
    t = O.quantize_ternary(w)
    _, packed, scale, thr, cnt = device_quantize(ctx, w)
    assert bits(thr) == bits(t.threshold)
    assert cnt == t.survivors
    assert bits(scale) == bits(t.scale)
    assert (packed == t.packed_data).all()


@pytest.mark.parametrize("shape,sigma", [((4096, 11008), 0.02), ((8192, 28672), 0.015)])
def test_quantize_ternary_bit_exact_full_shapes(ctx, shape, sigma):
    # the FFN up/gate matrix of the decode sweep and the 235 M-weight large-layer matrix: every
    # packed byte, the threshold and the scale against the oracle's sequential sums (which
    # drift to 0.83 and 0.34 of the true sum at these sizes, so a tree sum cannot pass)
    say("quantize full shape", shape)
    w = synth_normal(0x5EED1001 + shape[1], sigma, shape)
    t = O.quantize_ternary(w)
    true_thr = np.abs(w).astype(np.float64).mean() * 0.7
    assert float(t.threshold) < (0.9 if shape[0] == 4096 else 0.4) * true_thr
    _, packed, scale, thr, cnt = device_quantize(ctx, w)
    assert bits(thr) == bits(t.threshold)
    assert cnt == t.survivors
    assert bits(scale) == bits(t.scale)
    assert packed.size == w.size // 4 and (packed == t.packed_data).all()


def test_quantize_tree_mode_is_close_but_flagged(ctx):
    w = synth_normal(3, 0.02, (1 << 22,))
    _, packed, scale, thr, cnt = device_quantize(ctx, w, TREE)
    true_mean = np.abs(w).astype(np.float64).mean()
    assert abs(float(thr) - 0.7 * true_mean) < 1e-7
    surv = np.abs(w)[np.abs(w) > thr]
    assert cnt == surv.size and abs(float(scale) - surv.astype(np.float64).mean()) < 1e-6
    assert (packed == O.pack_ternary_bits(w, thr)).all()


@pytest.mark.parametrize("n", [1, 17, 4097, 70_001, 3_000_000, 60_000_000])
def test_quantize_tree_mode_threshold_from_the_device(ctx, n):
    """The tree-sum quantiser queues its packing pass behind the sum and takes the threshold from the
    device: threshold = (sum / n) * 0.7 of the sum it returns, bit for bit; count and packed codes are
    those of that threshold; the survivors' mean is their f64 mean."""
    w = synth_normal(40 + n % 97, 0.05, (n,))
    d_x = ctx.to_device(w)
    tree_sum, _ = ctx.abs_sum(d_x, n, TREE)
    _, packed, scale, thr, cnt = device_quantize(ctx, w, TREE)
    assert bits(thr) == bits(np.float32(np.float32(tree_sum) / np.float32(n)) * np.float32(0.7))
    assert abs(float(tree_sum) - np.abs(w).astype(np.float64).sum()) <= 1e-6 * max(1.0, float(tree_sum))
    keep = np.abs(w) > thr
    assert cnt == int(keep.sum())
    if cnt:
        assert abs(float(scale) - np.abs(w)[keep].astype(np.float64).mean()) < 1e-6
    assert (packed == O.pack_ternary_bits(w, thr)).all()


def test_quantize_edge_tensors(ctx):
    for x in (np.zeros(10, dtype=np.float32), np.full(37, 3.0, dtype=np.float32),
              np.array([np.nan, 1.0, -2.0, 0.25], dtype=np.float32)):
        t = O.quantize_ternary(x)
        _, packed, scale, thr, cnt = device_quantize(ctx, x)
        assert (packed == t.packed_data).all() and cnt == t.survivors
        assert bits(scale) == bits(t.scale)
        assert bits(thr) == bits(t.threshold) or (np.isnan(thr) and np.isnan(t.threshold))
    d_x = ctx.alloc(16)
    d_p, scale, thr, cnt = ctx.quantize_ternary(d_x, 0)
    assert np.isnan(thr) and scale == 1 and cnt == 0   # empty tensor


def test_dequantize_and_unpack(ctx):
    w = synth_normal(21, 0.02, (513,))
    t = O.quantize_ternary(w)
    d_p = ctx.to_device(np.concatenate([t.packed_data, np.zeros(32, np.uint8)]))
    got = ctx.dequantize_ternary(d_p, w.size, t.scale).download(np.float32, w.size)
    assert same_bits(got, O.dequantize_ternary(t))
    # code 11 reads as zero (quantization.rs:195, :289)
    raw = np.arange(256, dtype=np.uint8)
    d_raw = ctx.to_device(np.concatenate([raw, np.zeros(32, np.uint8)]))
    tt = O.TernaryTensor(raw, [1024], 2.0, 0.0, 1024)
    assert same_bits(ctx.dequantize_ternary(d_raw, 1024, 2.0).download(np.float32, 1024),
                     O.dequantize_ternary(tt))
    d_q, d_r = ctx.unpack_ternary_i8(d_raw, 16, 64, 64)
    vals = d_q.download(np.int8, 1024).reshape(16, 64)
    assert (vals.ravel() == tt.values()).all()
    assert (d_r.download(np.int32, 16) == vals.astype(np.int32).sum(1)).all()


@pytest.mark.parametrize("K,N", [(3, 2), (16, 16), (64, 64), (100, 37), (130, 200), (256, 1376)])
def test_tile_weights(ctx, K, N):
    w = synth_normal(31, 0.02, (K, N))
    t, vals = oracle_weights(w)
    d_p = ctx.to_device(np.concatenate([t.packed_data, np.zeros(32, np.uint8)]))
    d_t = ctx.tile_weights(d_p, K, N)
    words = d_t.download(np.uint32, ctx.lib.rbn_tiled_bytes(K, N) // 4)
    assert (decode_tiled(words, K, N) == vals).all()


def test_tile_weights_sanitises_invalid_code(ctx):
    raw = np.full(64 * 64 // 4, 0xFF, dtype=np.uint8)     # every field is 11
    d_t = ctx.tile_weights(ctx.to_device(raw), 64, 64)
    assert (decode_tiled(d_t.download(np.uint32, ctx.lib.rbn_tiled_bytes(64, 64) // 4), 64, 64) == 0).all()


# ---- (2) activation quantisation -----------------------------------------------------------

@pytest.mark.parametrize("M,K", [(1, 2048), (1, 4096), (4, 11008), (16, 4096), (3, 100), (5, 1), (2, 67),
                                 (3, 4100), (5, 8192), (4, 16384), (3, 16388), (2, 20000), (300, 1028)])
def test_act_quant_i8(ctx, M, K):
    # K % 4 == 0 up to 16384: the row stays in registers (4, 8 or 16 pieces per thread);
    # other K, or longer rows: two passes over the row
    x = synth_normal(0x5EED0001, 1.0, (M, K))
    if M >= 3:
        x[1, :] = 0.0                  # zero token: guarded scale, all zeros
        x[2, :] = x[2, :] * 1e-9
    q, s, rs = O.act_quant_i8(x)
    d_q, d_s, d_r = ctx.act_quant_i8(ctx.to_device(x), M, K)
    pitch = ctx.act_pitch(K)
    got = d_q.download(np.int8, M * pitch).reshape(M, pitch)
    assert (got[:, :K] == q).all() and (got[:, K:] == 0).all()
    assert same_bits(d_s.download(np.float32, M), s)
    assert (d_r.download(np.int32, M) == rs).all()


def test_act_quant_i8_ties_and_extremes(ctx):
    x = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49],
                  [-127.0, 126.5, -126.5, 125.5, 0.49999997, -0.0, 1e-30, -1e-30]], dtype=np.float32)
    q, s, rs = O.act_quant_i8(x)
    d_q, d_s, d_r = ctx.act_quant_i8(ctx.to_device(x), 2, 8)
    got = d_q.download(np.int8, 2 * ctx.act_pitch(8)).reshape(2, ctx.act_pitch(8))[:, :8]
    assert (got == q).all() and q[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 3]
    assert same_bits(d_s.download(np.float32, 2), s)


@pytest.mark.parametrize("M,K", [(1, 2048), (4, 4096), (64, 64), (7, 99)])
def test_act_quant_ternary_reference_mode(ctx, M, K):
    x = synth_normal(0x5EED0002, 1.0, (M, K))
    t = O.quantize_ternary(x)
    d_q, d_s, d_r, scale, thr = ctx.act_quant_ternary(ctx.to_device(x), M, K)
    pitch = ctx.act_pitch(K)
    got = d_q.download(np.int8, M * pitch).reshape(M, pitch)
    assert bits(scale) == bits(t.scale) and bits(thr) == bits(t.threshold)
    assert (got[:, :K] == t.values().reshape(M, K)).all() and (got[:, K:] == 0).all()
    assert same_bits(d_s.download(np.float32, M), np.full(M, t.scale, np.float32))
    assert (d_r.download(np.int32, M) == got.astype(np.int32).sum(1)).all()


# ---- (3)(4)(5) matmul ------------------------------------------------------------------------

def run_matmul(ctx, fn, x, w, int8_acts=True):
    """Device path from f32 inputs; returns (out, acc, q, act_scale, t_w)."""
    M, K = x.shape
    N = w.shape[1]
    d_w = ctx.to_device(w)
    d_p, w_scale, w_thr, _ = ctx.quantize_ternary(d_w, w.size)
    d_t = ctx.tile_weights(d_p, K, N)
    d_x = ctx.to_device(x)
    if int8_acts:
        acts = ctx.act_quant_i8(d_x, M, K)
    else:
        acts = ctx.act_quant_ternary(d_x, M, K)[:3]
    d_out, d_acc = fn(acts, d_t, w_scale, M, K, N, want_acc=True)
    pitch = ctx.act_pitch(K)
    q = acts[0].download(np.int8, M * pitch).reshape(M, pitch)[:, :K]
    s = acts[1].download(np.float32, M)
    return (d_out.download(np.float32, M * N).reshape(M, N),
            d_acc.download(np.int32, M * N).reshape(M, N), q, s, w_scale)


def check_against_oracle(x, w, out, acc, q, s, w_scale, literal):
    t, vals = oracle_weights(w)
    assert bits(w_scale) == bits(t.scale)
    if literal:   # the reference's own per-element loop
        want_out, want_acc = O.matmul_i8_ternary(q, s, t)
    else:         # same integers through BLAS (see util.exact_int_matmul)
        want_acc = exact_int_matmul(q, vals)
        want_out = epilogue(want_acc, s, t.scale)
    assert (acc == want_acc).all()
    assert same_bits(out, want_out)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 13, 16])
@pytest.mark.parametrize("K,N", [(64, 64), (2048, 2048), (100, 37), (4096, 96), (130, 1376)])
def test_gemv_small_literal(ctx, M, K, N):
    say("gemv", M, K, N)
    x = synth_normal(0x5EED0001 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1001 + K, 0.02, (K, N))
    res = run_matmul(ctx, ctx.gemv, x, w)
    check_against_oracle(x, w, *res, literal=(M * K * N <= 1 << 24))


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 11008), (11008, 4096)])
def test_gemv_decode_sweep_shapes(ctx, M, K, N):
    say("gemv sweep", M, K, N)
    x = synth_normal(0x5EED0001 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1001 + N, 0.02, (K, N))
    res = run_matmul(ctx, ctx.gemv, x, w)
    check_against_oracle(x, w, *res, literal=(M == 1 and K * N <= 4096 * 4096))


@pytest.mark.parametrize("M,K,N", [(1, 8192, 8452), (2, 8192, 8200), (1, 12288, 8200), (2, 15000, 260)])
def test_gemv_long_rows(ctx, M, K, N):
    # k long enough for eight (and more) 16-byte loads per lane: one round of eight in flight
    # for K around 8192, rounds of four beyond; ragged N
    say("gemv long rows", M, K, N)
    x = synth_normal(0x5EED0041 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1041 + N, 0.015, (K, N))
    res = run_matmul(ctx, ctx.gemv, x, w)
    check_against_oracle(x, w, *res, literal=False)


@pytest.mark.parametrize("M,K,N,count", [(1, 4096, 1024, 32), (1, 2048, 2048, 5), (2, 1000, 77, 3), (4, 256, 520, 32),
                                         (1, 11008, 256, 7), (16, 384, 130, 2), (1, 8192, 512, 1), (3, 640, 4096, 9)])
def test_gemv_grouped_every_problem_is_its_own_gemv(ctx, M, K, N, count):
    # `count` independent problems in one launch, each with its own activations, weights, scale
    # and outputs: every one against the oracle's integers (through BLAS) and bit for bit against
    # a launch of its own
    say("gemv grouped", M, K, N, count)
    problems, wants, singles = [], [], []
    for j in range(count):
        x = synth_normal(0x5EED0071 + 7 * j + M, 1.0 + 0.25 * j, (M, K))
        w = synth_normal(0x5EED1071 + 5 * j + N, 0.02, (K, N))
        d_p, w_scale, _, _ = ctx.quantize_ternary(ctx.to_device(w), w.size)
        d_t = ctx.tile_weights(d_p, K, N)
        acts = ctx.act_quant_i8(ctx.to_device(x), M, K)
        t, vals = oracle_weights(w)
        q, s, _ = O.act_quant_i8(x)
        acc = exact_int_matmul(q, vals)
        wants.append((acc, epilogue(acc, s, t.scale)))
        assert bits(w_scale) == bits(t.scale)
        d_out, d_acc = ctx.alloc(4 * M * N), (ctx.alloc(4 * M * N) if j % 2 == 0 else None)
        ctx.lib.rbn_fill_u8(ctx.handle, d_out.ptr, 0xFF, 4 * M * N)
        problems.append((acts, d_t, w_scale, d_out, d_acc))
        singles.append(ctx.gemv(acts, d_t, w_scale, M, K, N)[0].download(np.float32, M * N))
    ctx.gemv_grouped(ctx.gemv_problems(problems), M, K, N)
    ctx.sync()
    for j, ((acts, d_t, w_scale, d_out, d_acc), (want_acc, want_out)) in enumerate(zip(problems, wants)):
        got = d_out.download(np.float32, M * N).reshape(M, N)
        assert same_bits(got, want_out), j
        assert same_bits(got.ravel(), singles[j]), j
        if d_acc is not None:
            assert (d_acc.download(np.int32, M * N).reshape(M, N) == want_acc).all(), j


def test_gemv_grouped_at_the_benchmark_shape(ctx):
    # the benchmark's step: 32 complete GEMVs of M=1, K=4096, N=11008 in one launch, each with its own
    # activations and outputs (four distinct weight matrices, eight problems each), every output
    # against the oracle's integers and epilogue
    M, K, N, count = 1, 4096, 11008, 32
    say("gemv grouped", M, K, N, count)
    mats = []
    for j in range(4):
        w = synth_normal(0x5EED1091 + j, 0.02, (K, N))
        d_p, w_scale, _, _ = ctx.quantize_ternary(ctx.to_device(w), w.size)
        t, vals = oracle_weights(w)
        assert bits(w_scale) == bits(t.scale)
        mats.append((ctx.tile_weights(d_p, K, N), w_scale, t, vals))
        del w
    problems, wants = [], []
    for j in range(count):
        d_t, w_scale, t, vals = mats[j % 4]
        x = synth_normal(0x5EED0091 + j, 1.0 + 0.1 * j, (M, K))
        acts = ctx.act_quant_i8(ctx.to_device(x), M, K)
        q, s, _ = O.act_quant_i8(x)
        acc = exact_int_matmul(q, vals)
        wants.append((acc, epilogue(acc, s, t.scale)))
        d_out, d_acc = ctx.alloc(4 * M * N), ctx.alloc(4 * M * N)
        ctx.lib.rbn_fill_u8(ctx.handle, d_out.ptr, 0xFF, 4 * M * N)
        problems.append((acts, d_t, w_scale, d_out, d_acc))
    ctx.gemv_grouped(ctx.gemv_problems(problems), M, K, N)
    ctx.sync()
    for j, ((acts, d_t, w_scale, d_out, d_acc), (want_acc, want_out)) in enumerate(zip(problems, wants)):
        assert same_bits(d_out.download(np.float32, M * N).reshape(M, N), want_out), j
        assert (d_acc.download(np.int32, M * N).reshape(M, N) == want_acc).all(), j


def test_gemv_grouped_refused_arguments(ctx):
    d = ctx.alloc(4096)
    probs = ctx.gemv_problems([((d, d, d), d, 1.0, d, None)] * 33)
    for count, M in ((0, 1), (33, 1), (1, 0), (1, 17)):
        rc = ctx.lib.rbn_gemv_t2_i8_grouped(ctx.handle, probs, count, M, 64, 64)
        assert rc == _lib.RBN_ERR_INVALID, (count, M)
    assert ctx.lib.rbn_gemv_t2_i8_grouped(ctx.handle, None, 1, 1, 64, 64) == _lib.RBN_ERR_INVALID
    probs[1].d_out = None
    assert ctx.lib.rbn_gemv_t2_i8_grouped(ctx.handle, probs, 2, 1, 64, 64) == _lib.RBN_ERR_INVALID
    assert b"problem 1" in ctx.lib.rbn_last_error()
    probs[1].d_out = d.ptr
    probs[1].d_q = d.ptr + 4
    assert ctx.lib.rbn_gemv_t2_i8_grouped(ctx.handle, probs, 2, 1, 64, 64) == _lib.RBN_ERR_INVALID


def test_gemv_kernel_time_entry(ctx):
    # the measuring variant launches the same kernel and reports the dispatch's own duration
    M, K, N = 1, 2048, 1024
    x = synth_normal(0x5EED0051, 1.0, (M, K))
    w = synth_normal(0x5EED1051, 0.02, (K, N))
    ref = run_matmul(ctx, ctx.gemv, x, w)
    d_w = ctx.to_device(w)
    d_p, w_scale, _, _ = ctx.quantize_ternary(d_w, K * N, _lib.SUM_STRICT_SEQ)
    tiled = ctx.tile_weights(d_p, K, N)
    acts = ctx.act_quant_i8(ctx.to_device(x), M, K)
    d_out = ctx.alloc(4 * M * N)
    us = ctx.gemv_kernel_time_us(acts, tiled, w_scale, M, K, N, d_out)
    assert 0.5 < us < 1000.0
    assert same_bits(d_out.download(np.float32, M * N).reshape(M, N), ref[0])


def test_gemv_reference_mode_config1(ctx):
    # the single-BitLinear configuration, x[1,2048] . W[2048,2048], both operands ternarised as the reference does
    x = synth_normal(0x5EED0001, 1.0, (1, 2048))
    w = synth_normal(0x5EED1001, 0.02, (2048, 2048))
    want_out, want_acc = O.execute_ternary(x, w)
    out, acc = ctx.execute_ternary_matmul(x, w)
    assert (acc == want_acc).all() and same_bits(out, want_out)


@pytest.mark.parametrize("M,K,N", [(17, 64, 64), (64, 64, 64), (128, 256, 128), (200, 130, 100),
                                   (129, 4096, 257), (33, 100, 1376)])
def test_gemm_mfma_small(ctx, M, K, N):
    say("gemm", M, K, N)
    x = synth_normal(0x5EED0003 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1003 + N, 0.02, (K, N))
    res = run_matmul(ctx, ctx.gemm, x, w)
    check_against_oracle(x, w, *res, literal=(M * K * N <= 1 << 23))


@pytest.mark.parametrize("M,K,N", [(100, 1664, 600), (64, 8192, 1024), (300, 2560, 2560), (129, 1100, 4000),
                                   (65, 640, 300)])
def test_gemm_mfma_split_k(ctx, M, K, N):
    # few tiles: the 64-row kernel splits K over up to four workgroups per tile, which meet
    # through the context's workspace (13 K steps -> parts of 5, 5 and 3); run twice, the
    # second launch finds the tickets as the first one left them
    say("gemm split k", M, K, N)
    x = synth_normal(0x5EED000B + M, 1.0, (M, K))
    w = synth_normal(0x5EED100B + N, 0.02, (K, N))
    for _ in range(2):
        res = run_matmul(ctx, ctx.gemm, x, w)
        check_against_oracle(x, w, *res, literal=False)


@pytest.mark.parametrize("M,K,N", [(2000, 128, 11016), (1030, 256, 15000), (1100, 384, 15000),
                                   (2048, 512, 11008)])
def test_gemm_mfma_more_than_one_round(ctx, M, K, N):
    # more tiles than the 512 workgroups that fit the chip at once, with and without the
    # XCD-aware numbering (16 and 9 row tiles), ragged M and N; K steps 1 to 4 cover every
    # exit position of the three-stage ring
    say("gemm rounds", M, K, N)
    x = synth_normal(0x5EED000A + M, 1.0, (M, K))
    w = synth_normal(0x5EED100A + N, 0.02, (K, N))
    res = run_matmul(ctx, ctx.gemm, x, w)
    check_against_oracle(x, w, *res, literal=False)


def test_prefill_gemm_full_shape(ctx):
    # the prefill configuration at its own shape: M=2048, K=4096, N=11008, through the MFMA
    # kernel directly and through the dispatcher (which must pick it)
    M, K, N = 2048, 4096, 11008
    say("gemm full prefill shape", M, K, N)
    assert ctx.lib.rbn_matmul_kernel_choice(M, K, N) == 2
    x = synth_normal(0x5EED0004, 1.0, (M, K))
    w = synth_normal(0x5EED1004, 0.02, (K, N))
    res = run_matmul(ctx, ctx.gemm, x, w)
    check_against_oracle(x, w, *res, literal=False)
    again = run_matmul(ctx, ctx.matmul, x, w)
    assert (again[1] == res[1]).all() and same_bits(again[0], res[0])


class LargeLayer:
    """K=8192, N=28672 weights (sigma 0.015), ternarised by the oracle and by the device once."""

    def __init__(self, ctx):
        self.K, self.N = 8192, 28672
        say("large layer: generating and ternarising 8192 x 28672")
        w = synth_normal(0x5EED1005, 0.015, (self.K, self.N))
        self.t, self.vals = oracle_weights(w)
        d_w = ctx.to_device(w)
        d_p, self.w_scale, self.w_thr, self.survivors = ctx.quantize_ternary(d_w, w.size)
        self.packed = d_p.download(np.uint8, w.size // 4)
        self.d_tiled = ctx.tile_weights(d_p, self.K, self.N)
        ctx.sync()
        d_w.free()
        d_p.free()
        self.vals_f32 = self.vals.astype(np.float32)   # 128 * K < 2^24: f32 products are exact


@pytest.fixture(scope="module")
def large_layer(ctx):
    ll = LargeLayer(ctx)
    yield ll
    ll.d_tiled.free()


def test_large_layer_packed_bytes(ctx, large_layer):
    ll = large_layer
    assert bits(ll.w_thr) == bits(ll.t.threshold) and bits(ll.w_scale) == bits(ll.t.scale)
    assert ll.survivors == ll.t.survivors
    assert (ll.packed == ll.t.packed_data).all()
    words = ll.d_tiled.download(np.uint32, ctx.lib.rbn_tiled_bytes(ll.K, ll.N) // 4)
    assert (decode_tiled(words, ll.K, ll.N) == ll.vals).all()


@pytest.mark.parametrize("M,entry,kernel", [(1, "gemv", 0), (1, "matmul", 0), (8, "matmul", 1), (64, "matmul", 2),
                                            (64, "gemm", 2)])
def test_large_layer_matmul(ctx, large_layer, M, entry, kernel):
    # every token count of the large-layer configuration through the kernel the dispatcher
    # picks for it (M=1: dot8 GEMV, M=8: streaming small-batch kernel, M=64: MFMA tiles)
    ll = large_layer
    say("large layer matmul", M, entry)
    if entry == "matmul":
        assert ctx.lib.rbn_matmul_kernel_choice(M, ll.K, ll.N) == kernel
    x = synth_normal(0x5EED0005 + M, 1.0, (M, ll.K))
    acts = ctx.act_quant_i8(ctx.to_device(x), M, ll.K)
    d_out, d_acc = getattr(ctx, entry)(acts, ll.d_tiled, ll.w_scale, M, ll.K, ll.N, want_acc=True)
    q, s, rs = O.act_quant_i8(x)
    assert (acts[0].download(np.int8, M * ll.K).reshape(M, ll.K) == q).all()
    want_acc = np.rint(q.astype(np.float32) @ ll.vals_f32).astype(np.int32)
    want_out = epilogue(want_acc, s, ll.t.scale)
    assert (d_acc.download(np.int32, M * ll.N).reshape(M, ll.N) == want_acc).all()
    assert same_bits(d_out.download(np.float32, M * ll.N).reshape(M, ll.N), want_out)


@pytest.mark.parametrize("M", [1, 2, 3, 7, 16, 17, 31, 32, 33, 48, 64])
@pytest.mark.parametrize("K,N", [(64, 64), (128, 64), (2048, 2048), (100, 37), (4096, 96), (130, 1376),
                                 (1100, 130)])
def test_skinny_small_literal(ctx, M, K, N):
    say("skinny", M, K, N)
    x = synth_normal(0x5EED0005 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1005 + K, 0.02, (K, N))
    res = run_matmul(ctx, ctx.skinny, x, w)
    check_against_oracle(x, w, *res, literal=(M * K * N <= 1 << 23))


@pytest.mark.parametrize("M", [4, 16, 64])
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 11008), (11008, 4096), (8192, 28672)])
def test_skinny_sweep_shapes(ctx, M, K, N):
    # decode sweep and the large-layer shape; the expected integers come through BLAS
    if (K, N) == (8192, 28672):
        if M == 16:
            pytest.skip("the large-layer shape runs at M = 8 and 64")
        M = 8 if M == 4 else M
    say("skinny sweep", M, K, N)
    x = synth_normal(0x5EED0006 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1006 + N, 0.015 if K == 8192 else 0.02, (K, N))
    res = run_matmul(ctx, ctx.skinny, x, w)
    check_against_oracle(x, w, *res, literal=False)


@pytest.mark.parametrize("M,K,N", [(64, 256, 16400), (33, 192, 16384), (50, 128, 20000)])
def test_skinny_two_column_groups_per_wave(ctx, M, K, N):
    # wide matrices with four row tiles take two groups of 64 columns per wave; odd group
    # counts and ragged N exercise the clamped last group
    x = synth_normal(0x5EED0009 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1009 + N, 0.02, (K, N))
    res = run_matmul(ctx, ctx.skinny, x, w)
    check_against_oracle(x, w, *res, literal=False)


def test_skinny_saturated_activations(ctx):
    M, K, N = 48, 8192, 128
    x = np.where(synth_normal(7, 1.0, (M, K)) > 0, 1.0, -1.0).astype(np.float32)
    w = np.where(synth_normal(8, 1.0, (K, N)) > 0, 1.0, -1.0).astype(np.float32)
    res = run_matmul(ctx, ctx.skinny, x, w)
    check_against_oracle(x, w, *res, literal=False)
    assert np.abs(res[1]).max() > 127 * 100


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 16, 17, 64, 65, 128])
def test_matmul_dispatch_agrees_across_kernels(ctx, M):
    # rbn_matmul_t2_i8 picks gemv / skinny / mfma by M; every kernel that accepts the shape
    # must return the same bits
    K, N = 1024, 520
    x = synth_normal(0x5EED0007 + M, 1.0, (M, K))
    w = synth_normal(0x5EED1007, 0.02, (K, N))
    ref = run_matmul(ctx, ctx.matmul, x, w)
    check_against_oracle(x, w, *ref, literal=False)
    fns = [ctx.gemm]
    if M <= 16:
        fns.append(ctx.gemv)
    if M <= 64:
        fns.append(ctx.skinny)
    for fn in fns:
        got = run_matmul(ctx, fn, x, w)
        assert (got[1] == ref[1]).all() and same_bits(got[0], ref[0])


def test_matmul_two_tokens_wide_short_k(ctx):
    # two tokens go to the streaming kernel when k is short and the matrix wide, to the GEMV
    # otherwise: same bits either way (2560 x 13824 is the decoder's gate/up projection)
    M, K, N = 2, 2560, 13824
    assert ctx.lib.rbn_matmul_kernel_choice(M, K, N) == 1 and ctx.lib.rbn_matmul_kernel_choice(M, 4096, N) == 0
    x = synth_normal(0x5EED0031, 1.0, (M, K))
    w = synth_normal(0x5EED1031, 0.02, (K, N))
    ref = run_matmul(ctx, ctx.matmul, x, w)
    check_against_oracle(x, w, *ref, literal=False)
    got = run_matmul(ctx, ctx.gemv, x, w)
    assert (got[1] == ref[1]).all() and same_bits(got[0], ref[0])


def test_gemm_mfma_saturated_activations(ctx):
    # every activation at +-127/-128 and dense +-1 weights: the largest |acc| the path can see
    M, K, N = 64, 4096, 128
    x = np.where(synth_normal(5, 1.0, (M, K)) > 0, 1.0, -1.0).astype(np.float32)
    w = np.where(synth_normal(6, 1.0, (K, N)) > 0, 1.0, -1.0).astype(np.float32)
    res = run_matmul(ctx, ctx.gemm, x, w)
    check_against_oracle(x, w, *res, literal=False)
    assert np.abs(res[1]).max() > 127 * 100


def test_reference_execute_64_cubed(ctx):
    # the only shape the reference's provider compiles kernels for (provider.rs:157-159)
    a = synth_normal(41, 1.0, (64, 64))
    b = synth_normal(42, 0.02, (64, 64))
    want_out, want_acc = O.execute_ternary(a, b)
    out, acc = ctx.execute_ternary_matmul(a, b)
    assert (acc == want_acc).all() and same_bits(out, want_out)


# ---- error behaviour ------------------------------------------------------------------------------

def test_error_paths(ctx):
    d = ctx.alloc(1024)
    with pytest.raises(_lib.RbnError) as e:
        ctx.gemv((d, d, d), d, 1.0, 17, 64, 64)
    assert e.value.code == _lib.RBN_ERR_INVALID and "M <= 16" in e.value.message
    with pytest.raises(_lib.RbnError) as e:
        ctx.skinny((d, d, d), d, 1.0, 65, 64, 64)
    assert e.value.code == _lib.RBN_ERR_INVALID and "M <= 64" in e.value.message
    with pytest.raises(_lib.RbnError):
        ctx.gemv((d, d, d), d, 1.0, 0, 64, 64)
    rc = ctx.lib.rbn_quantize_ternary(ctx.handle, d.ptr + 4, 16, 0, d.ptr, None, None, None)
    assert rc == _lib.RBN_ERR_INVALID
    rc = ctx.lib.rbn_gemv_t2_i8(ctx.handle, None, None, None, None, 1.0, 1, 64, 64, None, None)
    assert rc == _lib.RBN_ERR_INVALID and b"null pointer" in ctx.lib.rbn_last_error()
    assert ctx.lib.rbn_sync(None) == _lib.RBN_ERR_INVALID


def test_synchronising_entry_points_refuse_a_capturing_stream(ctx):
    x = synth_normal(3, 1.0, (4, 64))
    d_x = ctx.to_device(x)
    bufs = ctx.alloc_acts(4, 64)
    ctx.act_quant_ternary(d_x, 4, 64, bufs=bufs)          # sizes the context's buffers beforehand
    out = np.empty((4, 4), np.float32)
    ctx.graph_begin()
    try:
        with pytest.raises(_lib.RbnError) as e:
            ctx.act_quant_ternary(d_x, 4, 64, bufs=bufs)
        assert e.value.code == _lib.RBN_ERR_INVALID and "captured" in e.value.message
        rc = ctx.lib.rbn_execute_ternary_matmul(ctx.handle, x.ctypes.data, x.T.copy().ctypes.data, 4, 4, 64, 0,
                                                out.ctypes.data, None)
        assert rc == _lib.RBN_ERR_INVALID
        ctx.act_quant_i8(d_x, 4, 64, bufs)                # an asynchronous call is recorded as before
    finally:
        g = ctx.graph_end()
    ctx.graph_launch(g)
    ctx.sync()
    ctx.graph_destroy(g)
    q, s, rs = O.act_quant_i8(x)
    assert (bufs[0].download(np.int8, 4 * ctx.act_pitch(64)).reshape(4, -1)[:, :64] == q).all()


def test_mfma_probe_reports_a_plausible_rate(ctx):
    const = ctx.probe_mfma_i8(0)
    tern = ctx.probe_mfma_i8(1)
    assert 1000 < tern <= const * 1.05 < 5500
    with pytest.raises(_lib.RbnError):
        ctx.probe_mfma_i8(7)


def test_captured_graph_replays_match_eager_results(ctx):
    """A graph of matmuls (GEMV, small-batch kernel with its cross-workgroup k split and
    ticket counters, MFMA GEMM) replayed several times, with eager work in between, gives
    the eager bits on every replay."""
    cases = []
    for M, K, N in ((1, 2048, 2048), (8, 4096, 1024), (16, 11008, 512), (200, 512, 384)):
        x = synth_normal(0x5EED0008 + M, 1.0, (M, K))
        w = synth_normal(0x5EED1008 + N, 0.02, (K, N))
        d_w = ctx.to_device(w)
        d_p, w_scale, _, _ = ctx.quantize_ternary(d_w, w.size)
        d_t = ctx.tile_weights(d_p, K, N)
        acts = ctx.act_quant_i8(ctx.to_device(x), M, K)
        eager, _ = ctx.matmul(acts, d_t, w_scale, M, K, N)
        cases.append((M, K, N, acts, d_t, w_scale, eager.download(np.float32, M * N), ctx.alloc(4 * M * N)))
    ctx.sync()
    ctx.graph_begin()
    for M, K, N, acts, d_t, w_scale, _, d_out in cases:
        ctx.matmul(acts, d_t, w_scale, M, K, N, d_out=d_out)
    g = ctx.graph_end()
    for rep in range(4):
        for c in cases:
            check_fill = ctx.lib.rbn_fill_u8(ctx.handle, c[7].ptr, 0xFF, 4 * c[0] * c[2])
            assert check_fill == 0
        ctx.graph_launch(g)
        ctx.sync()
        for M, K, N, acts, d_t, w_scale, want, d_out in cases:
            assert same_bits(d_out.download(np.float32, M * N), want), (rep, M, K, N)
        # eager work between replays (uses the same workspace and ticket counters)
        M, K, N, acts, d_t, w_scale, want, _ = cases[rep % len(cases)]
        again, _ = ctx.matmul(acts, d_t, w_scale, M, K, N)
        assert same_bits(again.download(np.float32, M * N), want)
    ctx.graph_destroy(g)

"""CPU-side checks: the C ABI loads and exports what the header declares, the host-only
helpers follow the reference's size rules, the exact sequential-sum arithmetic that the
HIP kernels share (ronn_amd/csrc/seqsum_core.h) reproduces a literal f32 fold, and the
test helpers agree with the literal oracle.  No GPU work is launched here.
"""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

from oracle import oracle as O
from ronn_amd import _lib
from util import epilogue, exact_int_matmul

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__ as g
        g.build()
    return _lib.load()


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "ronn_bitnet_hip.h")).read()
    declared = set(re.findall(r"\b(rbn_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 35
    for name in sorted(declared):
        assert hasattr(lib, name), "%s is declared in the header but not exported" % name
    # and the Python binding covers exactly the declared set
    assert declared == set(_lib.SIGNATURES)


def test_matmul_dispatch_rule(lib):
    # gemv for one or two tokens and for up to four on small matrices; the small-batch kernel
    # up to 16, 32 or 64 by the size of the matrix
    choice = lib.rbn_matmul_kernel_choice
    GEMV, SKINNY, MFMA = 0, 1, 2
    assert [choice(m, 4096, 11008) for m in (1, 2, 3, 4, 16, 32, 33, 64, 65)] == \
        [GEMV, GEMV, SKINNY, SKINNY, SKINNY, SKINNY, MFMA, MFMA, MFMA]
    assert [choice(m, 8192, 28672) for m in (1, 2, 3, 8, 16, 17, 64)] == \
        [GEMV, GEMV, SKINNY, SKINNY, SKINNY, MFMA, MFMA]
    assert [choice(m, 4096, 4096) for m in (3, 4, 5, 64, 65, 2048)] == [GEMV, GEMV, SKINNY, SKINNY, MFMA, MFMA]
    assert [choice(m, 2560, 13824) for m in (1, 2)] == [GEMV, SKINNY]   # short k, wide: two tokens stream


def test_provider_abi_exports(lib):
    from ronn_amd import bitnet
    header = open(os.path.join(ROOT, "include", "ronn_bitnet_provider.h")).read()
    declared = set(re.findall(r"\b(rbp_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    for name in sorted(declared):
        assert hasattr(lib, name), "%s is declared in the header but not exported" % name
    assert declared == set(bitnet.PROVIDER_SIGNATURES)


def test_provider_without_device_raises(lib):
    if lib.rbn_device_count() > 0:
        pytest.skip("a GPU is visible here")
    from ronn_amd import bitnet
    with pytest.raises(bitnet.Error, match="no HIP device"):
        bitnet.create_bitnet_provider()


def test_no_device_is_reported_not_faked(lib):
    if lib.rbn_device_count() > 0:
        pytest.skip("a GPU is visible here")
    h = C.c_void_p()
    rc = lib.rbn_ctx_create(0, C.byref(h))
    assert rc == _lib.RBN_ERR_NO_DEVICE and h.value is None
    assert b"no HIP device" in lib.rbn_last_error()
    from ronn_amd.device import Context
    with pytest.raises(_lib.RbnError):
        Context(0)


def test_size_rules_match_reference_allocator(lib):
    # allocator.rs:231-235, :257-261, :285-288 and the oracle's restatement of :39-75
    assert lib.rbn_tensor_bytes(1000, _lib.DT_BOOL) == 125
    assert lib.rbn_tensor_bytes(100, _lib.DT_U8) == 25
    assert lib.rbn_tensor_bytes(32 * 32, _lib.DT_BOOL) == 128
    for dt in range(10):
        for n in (0, 1, 3, 4, 5, 1000, 4097):
            assert lib.rbn_tensor_bytes(n, dt) == O.packed_size([n], dt)
        assert lib.rbn_tensor_alignment(dt) == O.alignment(dt)
    assert lib.rbn_packed_capacity(100) >= 25 and lib.rbn_packed_capacity(100) % 16 == 0
    assert lib.rbn_tiled_bytes(4096, 11008) == 4096 * 11008 // 4
    assert lib.rbn_tiled_bytes(3, 2) == 128 * 64 // 4         # padded to 128 x 64
    assert lib.rbn_act_pitch(2048) == 2048 and lib.rbn_act_pitch(100) == 128


def test_synthetic_generator_is_deterministic_and_normal(lib):
    from ronn_amd.device import synth_normal
    a = synth_normal(7, 0.02, (100000,))
    b = synth_normal(7, 0.02, (100000,))
    assert (a == b).all()
    # a range generated in two pieces equals the whole (counter-based)
    c = np.concatenate([synth_normal(7, 0.02, (33333,)), synth_normal(7, 0.02, (66667,), first=33333)])
    assert (a == c).all()
    assert abs(float(a.mean())) < 3e-4 and abs(float(a.std()) - 0.02) < 2e-4
    assert not (a == synth_normal(8, 0.02, (100000,))).any()


@pytest.fixture(scope="module")
def seqsum(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("seq") / "seqsum_host.so")
    src = os.path.join(ROOT, "tests", "host", "seqsum_host.cpp")
    subprocess.run(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", out, src], check=True)
    L = C.CDLL(out)
    L.seqsum_host.restype = C.c_float
    L.seqsum_host.argtypes = [C.c_void_p, C.c_uint64, C.c_int, C.c_float, C.POINTER(C.c_uint64),
                              C.POINTER(C.c_uint64)]
    L.seqsum_literal.restype = C.c_float
    L.seqsum_literal.argtypes = [C.c_void_p, C.c_uint64, C.c_int, C.c_float]
    L.seqsum_compare_term_splits.restype = C.c_uint64
    L.seqsum_compare_term_splits.argtypes = [C.c_uint64, C.c_uint64]
    L.seqsum_compare_block_forms.restype = C.c_uint64
    L.seqsum_compare_block_forms.argtypes = [C.c_uint64, C.c_uint64, C.POINTER(C.c_uint64)]
    L.seqsum_compare_map16.restype = C.c_uint64
    L.seqsum_compare_map16.argtypes = [C.c_uint64, C.c_uint64, C.POINTER(C.c_uint64)]
    L.seqsum_once_stats.restype = None
    L.seqsum_once_stats.argtypes = [C.POINTER(C.c_uint64)] * 3
    L.seqsum_check_map_slots.restype = C.c_uint64
    L.seqsum_check_map_slots.argtypes = [C.c_uint32]
    return L


def _cases():
    rng = np.random.default_rng(1)
    yield "weights", rng.normal(0, 0.02, 4096 * 3 + 17)
    yield "config1", rng.normal(0, 0.02, 2048 * 2048)
    yield "acts", rng.normal(0, 1, 4096)
    yield "zeros", np.zeros(10000)
    yield "ones", np.full(100000, 1.0)
    yield "ones_past_2^24", np.full((1 << 24) + 70000, 1.0)
    yield "denormals", rng.normal(0, 1e-40, 100000)
    yield "huge", rng.normal(0, 1e30, 100000)
    yield "overflow", rng.normal(0, 3e37, 100000)
    x = rng.normal(0, 1, 100000); x[5000] = np.inf
    yield "inf", x
    x = x.copy(); x[90000] = np.nan
    yield "inf_then_nan", x
    x = rng.normal(0, 1, 100000); x[5000] = np.inf; x[5100] = np.nan
    yield "inf_then_nan_same_block", x
    x = rng.normal(0, 1, 100000); x[70000] = np.nan
    yield "nan", x
    # growth that changes by orders of magnitude: the exponent prediction of the multi-binade windows fails
    x = rng.normal(0, 1, 700000)
    for lo, hi, f in ((0, 40000, 1e-6), (40000, 100000, 1.0), (100000, 230000, 1e-3), (230000, 350000, 300.0),
                      (350000, 520000, 0.0), (520000, 700000, 2e-2)):
        x[lo:hi] *= f
    yield "steps", x
    yield "lognormal", rng.lognormal(0, 6, 500000)
    yield "cauchy", np.abs(rng.standard_cauchy(300000))
    yield "ties_even", np.concatenate([[2.0 ** 20], np.full(300000, 2.0 ** -4)])
    yield "ties_odd", np.concatenate([[2.0 ** 20 + 2.0 ** -3], np.full(300000, 2.0 ** -4)])
    for n in (1, 2, 15, 16, 17, 4095, 4096, 4097):
        yield "n%d" % n, rng.normal(0, 1, n)


@pytest.mark.parametrize("name,x", list(_cases()), ids=lambda v: v if isinstance(v, str) else "")
def test_parallel_sequential_sum_is_bit_exact(seqsum, name, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    for mask, thr in ((0, 0.0), (1, float(np.median(np.abs(x[np.isfinite(x)]))) if x.size else 0.0)):
        got = np.float32(seqsum.seqsum_host(x.ctypes.data, x.size, mask, thr, None, None))
        want = np.float32(seqsum.seqsum_literal(x.ctypes.data, x.size, mask, thr))
        assert got.view(np.uint32) == want.view(np.uint32) or (np.isnan(got) and np.isnan(want)), \
            "%s mask=%d: %r vs %r" % (name, mask, got, want)


def test_transposed_map_slots_match_the_runs_of_the_window_end_kernel(seqsum):
    # every block of a window at slot i * 1024 + t of its thread's run, one block per slot, inside the buffer
    for win in (1, 2, 1023, 1024, 1025, 2047, 2048, 2049, 4565, 8192, 8193, 32767, 32768, 32769, 45005,
                65535, 65536, 65537, 100_000, 1_000_003):
        assert seqsum.seqsum_check_map_slots(win) == 0, win


def test_a_window_longer_than_one_stretch_is_walked_stretch_by_stretch(seqsum):
    # one term of 1.0 per block behind a first term of 2^16: the window behind block 8192 is 63,000 blocks
    # long and S leaves its binade beyond block 57,000 of it (second stretch of 32,768 maps); all sums exact
    blocks = 72_000
    x = np.zeros(blocks * 4096, dtype=np.float32)
    x[5::4096] = -1.0
    x[0] = 65536.0
    it = C.c_uint64()
    got = np.float32(seqsum.seqsum_host(x.ctypes.data, x.size, 0, 0.0, C.byref(it), None))
    assert got == np.float32(65536 + blocks) and it.value == 5


def test_two_barrier_replay_agrees_with_the_general_one(seqsum):
    # every crossing block that the short replay (one crossing, one binade up) resolves must come out as the
    # general replay has it: state after the block, state behind the crossing chunk, chunks folded up to it
    rng = np.random.default_rng(11)
    for scale, n in ((0.02, 3_000_000), (1.0, 700_000), (1e-3, 2_000_000), (30.0, 400_001)):
        x = (rng.standard_normal(n) * scale).astype(np.float32)
        x[rng.integers(0, n, 50)] *= 1000.0          # a few terms that jump over binades
        for mask, thr in ((0, 0.0), (1, float(np.median(np.abs(x))))):
            got = np.float32(seqsum.seqsum_host(x.ctypes.data, n, mask, thr, None, None))
            want = np.float32(seqsum.seqsum_literal(x.ctypes.data, n, mask, thr))
            assert got.view(np.uint32) == want.view(np.uint32)
    tried, used, differs = C.c_uint64(), C.c_uint64(), C.c_uint64()
    seqsum.seqsum_once_stats(C.byref(tried), C.byref(used), C.byref(differs))
    assert differs.value == 0 and used.value > 20 and tried.value >= used.value


def test_float_and_integer_term_splits_agree(seqsum):
    # seq_append_abs (float split, used for es >= 26) against seq_append (integer split)
    assert seqsum.seqsum_compare_term_splits(3_000_000, 1) == 0
    assert seqsum.seqsum_compare_term_splits(1_000_000, 2) == 0


def test_map_of_sixteen_terms_equals_term_by_term(seqsum):
    # seq_map16 (one sum of sixteen roundings unless a term is an exact tie) against sixteen seq_append_abs
    ties = C.c_uint64()
    assert seqsum.seqsum_compare_map16(400_000, 5, C.byref(ties)) == 0
    assert 1000 < ties.value < 399_000      # both branches were taken


def test_a_block_without_ties_is_the_sum_of_its_roundings_in_any_order(seqsum):
    # the maps kernel's streaming form (coalesced loads, plain sums) against the ordered composition
    used = C.c_uint64()
    assert seqsum.seqsum_compare_block_forms(600, 9, C.byref(used)) == 0
    assert 100 < used.value < 600           # blocks with and without ties were drawn


def test_sequential_sum_traffic_is_bounded(seqsum):
    # the window policy re-reads at most ~2x the data on the sizes that matter
    x = np.random.default_rng(2).normal(0, 0.02, 4096 * 4096).astype(np.float32)
    it, rd = C.c_uint64(), C.c_uint64()
    seqsum.seqsum_host(x.ctypes.data, x.size, 0, 0.0, C.byref(it), C.byref(rd))
    assert rd.value <= 2.0 * x.size and it.value <= 40


def test_blas_helper_equals_literal_oracle_loop():
    rng = np.random.default_rng(4)
    for m, k, n in ((1, 300, 40), (5, 1000, 33), (16, 4096, 16)):
        x = rng.normal(0, 1, (m, k)).astype(np.float32)
        w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
        q, s, _ = O.act_quant_i8(x)
        t = O.quantize_ternary(w)
        out, acc = O.matmul_i8_ternary(q, s, t)
        acc2 = exact_int_matmul(q, t.values().reshape(k, n))
        assert (acc == acc2).all()
        assert (out.view(np.uint32) == epilogue(acc2, s, t.scale).view(np.uint32)).all()


# ---- packed-weight files (no GPU needed) ----------------------------------------------------------

def test_packed_weight_file_round_trip(lib, tmp_path):
    from ronn_amd import bitnet
    rng = np.random.default_rng(9)
    for shape in ((64, 64), (7, 13), (5,), (2, 3, 4), (1, 1)):
        w = rng.normal(0, 0.02, shape).astype(np.float32)
        t = O.quantize_ternary(w)
        tt = bitnet.TernaryTensor.from_parts(t.packed_data, list(shape), t.scale, t.threshold)
        path = tmp_path / ("w_%s.rbnt" % "x".join(map(str, shape)))
        tt.save(path)
        back = bitnet.TernaryTensor.load(path)
        assert back.shape == list(shape) and back.element_count == w.size
        assert (back.packed_data == t.packed_data).all()
        assert np.float32(back.scale).view(np.uint32) == np.float32(t.scale).view(np.uint32)
        assert np.float32(back.threshold).view(np.uint32) == np.float32(t.threshold).view(np.uint32)
        assert [back.get_value(i) for i in range(min(w.size, 50))] == list(t.values()[:50])
        raw = open(path, "rb").read()
        assert raw[:8] == b"RBNTERN1" and len(raw) == 40 + 8 * len(shape) + (w.size + 3) // 4 + 4


def test_packed_weight_file_rejects_damage(lib, tmp_path):
    from ronn_amd import bitnet
    w = np.random.default_rng(10).normal(0, 0.02, (16, 9)).astype(np.float32)
    t = O.quantize_ternary(w)
    good = tmp_path / "good.rbnt"
    bitnet.TernaryTensor.from_parts(t.packed_data, [16, 9], t.scale, t.threshold).save(good)
    raw = bytearray(open(good, "rb").read())
    cases = {"flipped payload bit": (60, raw[60] ^ 4), "bad magic": (0, ord("X")), "version": (8, 2)}
    for name, (off, val) in cases.items():
        bad = bytearray(raw)
        bad[off] = val
        p = tmp_path / "bad.rbnt"
        open(p, "wb").write(bad)
        with pytest.raises(bitnet.Error):
            bitnet.TernaryTensor.load(p)
    open(tmp_path / "short.rbnt", "wb").write(raw[:-7])
    with pytest.raises(bitnet.Error, match="size|truncated"):
        bitnet.TernaryTensor.load(tmp_path / "short.rbnt")
    with pytest.raises(bitnet.Error, match="cannot open"):
        bitnet.TernaryTensor.load(tmp_path / "missing.rbnt")
    # from_parts enforces the quantiser's invariants
    with pytest.raises(bitnet.Error, match="packed size"):
        bitnet.TernaryTensor.from_parts(t.packed_data[:-1], [16, 9], 1.0, 0.0)
    odd = O.quantize_ternary(np.ones(5, np.float32))
    dirty = odd.packed_data.copy()
    dirty[-1] |= 0x80
    with pytest.raises(bitnet.Error, match="tail bits"):
        bitnet.TernaryTensor.from_parts(dirty, [5], 1.0, 0.0)


def test_small_batch_launch_shapes_meet_the_kernels_assumptions(lib):
    """The small-batch kernels trust their launch shape: a wave whose share of k were empty would
    read outside the matrix.  The rule that picks the shape is pure arithmetic, so it is swept
    here: every wave owns at least one step, no workgroup has more than 16 waves or 128 KiB of
    LDS, and the steps cover K exactly."""
    shape = (C.c_int32 * 8)()
    ks = list(range(1, 300)) + [511, 512, 513, 1000, 2048, 2560, 4096, 6912, 8192, 11008, 12288, 15000,
                                16384, 28672, 100000, 1 << 20]
    ns = [1, 3, 37, 64, 65, 130, 256, 1024, 1376, 2560, 4096, 8128, 8192, 11008, 16384, 28672, 32000, 200000]
    checked = 0
    for M in (1, 2, 7, 8, 9, 16, 17, 32, 33, 64):
        for K in ks:
            for N in ns:
                rc = lib.rbn_skinny_launch_shape(M, K, N, shape)
                assert rc == 0, (M, K, N, list(shape))
                ring, groups, splits, waves, step_k, steps, longest, lds = list(shape)
                kpad = (K + 127) // 128 * 128
                assert ring == (1 if M <= 16 else 0) and step_k == (128 if ring else 64)
                assert steps * step_k == kpad
                assert 1 <= waves <= 16 and splits >= 1 and splits * waves <= steps
                assert longest == -(-steps // (splits * waves)) and longest >= 1
                assert 0 < lds <= 128 * 1024
                assert groups >= 1 and groups * 64 * (2 if (M > 32 and -(-N // 64) >= 256) else 1) >= N
                if ring:
                    # workgroup g owns the quads [g*nquads/groups, (g+1)*nquads/groups): 1 to 16 of them
                    nquads = -(-N // 64) * 16
                    assert groups <= nquads and -(-nquads // groups) <= 16 and groups <= max(256, nquads // 16)
                # the partition the kernels use: wave w of g takes steps [w*steps/g, (w+1)*steps/g)
                g = splits * waves
                assert all((w + 1) * steps // g > w * steps // g for w in range(g))
                if splits > 1:
                    assert groups <= 1024 and groups * splits * -(-M // 16) <= 16384
                checked += 1
    assert checked > 50000
    for bad in ((0, 64, 64), (65, 64, 64), (1, 0, 64), (1, 64, 0)):
        assert lib.rbn_skinny_launch_shape(*bad, shape) == _lib.RBN_ERR_INVALID
    # the recorded shapes of the decode sweep
    lib.rbn_skinny_launch_shape(16, 4096, 11008, shape)
    assert list(shape)[:7] == [1, 172, 1, 16, 128, 32, 2]
    lib.rbn_skinny_launch_shape(16, 4096, 4096, shape)
    assert list(shape)[:4] == [1, 256, 1, 16]                # four quads each instead of a split along k
    lib.rbn_skinny_launch_shape(16, 11008, 4096, shape)
    assert list(shape)[:3] == [1, 64, 4]                     # long k: split along k, sixteen quads each
    lib.rbn_skinny_launch_shape(4, 2560, 2560, shape)
    assert list(shape)[:3] == [1, 40, 1]
    lib.rbn_skinny_launch_shape(8, 8192, 28672, shape)
    assert list(shape)[:4] == [1, 448, 1, 4]                 # sixteen quads each; more groups than CUs: four waves, several workgroups per CU

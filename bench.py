#!/usr/bin/env python3
"""Benchmark of the BitNet ternary hot path on one MI355X.

Headline (the JSON line's `value`): decode-regime ternary GEMV at K=4096, N=11008, M=1 (the
FFN up/gate shape of the decode sweep), int8 activations and tiled 2-bit weights already
resident in HBM.  One step = one batch of 32 complete, independent GEMVs - each with its own
activation vector, its own weight buffer and its own output - issued as ONE launch
(rbn_gemv_t2_i8_grouped), because a single GEMV of 11 MB is shorter than the gap between two
launches plus the ramp of its first loads; the one-GEMV-per-launch figure is reported next to
it in `extra`.  Consecutive steps alternate between two such batches: 64 weight buffers
(> 700 MB, against 256 MiB of Infinity Cache), so every GEMV streams its weights from HBM;
launches are replayed from captured HIP graphs.  Before anything
is timed every problem's int32 accumulators and f32 bits are compared with the CPU oracle's
integers, and every extra row is gated the same way at its own shape.

`roofline` prices the GEMV kernel's algorithmic bytes (K*N/4 + M*K + 4*M + 4*M*N per GEMV, times
the GEMVs of a launch) against the 8 TB/s HBM peak, with HIP events recorded on the library's own
stream around the timed region.  `cpu_baseline` times the CPU oracle (a C restatement of the
reference's scalar loops; the Rust original cannot be built here) on one host core.
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0     # MI355X published dense int8 MFMA rate (5.0 POP/s)
MALL_BYTES = 256 << 20
GROUP = 32                  # GEMVs per grouped launch (RBN_GEMV_GROUP_MAX)
HEADLINE_PROFILE = "gemv_grouped_m1_k4096_n11008.md"


def gemv_bytes(M, K, N):
    return K * N // 4 + M * K + 4 * M + 4 * M * N


def profile_facts(name):
    """The machine-readable block (```json ... ```) at the end of a summary under profiles/:
    what rocprofv3 measured for a kernel (name, average duration, HBM traffic per launch)."""
    try:
        text = open(os.path.join(ROOT, "profiles", name)).read()
    except OSError:
        return {}
    m = re.findall(r"```json\s*(\{.*?\})\s*```", text, re.S)
    try:
        return json.loads(m[-1]) if m else {}
    except ValueError:
        return {}


def exact_int_matmul(q, vals_f):
    """int32 product of int8 activations and ternary values through BLAS: with |q| <= 128 and
    |w| <= 1 every partial sum stays below 2^24 for K < 131072, so f32 arithmetic is exact."""
    return np.rint(q.astype(np.float32) @ vals_f).astype(np.int32)


def epilogue(acc, act_scale, w_scale):
    """kernels.rs:168: (acc as f32 * a.scale) * b.scale, left to right, in f32."""
    r = acc.astype(np.float32) * np.asarray(act_scale, dtype=np.float32).reshape(-1, 1)
    return (r.astype(np.float32) * np.float32(w_scale)).astype(np.float32)


class Weights:
    """One [K,N] weight matrix ternarised on the device (strict sequential sums unless told
    otherwise), tiled, and copied into as many buffers as `rotate_bytes` asks for."""

    def __init__(self, ctx, K, N, sigma, seed, rotate_bytes, mode=None, keep_host=False, n_buffers=None,
                 d_w=None):
        from ronn_amd import _lib
        from ronn_amd.device import synth_normal
        self.ctx, self.K, self.N = ctx, K, N
        given = d_w is not None           # an f32 matrix already on the device (the caller keeps it)
        w = None if given else synth_normal(seed, sigma, (K, N))
        d_w = d_w if given else ctx.to_device(w)
        mode = _lib.SUM_STRICT_SEQ if mode is None else mode
        d_p, self.w_scale, self.w_thr, _ = ctx.quantize_ternary(d_w, K * N, mode)
        self.tiled_bytes = ctx.lib.rbn_tiled_bytes(K, N)
        first = ctx.tile_weights(d_p, K, N)
        nbuf = n_buffers if n_buffers is not None else max(1, -(-rotate_bytes // self.tiled_bytes))
        self.tiled = [first]
        for _ in range(nbuf - 1):
            b = ctx.alloc(self.tiled_bytes)
            _lib.check(ctx.lib.rbn_d2d(ctx.handle, b.ptr, first.ptr, self.tiled_bytes))
            self.tiled.append(b)
        ctx.sync()
        if not given:
            d_w.free()
        d_p.free()
        self.w = w if keep_host else None

    def oracle(self):
        """(oracle TernaryTensor, ternary values as f32 [K,N]) of the host copy."""
        from oracle import oracle as O
        t = O.quantize_ternary(self.w)
        return t, t.values().reshape(self.K, self.N).astype(np.float32)


class Workload:
    """Quantised operands of one (M, K, N) problem, resident on the device."""

    def __init__(self, ctx, M, K, N, sigma_w, seed, rotate_bytes=MALL_BYTES + (64 << 20), mode=None,
                 want_host=False, weights=None):
        from ronn_amd.device import synth_normal
        self.ctx, self.M, self.K, self.N = ctx, M, K, N
        self.x = synth_normal(0x5EED0001 + seed, 1.0, (M, K))
        self.weights = weights or Weights(ctx, K, N, sigma_w, 0x5EED1001 + seed, rotate_bytes, mode, want_host)
        self.tiled, self.tiled_bytes, self.w_scale = self.weights.tiled, self.weights.tiled_bytes, self.weights.w_scale
        self.acts = ctx.act_quant_i8(ctx.to_device(self.x), M, K)
        self.d_out = ctx.alloc(4 * M * N)
        self.d_acc = ctx.alloc(4 * M * N)
        ctx.sync()

    def launch(self, fn, i, with_acc=False):
        fn(self.acts, self.tiled[i % len(self.tiled)], self.w_scale, self.M, self.K, self.N,
           d_out=self.d_out, d_acc=self.d_acc if with_acc else None, want_acc=False)

    def results(self, fn, buffer=0):
        self.launch(fn, buffer, with_acc=True)
        self.ctx.sync()
        n = self.M * self.N
        return (self.d_out.download(np.float32, n).reshape(self.M, self.N),
                self.d_acc.download(np.int32, n).reshape(self.M, self.N))

    def gate(self, fn, oracle_pair, what):
        """Bit-exact check of `fn` on this workload against the oracle's integers (BLAS) - on the
        first and on the last weight buffer."""
        from oracle import oracle as O
        t, vals_f = oracle_pair
        q, s, _ = O.act_quant_i8(self.x)
        want_acc = exact_int_matmul(q, vals_f)
        want_out = epilogue(want_acc, s, t.scale)
        ok = np.float32(self.w_scale).view(np.uint32) == np.float32(t.scale).view(np.uint32)
        for b in sorted({0, len(self.tiled) - 1}):
            out, acc = self.results(fn, b)
            ok = ok and bool((acc == want_acc).all()) and bool((out.view(np.uint32) == want_out.view(np.uint32)).all())
        if not ok:
            print("bench.py: PARITY FAILURE against the CPU oracle in %s" % what, file=sys.stderr)
            sys.exit(1)
        return True


class GroupedWorkload:
    """`n_problems` independent GEMVs of one shape: problem j has its own activation rows, its own
    weight buffer (a copy of matrix j % distinct) and its own outputs."""

    def __init__(self, ctx, M, K, N, sigma_w, n_problems, distinct=2, keep_host=True):
        from ronn_amd import _lib
        from ronn_amd.device import synth_normal
        self.ctx, self.M, self.K, self.N, self.n = ctx, M, K, N, n_problems
        per = -(-n_problems // distinct)
        self.mats = [Weights(ctx, K, N, sigma_w, 0x5EED1002 + 17 * d, 0, keep_host=keep_host, n_buffers=per)
                     for d in range(distinct)]
        self.tiled_bytes = self.mats[0].tiled_bytes
        self.x = synth_normal(0x5EED0002, 1.0, (n_problems * M, K))
        self.acts = ctx.act_quant_i8(ctx.to_device(self.x), n_problems * M, K)   # per-token: row = token
        pitch = ctx.act_pitch(K)
        self.d_out = ctx.alloc(4 * n_problems * M * N)
        self.d_acc = ctx.alloc(4 * n_problems * M * N)
        self.with_acc = (_lib.GemvProblem * n_problems)()
        self.plain = (_lib.GemvProblem * n_problems)()
        for j in range(n_problems):
            mat = self.mats[j % distinct]
            for arr, acc in ((self.with_acc, True), (self.plain, False)):
                p = arr[j]
                p.d_q = self.acts[0].ptr + j * M * pitch
                p.d_act_scale = self.acts[1].ptr + 4 * j * M
                p.d_rowsum = self.acts[2].ptr + 4 * j * M
                p.d_tiled = mat.tiled[j // distinct].ptr
                p.d_out = self.d_out.ptr + 4 * j * M * N
                p.d_acc = self.d_acc.ptr + 4 * j * M * N if acc else None
                p.w_scale, p.reserved = float(mat.w_scale), 0
        ctx.sync()

    def launch(self, first, count, with_acc=False):
        arr = self.with_acc if with_acc else self.plain
        self.ctx.gemv_grouped(arr, self.M, self.K, self.N, first, count)

    def launch_single(self, j):
        """Problem j as a launch of its own (rbn_gemv_t2_i8)."""
        from ronn_amd import _lib
        p = self.plain[j]
        _lib.check(self.ctx.lib.rbn_gemv_t2_i8(self.ctx.handle, p.d_q, p.d_act_scale, p.d_rowsum, p.d_tiled,
                                               p.w_scale, self.M, self.K, self.N, None, p.d_out))

    def parity(self, group):
        """Every problem of a grouped run against the oracle; returns (flags, oracle tensors)."""
        from oracle import oracle as O
        ctx, M, N, n = self.ctx, self.M, self.N, self.n
        ctx.lib.rbn_fill_u8(ctx.handle, self.d_out.ptr, 0xFF, 4 * n * M * N)
        ctx.lib.rbn_fill_u8(ctx.handle, self.d_acc.ptr, 0xFF, 4 * n * M * N)
        for first in range(0, n, group):
            self.launch(first, min(group, n - first), with_acc=True)
        ctx.sync()
        out = self.d_out.download(np.float32, n * M * N).reshape(n, M, N)
        acc = self.d_acc.download(np.int32, n * M * N).reshape(n, M, N)
        q, s, _ = O.act_quant_i8(self.x)
        oracles = [m.oracle() for m in self.mats]
        flags = {"w_scale_bits_equal": True, "acc_equal": True, "out_bits_equal": True, "problems_checked": n}
        for d, (t, vals_f) in enumerate(oracles):
            flags["w_scale_bits_equal"] &= bool(np.float32(self.mats[d].w_scale).view(np.uint32)
                                                == np.float32(t.scale).view(np.uint32))
            rows = [j for j in range(n) if j % len(self.mats) == d]
            idx = np.concatenate([np.arange(j * M, (j + 1) * M) for j in rows])
            want_acc = exact_int_matmul(q[idx], vals_f).reshape(len(rows), M, N)
            want_out = epilogue(want_acc.reshape(-1, N), s[idx], t.scale).reshape(len(rows), M, N)
            flags["acc_equal"] &= bool((acc[rows] == want_acc).all())
            flags["out_bits_equal"] &= bool((out[rows].view(np.uint32) == want_out.view(np.uint32)).all())
        return flags, oracles, (q, s), (out, acc)


def replay(ctx, record, units, steps, warmup, max_units_per_graph=256):
    """Times exactly `steps` units of work after `warmup` untimed ones.  record(first_unit, n)
    issues n consecutive units starting at unit index first_unit (inside a graph capture);
    `units` is the granularity record() works best at.  Returns (event ms, wall ms) per unit."""
    def graph_of(n):
        ctx.graph_begin()
        done = 0
        while done < n:
            c = min(units, n - done)
            record(done, c)
            done += c
        return ctx.graph_end()

    per = min(steps, max(units, (max_units_per_graph // units) * units))
    main, reps, rem = graph_of(per), steps // per, steps % per
    tail = graph_of(rem) if rem else None
    for _ in range(warmup // per):
        ctx.graph_launch(main)
    if warmup % per:
        wg = graph_of(warmup % per)
        ctx.graph_launch(wg)
        ctx.sync()
        ctx.graph_destroy(wg)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(reps):
        ctx.graph_launch(main)
    if tail is not None:
        ctx.graph_launch(tail)
    ev_ms = ctx.timer_stop()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ctx.graph_destroy(main)
    if tail is not None:
        ctx.graph_destroy(tail)
    return ev_ms / steps, wall_ms / steps


def time_graph(ctx, wl, fn, steps, warmup):
    """Average milliseconds per launch of fn on a Workload, weight buffers rotating."""
    nbuf = len(wl.tiled)
    ev, wall = replay(ctx, lambda first, n: [wl.launch(fn, first + i) for i in range(n)], nbuf, steps, warmup,
                      max_units_per_graph=max(nbuf, 64))
    return ev, wall, steps


def time_plain(ctx, fn_call, reps):
    fn_call()
    ctx.sync()
    ctx.timer_start()
    for _ in range(reps):
        fn_call()
    ms = ctx.timer_stop()
    return ms / reps


def upload_synth(ctx, seed, sigma, K, N, keep=False):
    """A K x N f32 matrix generated and uploaded in slices (bounds host memory unless kept)."""
    from ronn_amd import _lib
    from ronn_amd.device import synth_normal
    d_w = ctx.alloc(4 * K * N)
    rows, host = 512, []
    for r0 in range(0, K, rows):
        part = synth_normal(seed, sigma, (min(rows, K - r0) * N,), first=r0 * N)
        _lib.check(ctx.lib.rbn_h2d(ctx.handle, d_w.ptr + 4 * r0 * N, part.ctypes.data, part.nbytes))
        if keep:
            host.append(part)
    return d_w, (np.concatenate(host).reshape(K, N) if keep else None)


def time_ternarize(ctx, d_w, w_host, K, N):
    """Absmean ternarisation + 2-bit packing of a K x N f32 matrix resident in HBM.

    strict: the reference's sequential f32 sums reproduced exactly (bit-exact threshold and
    scale; gated here against the oracle's packed bytes); tree: pairwise sums (not reference-exact).
    Algorithmic bytes: 2 x 4 n + n / 4 (two reads are inherent: the threshold depends on
    the global mean; the survivor sum can ride on the packing pass).
    """
    from oracle import oracle as O
    from ronn_amd import _lib
    n = K * N
    d_p = ctx.alloc(ctx.lib.rbn_packed_capacity(n))
    out = {"K": K, "N": N, "weights": n}
    for name, mode in (("strict", _lib.SUM_STRICT_SEQ), ("tree", _lib.SUM_TREE)):
        _, scale, thr, _ = ctx.quantize_ternary(d_w, n, mode, d_p)
        ctx.sync()
        if name == "strict":
            t0 = time.perf_counter()
            t = O.quantize_ternary(w_host)
            out["cpu_oracle_ms"] = (time.perf_counter() - t0) * 1e3
            same = (np.float32(scale).view(np.uint32) == np.float32(t.scale).view(np.uint32)
                    and np.float32(thr).view(np.uint32) == np.float32(t.threshold).view(np.uint32)
                    and bool((d_p.download(np.uint8, n // 4) == t.packed_data).all()))
            if not same:
                print("bench.py: PARITY FAILURE: packed weights of the %d x %d ternarize differ" % (K, N), file=sys.stderr)
                sys.exit(1)
            out["packed_bytes_equal_oracle"] = True
            oracle_t = t
        ctx.quantize_ternary(d_w, n, mode, d_p)   # untimed: the GPU has idled through the oracle's pass above
        ctx.sync()
        t0 = time.perf_counter()
        reps = 3
        for _ in range(reps):
            ctx.quantize_ternary(d_w, n, mode, d_p)
        ctx.sync()
        ms = (time.perf_counter() - t0) * 1e3 / reps
        b = 2 * 4 * n + n // 4
        out[name] = {"ms": ms, "Gweights_per_s": n / ms / 1e6, "GBps": b / ms / 1e6,
                     "frac_hbm_peak": b / ms / 1e6 / HBM_PEAK_GBS}
    d_p.free()
    return out, oracle_t


def time_act_quant(ctx):
    """Per-token absmax int8 quantisation (5 M K + 8 M algorithmic bytes), graph replay."""
    from ronn_amd.device import synth_normal
    rows = []
    for M, K in ((1, 4096), (16, 4096), (2048, 4096), (2048, 11008)):
        x = synth_normal(0x5EED0009, 1.0, (M, K))
        n_in = max(1, -(-(MALL_BYTES + (64 << 20)) // x.nbytes)) if M >= 2048 else 8
        ins = [ctx.to_device(x) for _ in range(min(n_in, 24))]
        bufs = ctx.alloc_acts(M, K)
        ev, _ = replay(ctx, lambda first, n: [ctx.act_quant_i8(ins[(first + i) % len(ins)], M, K, bufs) for i in range(n)],
                       len(ins), 20 * len(ins), 2 * len(ins), max_units_per_graph=len(ins))
        b = 5 * M * K + 8 * M
        rows.append({"M": M, "K": K, "us": ev * 1e3, "GBps": b / (ev * 1e-3) / 1e9,
                     "frac_hbm_peak": b / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS, "input_buffers": len(ins)})
        del ins
    return rows


def time_stream_floor(ctx):
    """What launches that compute nothing cost on this machine: an empty kernel, and kernels
    that only read (the GEMV's access pattern) 4, 11, 22, 59, 181 and 362 MB from rotating addresses
    (the last two are what 16 and 32 grouped GEMVs of the headline shape read in one launch)."""
    from ronn_amd import _lib
    lib, h = ctx.lib, ctx.handle
    ev, _ = replay(ctx, lambda first, n: [_lib.check(lib.rbn_probe_empty_launch(h)) for _ in range(n)], 64, 640, 64,
                   max_units_per_graph=64)
    out = {"empty_launch_us": ev * 1e3, "reads": []}
    pool_bytes = 768 << 20
    pool = ctx.alloc(pool_bytes)
    _lib.check(lib.rbn_fill_u8(h, pool.ptr, 0x55, pool_bytes))
    for size in (4194304, 11272192, 22544384, 58720256, 16 * 11320324 // 16 * 16, 32 * 11320324 // 16 * 16):
        slots = pool_bytes // size
        row = {"bytes": size}
        for nt in (0, 1):
            ev, _ = replay(ctx, lambda first, n: [_lib.check(lib.rbn_probe_stream_read(
                h, pool.ptr + ((first + i) % slots) * size, size, nt)) for i in range(n)], slots, 10 * slots, slots,
                max_units_per_graph=slots)
            row["nontemporal_us" if nt else "plain_us"] = ev * 1e3
            row["nontemporal_GBps" if nt else "plain_GBps"] = size / (ev * 1e-3) / 1e9
        out["reads"].append(row)
    pool.free()
    return out


def time_decoder(ctx, prompt_len=512, new_tokens=128, use_graph=True):
    """BitNet-b1.58 2B-class decoder, random-initialised on the device: 24 layers, hidden
    2560, 20 heads of 128, SwiGLU FFN 6912, vocabulary 32000, f16 K/V.  Batch 1: a prompt of
    prompt_len tokens, then new_tokens greedy tokens replayed from one captured HIP graph."""
    from ronn_amd.decoder import BitNetDecoder, DecoderConfig
    cfg = DecoderConfig(max_seq=prompt_len + new_tokens + 8)
    dec = BitNetDecoder(ctx, cfg, max_batch_tokens=prompt_len)
    t0 = time.perf_counter()
    dec.init_random(seed=4)
    t_init = time.perf_counter() - t0
    prompt = (np.arange(prompt_len, dtype=np.int64) * 7919 % cfg.vocab).astype(np.int32)
    dec.prefill(prompt)       # warm-up (also sizes every workspace before the capture)
    ctx.sync()
    t0 = time.perf_counter()
    dec.prefill(prompt)
    ctx.sync()
    t_prefill = time.perf_counter() - t0
    dec.decode(4, use_graph)  # captures the graph, warms it up
    dec.prefill(prompt)
    tokens, dt = dec.decode(new_tokens, use_graph)
    w_bytes = cfg.packed_weight_bytes_per_token()
    kv_bytes = 2 * 2 * cfg.layers * cfg.attn_dim * (prompt_len + new_tokens / 2.0)   # average over the run
    per_tok = dt / new_tokens
    return {"config": dataclass_dict(cfg), "prompt_tokens": prompt_len, "new_tokens": new_tokens,
            "decode_tok_per_s": new_tokens / dt, "ms_per_token": per_tok * 1e3,
            "prefill_ms": t_prefill * 1e3, "prefill_tok_per_s": prompt_len / t_prefill,
            "weight_init_s": t_init, "launches_per_token": dec.launches_per_token(),
            "bytes_per_token": {"packed_weights": w_bytes, "kv_cache_f16_avg": kv_bytes},
            "GBps": (w_bytes + kv_bytes) / per_tok / 1e9,
            "frac_hbm_peak": (w_bytes + kv_bytes) / per_tok / 1e9 / HBM_PEAK_GBS,
            "first_tokens": [int(t) for t in tokens[:8]]}


def dataclass_dict(obj):
    import dataclasses
    return dataclasses.asdict(obj)


def cpu_headline(gw, oracles, qs, outs, budget_s=8.0):
    """Times the oracle's matmul (the reference's get_value inner loop) on problem 0 of the
    headline workload, one core; its integers also gate problem 0 literally."""
    from oracle import oracle as O
    q, s = qs
    out, acc = outs
    tw = oracles[0][0]
    M = gw.M
    reps, t_mm = 0, 0.0
    want_out = want_acc = None
    while reps < 2 or (t_mm < budget_s and reps < 40):
        t0 = time.perf_counter()
        want_out, want_acc = O.matmul_i8_ternary(q[:M], s[:M], tw)
        t_mm += time.perf_counter() - t0
        reps += 1
    t_mm /= reps
    literal_ok = bool((acc[0] == want_acc).all()) and bool((out[0].view(np.uint32) == want_out.view(np.uint32)).all())
    gb = gemv_bytes(gw.M, gw.K, gw.N) / 1e9
    base = {
        "value": gb / t_mm, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": ("oracle matmul (reference's get_value inner loop, kernels.rs:159-165) on problem 0 of the "
                   "headline workload, M=%d K=%d N=%d, %d repetitions, %.3f s each; `variants` holds the "
                   "reference's own two-operand ternary path per configuration" % (gw.M, gw.K, gw.N, reps, t_mm)),
        "ms_per_gemv": t_mm * 1e3,
        "host_cpus": os.cpu_count(),
    }
    return base, literal_ok


def cpu_variants(large=None):
    """The reference's CPU path per configuration, one core: `matmul_only` =
    execute_ternary_matmul on operands ternarised beforehand (kernels.rs:134-178), `full_execute`
    = CompiledKernel::execute, which ternarises BOTH operands on every call and then multiplies
    (kernels.rs:271-283).  Small cases are timed directly; the prefill shape and the large layer
    at M=64 are timed at M=4 and scaled linearly in M (labelled)."""
    from oracle import oracle as O
    from ronn_amd.device import synth_normal
    rows = []

    def case(name, M, K, N, sigma, w=None, measure_m=None, seed=0):
        mm = measure_m or M
        x = synth_normal(0x5EED0001 + seed, 1.0, (mm, K))
        if w is None:
            w = synth_normal(0x5EED1001 + seed, sigma, (K, N))
        t0 = time.perf_counter()
        ta = O.quantize_ternary(x)
        t_qa = time.perf_counter() - t0
        t0 = time.perf_counter()
        tb = O.quantize_ternary(w)
        t_qb = time.perf_counter() - t0
        t0 = time.perf_counter()
        O.ternary_matmul(ta, tb, mm, N, K)
        t_mm = time.perf_counter() - t0
        scale = M / mm
        row = {"config": name, "M": M, "K": K, "N": N,
               "matmul_only_ms": t_mm * scale * 1e3, "full_execute_ms": (t_qa * scale + t_qb + t_mm * scale) * 1e3,
               "quantize_weights_ms": t_qb * 1e3}
        if measure_m:
            row["extrapolated_from_M"] = mm
        rows.append(row)
        return w

    case("C1 single BitLinear", 1, 2048, 2048, 0.02, seed=1)
    for i, (K, N) in enumerate(((4096, 4096), (4096, 11008), (11008, 4096))):
        w = None
        for M in (1, 4, 16):
            w = case("C2 decode sweep", M, K, N, 0.02, w=w, seed=2 + i)
        if (K, N) == (4096, 11008):
            case("C3 prefill", 2048, K, N, 0.02, w=w, measure_m=4, seed=5)
    if large is not None:
        case("C5 large layer", 1, 8192, 28672, 0.015, w=large, seed=6)
        case("C5 large layer", 64, 8192, 28672, 0.015, w=large, measure_m=4, seed=6)
    return rows


def profile_kernel(ctx, which, launches):
    """Launches one kernel `launches` times on its real shape, for rocprofv3 runs.

    gemv_grouped: 32 GEMVs of M=1 K=4096 N=11008 per launch, rotating over 64 weight buffers.
    gemv: the same GEMVs one per launch.  skinny: M=16, same matrix.  gemm: M=2048 K=4096
    N=11008.  pack / quantize: the 8192 x 28672 weight matrix of the large-layer config.
    act_quant: 2048 x 4096 f32 rows.  stream: the read-only floor kernels (prints their
    timings).  copy: a device-to-device copy of 256 MiB, whose known traffic calibrates the
    FETCH_SIZE / WRITE_SIZE counters.
    """
    from ronn_amd import _lib
    from ronn_amd.device import synth_normal
    if which in ("gemv_grouped", "gemv"):
        gw = GroupedWorkload(ctx, 1, 4096, 11008, 0.02, 2 * GROUP, keep_host=False)
        for i in range(launches):
            if which == "gemv":
                gw.launch_single(i % gw.n)
            else:
                gw.launch((i * GROUP) % gw.n, GROUP)
    elif which == "skinny":
        wl = Workload(ctx, 16, 4096, 11008, 0.02, seed=3, mode=1)
        for i in range(launches):
            wl.launch(ctx.skinny, i)
    elif which == "gemm":
        wl = Workload(ctx, 2048, 4096, 11008, 0.02, seed=4, rotate_bytes=1, mode=1)
        for i in range(launches):
            wl.launch(ctx.gemm, 0)
    elif which in ("pack", "quantize"):
        K, N = 8192, 28672
        d_w, _ = upload_synth(ctx, 0x5EED1005, 0.015, K, N)
        d_p = ctx.alloc(ctx.lib.rbn_packed_capacity(K * N))
        for i in range(min(launches, 4)):
            if which == "pack":
                ctx.pack_ternary(d_w, K * N, 0.0028, d_p)
            else:
                ctx.quantize_ternary(d_w, K * N, _lib.SUM_STRICT_SEQ, d_p)
    elif which == "act_quant":
        M, K = 2048, 4096
        ins = [ctx.to_device(synth_normal(0x5EED0009, 1.0, (M, K))) for _ in range(12)]
        bufs = ctx.alloc_acts(M, K)
        for i in range(launches):
            ctx.act_quant_i8(ins[i % len(ins)], M, K, bufs)
    elif which == "stream":
        print(json.dumps(time_stream_floor(ctx)))
        return
    elif which == "skinny_trace":
        # needs a library built with the cycle stamps: make -B -C ronn_amd/csrc EXTRA=-DRBN_SK_TRACE
        fn = getattr(ctx.lib, "rbn_debug_sk_trace", None)
        if fn is None:
            print("bench.py: this library has no cycle stamps; rebuild with "
                  "`make -B -C ronn_amd/csrc EXTRA=-DRBN_SK_TRACE`", file=sys.stderr)
            sys.exit(2)
        fn.argtypes, fn.restype = [C.c_void_p, C.c_int], C.c_int
        wl = Workload(ctx, 16, 4096, 11008, 0.02, seed=3, mode=1)
        for i in range(40):
            wl.launch(ctx.skinny, i)
        ctx.sync()
        wl.launch(ctx.skinny, 17)
        ctx.sync()
        buf = np.zeros(64 * 16 * 8, dtype=np.int64)
        _lib.check(fn(buf.ctypes.data, buf.size))
        t = buf.reshape(64, 16, 8)[:, :, :5]
        t = t - t[:, :, 0:1].min(axis=1, keepdims=True)      # cycles since the workgroup's first wave started
        names = ["start", "transfers_issued", "last_mfma_done", "past_join_barrier", "stores_acknowledged"]
        print(json.dumps({"kernel": "skinny_dma_kernel", "M": 16, "K": 4096, "N": 11008, "unit": "shader clock cycles",
                          "workgroup_0": {n: [int(v) for v in t[0, :, i]] for i, n in enumerate(names)},
                          "median_over_64_workgroups_of_the_slowest_wave": {
                              n: float(np.median(t[:, :, i].max(axis=1))) for i, n in enumerate(names)}}))
        return
    elif which in ("decoder", "decoder_eager"):
        # decoder_eager launches kernel by kernel instead of replaying the captured graph
        # (for per-kernel traces)
        print(json.dumps(time_decoder(ctx, new_tokens=min(launches, 32), use_graph=which == "decoder")))
        return
    elif which == "copy":
        n = 256 << 20
        a, b = ctx.alloc(n), ctx.alloc(n)
        _lib.check(ctx.lib.rbn_fill_u8(ctx.handle, a.ptr, 1, n))
        for i in range(launches):
            _lib.check(ctx.lib.rbn_d2d(ctx.handle, b.ptr, a.ptr, n))
    ctx.sync()
    print(json.dumps({"profiled_kernel": which, "launches": launches}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256, help="timed steps; a step is one launch of 32 independent GEMVs")
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-extra", action="store_true", help="headline only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline timings (parity is still gated)")
    ap.add_argument("--kernel", choices=["gemv_grouped", "gemv", "skinny", "gemm", "pack", "quantize", "copy",
                                         "act_quant", "stream", "skinny_trace", "decoder", "decoder_eager"],
                    help="profiling aid: launch only this kernel a few times (for rocprofv3) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if args.steps < 1 or args.warmup < 0:
        print("bench.py: --steps must be positive and --warmup non-negative", file=sys.stderr)
        sys.exit(2)

    from ronn_amd.device import Context
    ctx = Context(0)
    info = ctx.device_info()
    if args.kernel:
        profile_kernel(ctx, args.kernel, max(1, min(args.steps, 64)))
        return

    M, K, N = 1, 4096, 11008
    gw = GroupedWorkload(ctx, M, K, N, 0.02, 2 * GROUP)
    parity, oracles, qs, outs = gw.parity(GROUP)
    # set-up, not steps: a quarter of a second of the same launches, so that the warm-up and the
    # timed steps run at the clocks of a busy GPU whatever --steps and --warmup are
    t_heat = time.perf_counter()
    while time.perf_counter() - t_heat < 0.25:
        for first in range(0, gw.n, GROUP):
            gw.launch(first, GROUP)
        ctx.sync()
    batches = gw.n // GROUP
    ev_ms, wall_ms = replay(ctx, lambda first, n: [gw.launch(((first + i) % batches) * GROUP, GROUP) for i in range(n)],
                            batches, args.steps, args.warmup)
    bytes_per_gemv = gemv_bytes(M, K, N)
    bytes_per_step = bytes_per_gemv * GROUP
    achieved = bytes_per_step / (ev_ms * 1e-3) / 1e9
    facts = profile_facts(HEADLINE_PROFILE)

    result = {
        "metric": "ternary GEMV HBM GB/s (% of peak) + prefill int8 TOPS; BitNet decode tok/s",
        "value": bytes_per_step / (wall_ms * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x 2-bit ternary -> int32",
        "data": "synthetic (seeded N(0,1) activations, N(0,0.02) weights, absmean-ternarised on device)",
        "config": {"workload": "decode ternary GEMV, M=1 K=4096 N=11008 (FFN up/gate); one step = one batch of %d "
                               "complete independent GEMVs (each its own activations, weight buffer and output) in "
                               "one launch (rbn_gemv_t2_i8_grouped); steps alternate over %d weight buffers (%.0f MiB) "
                               "so every GEMV streams from HBM; HIP-graph replay; the one-GEMV-per-launch figure is "
                               "extra.gemv_one_per_launch" % (GROUP, gw.n, gw.n * gw.tiled_bytes / 2**20),
                   "M": M, "K": K, "N": N, "gemvs_per_launch": GROUP, "weight_buffers": gw.n,
                   "realistic_groups": "extra.gemv_realistic_groups: fraction of HBM peak at 1, 2, 3, 8 and 32 GEMVs "
                                       "per launch, with the caller that reaches each",
                   "gemvs_timed": args.steps * GROUP,
                   "preheat": "0.25 s of the same launches during set-up, before the warm-up steps (clock ramp)",
                   "device": info["name"] or info["arch"], "arch": info["arch"],
                   "compute_units": info["compute_units"], "clock_mhz": info["clock_khz"] / 1000.0},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": facts.get("traffic_bytes_per_launch"),
                     "traffic_source": ("profiles/%s (rocprofv3 FETCH_SIZE and WRITE_SIZE, scaled by a 256 MiB copy)"
                                        % HEADLINE_PROFILE) if facts.get("traffic_bytes_per_launch") else None,
                     "kernel": facts.get("kernel", "gemv_t2_i8_grouped_kernel"),
                     "bytes_per_launch": bytes_per_step, "gemvs_per_launch": GROUP,
                     "us_per_launch": ev_ms * 1e3, "us_per_gemv": ev_ms * 1e3 / GROUP,
                     "profile_avg_us_per_launch": facts.get("avg_us_per_launch")},
        "parity": parity,
    }
    if not all(parity.values()):
        print(json.dumps(result))
        print("bench.py: PARITY FAILURE against the CPU oracle: %s" % parity, file=sys.stderr)
        sys.exit(1)

    if not args.no_cpu:
        base, literal_ok = cpu_headline(gw, oracles, qs, outs)
        result["cpu_baseline"] = base
        result["parity"]["problem0_equals_literal_loop"] = literal_ok
        if not literal_ok:
            print(json.dumps(result))
            print("bench.py: PARITY FAILURE against the oracle's literal loop", file=sys.stderr)
            sys.exit(1)

    if not args.no_extra:
        extra = {}
        # the same GEMVs one to a launch (what a caller with a single matrix gets)
        ev1, _ = replay(ctx, lambda first, n: [gw.launch_single((first + i) % gw.n) for i in range(n)], gw.n,
                        32 * gw.n, 4 * gw.n, max_units_per_graph=gw.n)
        extra["gemv_one_per_launch"] = {"M": M, "K": K, "N": N, "us": ev1 * 1e3,
                                        "GBps": bytes_per_gemv / (ev1 * 1e-3) / 1e9,
                                        "frac_hbm_peak": bytes_per_gemv / (ev1 * 1e-3) / 1e9 / HBM_PEAK_GBS}
        rows = []
        for g in (2, 3, 4, 8, 16, 32):
            evg, _ = replay(ctx, lambda first, n: gw.launch(first % gw.n, n), g, 16 * gw.n, 2 * gw.n,
                            max_units_per_graph=gw.n)
            rows.append({"gemvs_per_launch": g, "us_per_gemv": evg * 1e3,
                         "frac_hbm_peak": bytes_per_gemv / (evg * 1e-3) / 1e9 / HBM_PEAK_GBS})
        extra["gemv_group_size_sweep"] = rows
        # which callers reach which group size: one MatMul node per execute() is 1; the same-input
        # projections of one token that BitNetKernel::execute_group / rbp_kernel_execute_group run as one
        # launch are 2 (gate, up) and 3 (q, k, v); 8 and more need several sequences or experts per call
        by_g = {r["gemvs_per_launch"]: r for r in rows}
        extra["gemv_realistic_groups"] = {
            "1 (CompiledKernel::execute, one MatMul node)": extra["gemv_one_per_launch"]["frac_hbm_peak"],
            "2 (gate/up through execute_group)": by_g[2]["frac_hbm_peak"],
            "3 (q/k/v through execute_group)": by_g[3]["frac_hbm_peak"],
            "8 (eight sequences or experts through execute_group)": by_g[8]["frac_hbm_peak"],
            "32 (the headline step)": by_g[32]["frac_hbm_peak"]}
        # warm variant: one buffer, lives in L2 / Infinity Cache
        evw, _ = replay(ctx, lambda first, n: [gw.launch_single(0) for _ in range(n)], 32, 2048, 256,
                        max_units_per_graph=64)
        extra["gemv_warm_cache"] = {"M": M, "K": K, "N": N, "us": evw * 1e3,
                                    "GBps": bytes_per_gemv / (evw * 1e-3) / 1e9,
                                    "note": "single 11 MiB weight buffer re-read from cache, not HBM"}
        # One launch at a time on an idle stream, timed by the dispatch's own begin and end
        # timestamps: what a profiler's kernel trace reports.
        iso_us = []
        for i in range(130):
            p = gw.plain[i % gw.n]
            us = C.c_float()
            from ronn_amd import _lib
            _lib.check(ctx.lib.rbn_gemv_t2_i8_kernel_time(ctx.handle, p.d_q, p.d_act_scale, p.d_rowsum, p.d_tiled,
                                                          p.w_scale, M, K, N, None, p.d_out, C.byref(us)))
            iso_us.append(us.value)
        iso_us = sorted(iso_us[30:])
        extra["gemv_isolated_dispatch"] = {"us_mean": sum(iso_us) / len(iso_us), "us_median": iso_us[len(iso_us) // 2],
                                           "us_min": iso_us[0],
                                           "note": "begin-to-end timestamps of single dispatches on an idle stream "
                                                   "(rbn_gemv_t2_i8_kernel_time)"}
        extra["stream_floor"] = time_stream_floor(ctx)
        del gw, outs, qs, oracles

        def kernel_for(m, k, n):
            return ("gemv", "skinny_mfma", "gemm_mfma")[ctx.lib.rbn_matmul_kernel_choice(m, k, n)]

        def sweep_over(shapes, ms, sigma, seed, weights=None, oracle_pair=None):
            rows = []
            for (k, n) in shapes:
                wts = weights or Weights(ctx, k, n, sigma, 0x5EED1001 + seed, MALL_BYTES + (64 << 20), keep_host=True)
                pair = oracle_pair or wts.oracle()
                wts.w = None
                for m in ms:
                    w2 = Workload(ctx, m, k, n, sigma, seed=seed + m, weights=wts)
                    w2.gate(ctx.matmul, pair, "the sweep at M=%d K=%d N=%d" % (m, k, n))
                    ev, _, _ = time_graph(ctx, w2, ctx.matmul, 1500, 150)
                    b = gemv_bytes(m, k, n)
                    rows.append({"M": m, "K": k, "N": n, "kernel": kernel_for(m, k, n), "us": ev * 1e3,
                                 "GBps": b / (ev * 1e-3) / 1e9,
                                 "frac_hbm_peak": b / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS, "parity_gated": True})
                    del w2
                del wts, pair
            return rows

        # rbn_matmul_t2_i8 picks the kernel by M; weights rotate through > 256 MiB of buffers
        extra["decode_sweep"] = sweep_over(((4096, 4096), (4096, 11008), (11008, 4096)), (1, 4, 16), 0.02, seed=3)
        # large layer: the f32 matrix stays on the device for the ternarize timing, the host copy
        # feeds the oracle (packed bytes, BLAS integers) and the CPU baseline
        LK, LN = 8192, 28672
        d_w, w_large = upload_synth(ctx, 0x5EED1005, 0.015, LK, LN, keep=True)
        extra["large_layer_ternarize"], t_large = time_ternarize(ctx, d_w, w_large, LK, LN)
        vals_large = t_large.values().reshape(LK, LN).astype(np.float32)
        lw = Weights(ctx, LK, LN, 0.015, 0, MALL_BYTES + (64 << 20), d_w=d_w)
        d_w.free()
        extra["large_layer"] = sweep_over(((LK, LN),), (1, 8, 64), 0.015, seed=7, weights=lw,
                                          oracle_pair=(t_large, vals_large))
        del lw, vals_large
        # prefill GEMM, int8 MFMA
        pm, pk, pn = 2048, 4096, 11008
        pwt = Weights(ctx, pk, pn, 0.02, 0x5EED1004, 1, keep_host=True)
        pw = Workload(ctx, pm, pk, pn, 0.02, seed=4, weights=pwt)
        pw.gate(ctx.gemm, pwt.oracle(), "the prefill GEMM at M=2048 K=4096 N=11008")
        pwt.w = None
        # one burst of 20 back-to-back launches after a warm-up launch, as in the rocprofv3 profile
        # (longer bursts run into the power cap: the second and third burst of 20 take 15-20 % longer)
        ms = time_plain(ctx, lambda: pw.launch(ctx.gemm, 0), 20)
        ops = 2.0 * pm * pk * pn
        gfacts = profile_facts("gemm_m2048_k4096_n11008.md")
        extra["prefill_gemm"] = {"M": pm, "K": pk, "N": pn, "ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
                                 "frac_int8_peak": ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, "parity_gated": True,
                                 "roofline": {"bound": "mfma", "achieved": ops / (ms * 1e-3) / 1e12,
                                              "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                              "frac": ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS,
                                              "traffic": gfacts.get("traffic_bytes_per_launch"),
                                              "kernel": gfacts.get("kernel", "gemm_t2_i8_mfma_kernel")}}
        del pw, pwt
        extra["act_quant_i8"] = time_act_quant(ctx)
        # what a loop of nothing but int8 MFMA sustains on this box, by operand values
        extra["mfma_i8_probe_TOPS"] = {"constant_operands": ctx.probe_mfma_i8(0),
                                       "int8_x_ternary_codes": ctx.probe_mfma_i8(1),
                                       "int8_x_int8": ctx.probe_mfma_i8(2)}
        extra["decoder"] = time_decoder(ctx)
        result["extra"] = extra
        if not args.no_cpu:
            result["cpu_baseline"]["variants"] = cpu_variants(w_large)
            result["cpu_baseline"]["variants_note"] = (
                "oracle (C restatement of the reference, one core): matmul_only = execute_ternary_matmul on "
                "pre-ternarised operands; full_execute = execute(), which ternarises both operands on every call; "
                "rows with extrapolated_from_M were timed at that M and scaled linearly")

    print(json.dumps(result))


if __name__ == "__main__":
    main()

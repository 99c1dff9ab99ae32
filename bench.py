#!/usr/bin/env python3
"""Benchmark of the BitNet ternary hot path on one MI355X.

Headline (the JSON line's `value`): decode-regime ternary GEMV at K=4096, N=11008,
M=1 (the FFN up/gate shape of the decode sweep), int8 activations and
tiled 2-bit weights already resident in HBM.  One step = one GEMV launch.  The steps
rotate over enough distinct weight buffers (> 256 MiB in total) that every launch
streams its weights from HBM rather than from the Infinity Cache; launches are
replayed from a captured HIP graph so that host launch cost does not throttle a
kernel of a few microseconds.  `roofline` prices the GEMV kernel's algorithmic bytes
(K*N/4 + M*K + 4*M + 4*M*N per launch) against the 8 TB/s HBM peak using HIP events
recorded on the library's own stream.  `extra` carries the rest of the sweep, the
prefill int8-MFMA GEMM and the ternarize+pack kernel.  `cpu_baseline` times the CPU
oracle (a C restatement of the reference's scalar loop; the Rust original cannot be
built here) on one host core on the same inputs, and doubles as the parity gate.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0     # MI355X published dense int8 MFMA rate (5.0 POP/s)
MALL_BYTES = 256 << 20
# HBM bytes per launch of the headline GEMV, from rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a
# 256 MiB copy (profiles/gemv_m1_k4096_n11008.md)
GEMV_HEADLINE_TRAFFIC_BYTES = 11415105


def gemv_bytes(M, K, N):
    return K * N // 4 + M * K + 4 * M + 4 * M * N


class Workload:
    """Quantised operands of one (M, K, N) problem, resident on the device."""

    def __init__(self, ctx, M, K, N, sigma_w, seed, rotate_bytes=MALL_BYTES + (64 << 20),
                 mode=None, want_host=False):
        from ronn_amd import _lib
        from ronn_amd.device import synth_normal
        self.ctx, self.M, self.K, self.N = ctx, M, K, N
        self.x = synth_normal(0x5EED0001 + seed, 1.0, (M, K))
        self.w = synth_normal(0x5EED1001 + seed, sigma_w, (K, N))
        d_w = ctx.to_device(self.w)
        mode = _lib.SUM_STRICT_SEQ if mode is None else mode
        d_p, self.w_scale, self.w_thr, _ = ctx.quantize_ternary(d_w, K * N, mode)
        self.d_packed = d_p
        self.tiled_bytes = ctx.lib.rbn_tiled_bytes(K, N)
        first = ctx.tile_weights(d_p, K, N)
        nbuf = max(1, -(-rotate_bytes // self.tiled_bytes))
        self.tiled = [first]
        for _ in range(nbuf - 1):
            b = ctx.alloc(self.tiled_bytes)
            _lib.check(ctx.lib.rbn_d2d(ctx.handle, b.ptr, first.ptr, self.tiled_bytes))
            self.tiled.append(b)
        d_w.free()
        self.acts = ctx.act_quant_i8(ctx.to_device(self.x), M, K)
        self.d_out = ctx.alloc(4 * M * N)
        self.d_acc = ctx.alloc(4 * M * N)
        ctx.sync()
        if not want_host:
            self.w = None

    def launch(self, fn, i, with_acc=False):
        fn(self.acts, self.tiled[i % len(self.tiled)], self.w_scale, self.M, self.K, self.N,
           d_out=self.d_out, d_acc=self.d_acc if with_acc else None, want_acc=False)

    def results(self, fn):
        self.launch(fn, 0, with_acc=True)
        self.ctx.sync()
        n = self.M * self.N
        return (self.d_out.download(np.float32, n).reshape(self.M, self.N),
                self.d_acc.download(np.int32, n).reshape(self.M, self.N))


def time_graph(ctx, wl, fn, steps, warmup):
    """Average milliseconds per launch over `steps` launches replayed from a HIP graph."""
    # at least 32 launches per graph replay, so that the cost of launching the graph itself
    # (several microseconds) does not hide the kernel; a whole number of buffer rotations
    nbuf = len(wl.tiled)
    per_graph = nbuf * max(1, -(-32 // nbuf))
    ctx.graph_begin()
    for i in range(per_graph):
        wl.launch(fn, i)
    g = ctx.graph_end()
    reps_w = max(1, -(-warmup // per_graph))
    reps = max(1, -(-steps // per_graph))
    for _ in range(reps_w):
        ctx.graph_launch(g)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(reps):
        ctx.graph_launch(g)
    ev_ms = ctx.timer_stop()
    ctx.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ctx.graph_destroy(g)
    n = reps * per_graph
    return ev_ms / n, wall_ms / n, n


def time_plain(ctx, fn_call, reps):
    fn_call()
    ctx.sync()
    ctx.timer_start()
    for _ in range(reps):
        fn_call()
    ms = ctx.timer_stop()
    return ms / reps


def time_ternarize(ctx, K, N, sigma):
    """Absmean ternarisation + 2-bit packing of a K x N f32 matrix resident in HBM.

    strict: the reference's sequential f32 sums reproduced exactly (bit-exact threshold and
    scale); tree: pairwise sums (same packed bytes unless the threshold's last bit differs).
    Algorithmic bytes: 2 x 4 n + n / 4 (two reads are inherent: the threshold depends on
    the global mean; the survivor sum can ride on the packing pass).
    """
    from ronn_amd import _lib
    from ronn_amd.device import synth_normal
    n = K * N
    d_w = ctx.alloc(4 * n)
    rows = 512
    for r0 in range(0, K, rows):   # generated and uploaded in slices to bound host memory
        part = synth_normal(0x5EED1005, sigma, (rows * N,), first=r0 * N)
        _lib.check(ctx.lib.rbn_h2d(ctx.handle, d_w.ptr + 4 * r0 * N, part.ctypes.data, part.nbytes))
    d_p = ctx.alloc(ctx.lib.rbn_packed_capacity(n))
    out = {"K": K, "N": N, "weights": n}
    for name, mode in (("strict", _lib.SUM_STRICT_SEQ), ("tree", _lib.SUM_TREE)):
        ctx.quantize_ternary(d_w, n, mode, d_p)
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
    d_w.free()
    d_p.free()
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
            "weight_init_s": t_init, "launches_per_token": 5 * cfg.layers + 2,
            "bytes_per_token": {"packed_weights": w_bytes, "kv_cache_f16_avg": kv_bytes},
            "GBps": (w_bytes + kv_bytes) / per_tok / 1e9,
            "frac_hbm_peak": (w_bytes + kv_bytes) / per_tok / 1e9 / HBM_PEAK_GBS,
            "first_tokens": [int(t) for t in tokens[:8]]}


def dataclass_dict(obj):
    import dataclasses
    return dataclasses.asdict(obj)


def cpu_baseline(wl, out, acc, budget_s=20.0):
    """Times the CPU oracle on the headline inputs (one core) and gates parity."""
    from oracle import oracle as O
    q, s, rs = O.act_quant_i8(wl.x)
    t0 = time.perf_counter()
    tw = O.quantize_ternary(wl.w)
    t_quant = time.perf_counter() - t0
    reps, t_mm = 0, 0.0
    want_out = want_acc = None
    while reps < 2 or (t_mm < budget_s * 0.5 and reps < 40):
        t0 = time.perf_counter()
        want_out, want_acc = O.matmul_i8_ternary(q, s, tw)
        t_mm += time.perf_counter() - t0
        reps += 1
    t_mm /= reps
    parity = {
        "w_scale_bits_equal": bool(np.float32(wl.w_scale).view(np.uint32) == np.float32(tw.scale).view(np.uint32)),
        "acc_equal": bool((acc == want_acc).all()),
        "out_bits_equal": bool((out.view(np.uint32) == want_out.view(np.uint32)).all()),
    }
    gb = gemv_bytes(wl.M, wl.K, wl.N) / 1e9
    base = {
        "value": gb / t_mm, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": ("oracle matmul (reference's get_value inner loop, kernels.rs:159-165) on the "
                   "same M=%d K=%d N=%d operands, %d repetitions, %.3f s each; ternarising W "
                   "(quantize_ternary, sequential f32 sums) takes another %.3f s per call in the "
                   "reference, which repeats it on every execute()" % (wl.M, wl.K, wl.N, reps, t_mm, t_quant)),
        "ms_per_step": t_mm * 1e3,
        "ms_quantize_weights": t_quant * 1e3,
        "host_cpus": os.cpu_count(),
    }
    return base, parity


def profile_kernel(ctx, which, launches):
    """Launches one kernel `launches` times on its real shape, for rocprofv3 runs.

    gemv: M=1 K=4096 N=11008, rotating weight buffers.  skinny: M=16, same matrix.
    gemm: M=2048 K=4096 N=11008.
    pack / quantize: the 8192 x 28672 weight matrix of the large-layer config.
    copy: a device-to-device copy of 256 MiB, whose known traffic calibrates the
    FETCH_SIZE / WRITE_SIZE counters.
    """
    from ronn_amd import _lib
    from ronn_amd.device import synth_normal
    if which == "gemv":
        wl = Workload(ctx, 1, 4096, 11008, 0.02, seed=2, mode=1)
        for i in range(launches):
            wl.launch(ctx.gemv, i)
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
        d_w = ctx.alloc(4 * K * N)
        rows = 512
        for r0 in range(0, K, rows):   # generated and uploaded in slices to bound host memory
            part = synth_normal(0x5EED1005, 0.015, (rows * N,), first=r0 * N)
            _lib.check(ctx.lib.rbn_h2d(ctx.handle, d_w.ptr + 4 * r0 * N, part.ctypes.data, part.nbytes))
        d_p = ctx.alloc(ctx.lib.rbn_packed_capacity(K * N))
        for i in range(min(launches, 4)):
            if which == "pack":
                ctx.pack_ternary(d_w, K * N, 0.0028, d_p)
            else:
                ctx.quantize_ternary(d_w, K * N, _lib.SUM_STRICT_SEQ, d_p)
    elif which in ("decoder", "decoder_eager"):
        # decoder_eager launches kernel by kernel instead of replaying the captured graph
        # (for per-kernel traces: the profiler does not survive the 269-node graph)
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
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=400)
    ap.add_argument("--no-extra", action="store_true", help="headline only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity gate")
    ap.add_argument("--kernel", choices=["gemv", "skinny", "gemm", "pack", "quantize", "copy", "decoder", "decoder_eager"],
                    help="profiling aid: launch only this kernel a few times (for rocprofv3) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from ronn_amd.device import Context
    ctx = Context(0)
    info = ctx.device_info()
    if args.kernel:
        profile_kernel(ctx, args.kernel, max(1, min(args.steps, 64)))
        return

    M, K, N = 1, 4096, 11008
    wl = Workload(ctx, M, K, N, 0.02, seed=2, want_host=not args.no_cpu)
    out, acc = wl.results(ctx.gemv)
    ev_ms, wall_ms, n_timed = time_graph(ctx, wl, ctx.gemv, args.steps, args.warmup)
    bytes_per_launch = gemv_bytes(M, K, N)
    achieved = bytes_per_launch / (ev_ms * 1e-3) / 1e9

    result = {
        "metric": "ternary GEMV HBM GB/s (% of peak) + prefill int8 TOPS; BitNet decode tok/s",
        "value": bytes_per_launch / (wall_ms * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1, "steps": n_timed, "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x 2-bit ternary -> int32",
        "data": "synthetic (seeded N(0,1) activations, N(0,0.02) weights, absmean-ternarised on device)",
        "config": {"workload": "decode ternary GEMV, M=1 K=4096 N=11008 (FFN up/gate), weights rotated over %d "
                               "buffers (%.0f MiB) so each launch streams from HBM; HIP-graph replay"
                               % (len(wl.tiled), len(wl.tiled) * wl.tiled_bytes / 2**20),
                   "M": M, "K": K, "N": N, "device": info["name"], "arch": info["arch"],
                   "compute_units": info["compute_units"], "clock_mhz": info["clock_khz"] / 1000.0},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": GEMV_HEADLINE_TRAFFIC_BYTES,
                     "kernel": "gemv_t2_i8_kernel<1, 1, 4, true>", "bytes_per_launch": bytes_per_launch,
                     "us_per_launch": ev_ms * 1e3},
    }

    if not args.no_cpu:
        base, parity = cpu_baseline(wl, out, acc)
        result["cpu_baseline"] = base
        result["parity"] = parity
        if not all(parity.values()):
            print(json.dumps(result))
            print("bench.py: PARITY FAILURE against the CPU oracle: %s" % parity, file=sys.stderr)
            sys.exit(1)
    wl.w = None

    if not args.no_extra:
        extra = {}
        # warm variant: one buffer, lives in L2 / Infinity Cache
        one = Workload(ctx, M, K, N, 0.02, seed=2, rotate_bytes=1, mode=1)
        ev1, _, _ = time_graph(ctx, one, ctx.gemv, 2000, 200)
        extra["gemv_warm_cache"] = {"M": M, "K": K, "N": N, "us": ev1 * 1e3,
                                    "GBps": bytes_per_launch / (ev1 * 1e-3) / 1e9,
                                    "note": "single 11 MiB weight buffer re-read from cache, not HBM"}
        del one
        # One launch at a time on an idle stream, timed by the dispatch's own begin and end
        # timestamps: what a profiler's kernel trace reports.  Back to back (the timed region
        # above) a launch starts while the one before it drains, so a step is shorter than this.
        iso = Workload(ctx, M, K, N, 0.02, seed=2, mode=1)  # default rotation: more than the Infinity Cache
        iso_us = []
        for i in range(130):
            j = i % len(iso.tiled)
            iso_us.append(ctx.gemv_kernel_time_us(iso.acts, iso.tiled[j], iso.w_scale, M, K, N, iso.d_out))
        iso_us = sorted(iso_us[30:])
        extra["gemv_isolated_dispatch"] = {"us_mean": sum(iso_us) / len(iso_us), "us_median": iso_us[len(iso_us) // 2],
                                           "us_min": iso_us[0],
                                           "note": "begin-to-end timestamps of single dispatches on an idle stream "
                                                   "(rbn_gemv_t2_i8_kernel_time); compare rocprofv3's kernel trace"}
        del iso
        def kernel_for(m, k, n):
            return ("gemv", "skinny_mfma", "gemm_mfma")[ctx.lib.rbn_matmul_kernel_choice(m, k, n)]

        def sweep_over(shapes, ms, sigma):
            rows = []
            for (k, n) in shapes:
                for m in ms:
                    w2 = wl if (m, k, n) == (M, K, N) else Workload(ctx, m, k, n, sigma, seed=3, mode=1)
                    ev, _, _ = time_graph(ctx, w2, ctx.matmul, 1500, 150)
                    b = gemv_bytes(m, k, n)
                    rows.append({"M": m, "K": k, "N": n, "kernel": kernel_for(m, k, n), "us": ev * 1e3,
                                 "GBps": b / (ev * 1e-3) / 1e9,
                                 "frac_hbm_peak": b / (ev * 1e-3) / 1e9 / HBM_PEAK_GBS})
                    if w2 is not wl:
                        del w2
            return rows

        # rbn_matmul_t2_i8 picks the kernel by M; weights rotate through > 256 MiB of buffers
        extra["decode_sweep"] = sweep_over(((4096, 4096), (4096, 11008), (11008, 4096)), (1, 4, 16), 0.02)
        extra["large_layer"] = sweep_over(((8192, 28672),), (1, 8, 64), 0.015)
        extra["large_layer_ternarize"] = time_ternarize(ctx, 8192, 28672, 0.015)
        # prefill GEMM, int8 MFMA
        pm, pk, pn = 2048, 4096, 11008
        pw = Workload(ctx, pm, pk, pn, 0.02, seed=4, rotate_bytes=1, mode=1)
        # one burst of 20 back-to-back launches after a warm-up launch, as in the rocprofv3 profile
        # (longer bursts run into the power cap: the second and third burst of 20 take 15-20 % longer)
        ms = time_plain(ctx, lambda: pw.launch(ctx.gemm, 0), 20)
        ops = 2.0 * pm * pk * pn
        extra["prefill_gemm"] = {"M": pm, "K": pk, "N": pn, "ms": ms, "TOPS": ops / (ms * 1e-3) / 1e12,
                                 "frac_int8_peak": ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS,
                                 "roofline": {"bound": "mfma", "achieved": ops / (ms * 1e-3) / 1e12,
                                              "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                              "frac": ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS,
                                              "kernel": "gemm_t2_i8_mfma_kernel<2>"}}
        del pw
        # what a loop of nothing but int8 MFMA sustains on this box, by operand values
        extra["mfma_i8_probe_TOPS"] = {"constant_operands": ctx.probe_mfma_i8(0),
                                       "int8_x_ternary_codes": ctx.probe_mfma_i8(1),
                                       "int8_x_int8": ctx.probe_mfma_i8(2)}
        extra["decoder"] = time_decoder(ctx)
        result["extra"] = extra

    print(json.dumps(result))


if __name__ == "__main__":
    main()

// Exact parallel evaluation of a sequential f32 sum of non-negative terms.
//
// The reference computes `data.iter().map(|x| x.abs()).sum::<f32>()`
// (crates/ronn-providers/src/bitnet/quantization.rs:79 and :96): a strict left
// fold S <- fl(S + x_i) in f32.  Its result depends on the order, so a tree
// reduction cannot reproduce it.  This header holds the arithmetic that lets the
// fold be evaluated in parallel and still bit-exactly; it is shared by the HIP
// kernels and by a host build used in the CPU tests.
//
// Idea.  All terms are >= 0, so S never decreases.  While S stays inside one
// binade [2^e, 2^(e+1)) its ulp u = 2^(e-23) is fixed: S = k*u with an integer k in
// [2^23, 2^24).  Adding x = q*u + r (0 <= r < u) and rounding to nearest-even gives
//      k' = k + q + [r > u/2] + [r == u/2 and (k+q) odd]
// as long as the result stays <= 2^24 (the binade's upper edge, itself
// representable).  So each term acts on k as  k -> k + d(k mod 2)  with two small
// integers d(0), d(1); such maps compose associatively:
//      (B after A)(p) = A(p) + B((p + A(p)) mod 2).
// A block of terms therefore reduces, in parallel and in any grouping, to one pair
// (d0,d1) that is valid for every incoming k of the assumed binade.  Values that
// would leave the binade saturate at SEQ_SAT; the caller scans the block maps from
// the true k, finds the first block in which k reaches 2^24, replays that one block
// with ordinary f32 additions, and continues in the new binade.
//
// Subnormal S shares the ulp of the first normal binade, so biased exponent 0 is
// treated as exponent 1 with k in [0, 2^23).
#ifndef RONN_SEQSUM_CORE_H
#define RONN_SEQSUM_CORE_H

#include <stdint.h>

#if defined(__HIPCC__)
#define SEQ_HD __host__ __device__ __forceinline__
#else
#define SEQ_HD inline
#endif

#define SEQ_K_LIMIT (1u << 24)  // k >= this: S has left the binade
#define SEQ_SAT (1u << 25)      // saturation value of d0/d1
#define SEQ_BLOCK_ELEMS 4096u   // elements per block map

struct SeqMap {
    uint32_t d0;  // increment of k when the incoming k is even
    uint32_t d1;  // increment of k when the incoming k is odd
};

SEQ_HD SeqMap seq_identity() {
    SeqMap m;
    m.d0 = 0u;
    m.d1 = 0u;
    return m;
}

SEQ_HD uint32_t seq_min_u32(uint32_t a, uint32_t b) { return a < b ? a : b; }

// Splits the f32 state S (S >= 0, finite) into (es, k): S = k * 2^(es-150), es >= 1.
SEQ_HD void seq_state_split(uint32_t s_bits, uint32_t *es, uint32_t *k) {
    uint32_t e = (s_bits >> 23) & 0xffu;
    uint32_t f = s_bits & 0x7fffffu;
    *es = e == 0u ? 1u : e;
    *k = e == 0u ? f : (f | 0x800000u);
}

// Inverse of seq_state_split for k < 2^24.
SEQ_HD uint32_t seq_state_join(uint32_t es, uint32_t k) {
    if (k < 0x800000u) return k;  // subnormal or zero; es is 1 then
    return (es << 23) | (k & 0x7fffffu);
}

// Appends one term (|x| given as raw f32 bits with the sign bit already cleared)
// to the running map `m`, for a state whose exponent is `es`.  A non-finite term
// (Inf/NaN) saturates the map so the caller replays its block with real f32 adds.
SEQ_HD SeqMap seq_append(SeqMap m, uint32_t ax_bits, uint32_t es) {
    uint32_t e = ax_bits >> 23;
    uint32_t f = ax_bits & 0x7fffffu;
    uint32_t mx = e == 0u ? f : (f | 0x800000u);
    uint32_t ex = e == 0u ? 1u : e;
    uint32_t q, gt, eq;
    if (e == 0xffu || ex > es) {
        // non-finite, or a normal term at least 2 ulp-exponents above the state:
        // the sum leaves the binade for certain.
        q = SEQ_SAT;
        gt = 0u;
        eq = 0u;
    } else {
        uint32_t sh = es - ex;  // >= 0
        if (sh > 31u) sh = 31u;
        if (sh == 0u) {
            q = mx;
            gt = 0u;
            eq = 0u;
        } else {
            uint32_t half = 1u << (sh - 1u);
            uint32_t rem = mx & ((half << 1) - 1u);
            q = mx >> sh;
            gt = rem > half ? 1u : 0u;
            eq = rem == half ? 1u : 0u;
        }
    }
    uint32_t t0 = m.d0 + q;
    uint32_t t1 = m.d1 + q;
    // incoming parity p, current k parity = (p + d_p) & 1, after adding q: (p + t_p) & 1
    m.d0 = seq_min_u32(t0 + gt + (eq & (t0 & 1u)), SEQ_SAT);
    m.d1 = seq_min_u32(t1 + gt + (eq & ((t1 + 1u) & 1u)), SEQ_SAT);
    return m;
}

// 2^(150 - es) as a float: multiplying a term by it expresses the term in units of the
// state's ulp.  Representable for 23 <= es <= 276.
SEQ_HD float seq_ulp_scale(uint32_t es) {
    uint32_t bits = (277u - es) << 23;
    float f;
    __builtin_memcpy(&f, &bits, 4);
    return f;
}

// seq_append for a term given as a non-negative float, with `scale` = seq_ulp_scale(es).
// For es >= 26 the split of the term into (q, remainder) is done in floating point, which
// takes a third fewer operations than the integer version and gives the same (q, >, ==):
//   v = a * scale is exact (a power of two times a 24-bit mantissa) unless it overflows
//   (a is far above the binade: saturate, as the integer version does for any term whose
//   exponent exceeds the state's) or falls below 2^-126 (then a is below half an ulp
//   whatever the rounding of v does, and for es >= 26 every subnormal a is in this case);
//   floor(v) and v - floor(v) are exact for v < 2^25.
// v in [2^24, 2^25) is not saturated here but yields q >= 2^24, which takes any k >= 2^23
// past the limit just the same; the exact value of a map beyond the limit is never used.
SEQ_HD SeqMap seq_append_abs(SeqMap m, float a, uint32_t es, float scale) {
    if (es < 26u) {
        uint32_t bits;
        __builtin_memcpy(&bits, &a, 4);
        return seq_append(m, bits, es);
    }
    const float v = a * scale;
    uint32_t q = SEQ_SAT, gt = 0u, eq = 0u;
    if (v < 33554432.0f) {  // false for NaN as well
        const float fl = __builtin_floorf(v);
        const float fr = v - fl;
        q = (uint32_t)fl;
        gt = fr > 0.5f ? 1u : 0u;
        eq = fr == 0.5f ? 1u : 0u;
    }
    uint32_t t0 = m.d0 + q;
    uint32_t t1 = m.d1 + q;
    m.d0 = seq_min_u32(t0 + gt + (eq & (t0 & 1u)), SEQ_SAT);
    m.d1 = seq_min_u32(t1 + gt + (eq & ((t1 + 1u) & 1u)), SEQ_SAT);
    return m;
}

// The map of sixteen consecutive terms a[0..15] (non-negative; a term of +0.0 is the identity and
// stands for an element that the mask skips) for a state of exponent es, scale = seq_ulp_scale(es).
// A term changes k by q + [r > u/2] = round-to-nearest(v), v = a * scale, whatever k is - unless v
// lies exactly half way between two integers, the one case in which the parity of k decides.  So
// when none of the sixteen is such a tie (the rule: a tie needs a term whose low bits are exactly
// 1000...0 at the state's ulp), the map is one sum of sixteen independent roundings, d0 = d1, and
// the sixteen terms do not wait for each other as they do in seq_append_abs; with a tie among them
// the terms are appended one by one.  v is clamped to 2^25 = SEQ_SAT first (NaN included), so a
// sum of sixteen stays below 2^32 and a term far above the binade saturates the map exactly as it
// does in seq_append_abs.
// Maps without a tie are plain increments (d0 = d1), and composing increments is adding them, in any
// order and any grouping: as long as no term of a whole block is a tie, the block's map is the
// (saturated) sum of all its roundings however its elements are dealt to the threads.
//
// The sum of the sixteen roundings, and in *tie whether it may NOT be used: a term is an exact tie,
// or es < 26 (there the term is split in integer arithmetic, by seq_append).
SEQ_HD uint32_t seq_sum16(const float *a, uint32_t es, float scale, bool *tie) {
    // Stage by stage over all sixteen terms, so that what a wave issues back to back is independent
    // (term by term every instruction waited for the one before it: 0.6 us per call where one wave
    // has a SIMD to itself).
    float v[16], r[16];
    for (int i = 0; i < 16; ++i) {
        // the clamp on the bit patterns: for v >= +0 they order as the values do, NaNs above all
        const float p = a[i] * scale;
        uint32_t vb;
        __builtin_memcpy(&vb, &p, 4);
        vb = seq_min_u32(vb, 0x4c000000u);  // 2^25
        __builtin_memcpy(&v[i], &vb, 4);
    }
    for (int i = 0; i < 16; ++i) r[i] = __builtin_rintf(v[i]);  // to nearest, ties to even (the default rounding mode)
    // |v - r| <= 1/2, with equality exactly for a tie: one maximum instead of sixteen comparisons
    float off = 0.0f;
    for (int i = 0; i < 16; ++i) off = __builtin_fmaxf(off, __builtin_fabsf(v[i] - r[i]));
    uint32_t sum = 0u;
    for (int i = 0; i < 16; ++i) sum += (uint32_t)r[i];
    *tie = es < 26u || off == 0.5f;
    return sum;
}

SEQ_HD SeqMap seq_map16(const float *a, uint32_t es, float scale) {
    SeqMap m = seq_identity();
    bool tie;
    const uint32_t sum = seq_sum16(a, es, scale, &tie);
    if (!tie) {
        m.d0 = m.d1 = seq_min_u32(sum, SEQ_SAT);
    } else {
        for (int i = 0; i < 16; ++i) m = seq_append_abs(m, a[i], es, scale);
    }
    return m;
}

// Map of "first a, then b".
SEQ_HD SeqMap seq_compose(SeqMap a, SeqMap b) {
    SeqMap r;
    uint32_t b_after_even = (a.d0 & 1u) ? b.d1 : b.d0;        // parity (0 + a.d0) & 1
    uint32_t b_after_odd = ((a.d1 + 1u) & 1u) ? b.d1 : b.d0;  // parity (1 + a.d1) & 1
    r.d0 = seq_min_u32(a.d0 + b_after_even, SEQ_SAT);
    r.d1 = seq_min_u32(a.d1 + b_after_odd, SEQ_SAT);
    return r;
}

// Applies a map to a concrete k.
SEQ_HD uint32_t seq_apply(SeqMap m, uint32_t k) { return k + ((k & 1u) ? m.d1 : m.d0); }

// ---- window policy ---------------------------------------------------------------------------
// The block maps of a window are valid for one binade, so a window should end where S is
// expected to leave it.  `s_now` is the current sum, `rate` its growth per block (<= 0: unknown)
// measured over `rate_elems` elements.  The growth differs from binade to binade (in a higher one
// rounding eats more of every term, up to all of it), so the rate that counts is the one since S
// entered its present binade: the window-end kernel measures it from the last crossing on, be it
// over the rest of the crossing block only.  Without a rate the window is half again what has been
// summed so far (S of similar terms doubles when the position doubles); with one, the distance to
// the binade's upper edge at that rate plus a margin of 10 % and of 2.5 standard errors of a mean of
// `rate_elems` half-normal terms (0.75 / sqrt(m) each).  A window that ends short of the crossing
// costs a pair of launches (12 us); the blocks past a crossing are the only wasted reads (2.5 ns
// each).
#include <math.h>
SEQ_HD uint64_t seq_next_window(uint64_t pos, uint64_t total_blocks, double s_now, double rate, double rate_elems) {
    uint64_t win = pos + pos / 2;
    if (rate > 0.0 && s_now > 0.0 && isfinite(s_now)) {
        int e = 0;
        (void)frexp(s_now, &e);  // s_now = m * 2^e, m in [0.5, 1): the binade ends at 2^e
        const double need = (ldexp(1.0, e) - s_now) / rate;
        const double margin = 1.10 + (rate_elems >= 1.0 && rate_elems < 1e8 ? 1.9 / sqrt(rate_elems) : 0.0);
        win = need < 1e15 ? (uint64_t)(need * margin) + 4u : total_blocks;
    }
    if (win < 64u) win = 64u;
    if (win > total_blocks - pos) win = total_blocks - pos;
    return win;
}

// The growth per block that sizes the next window, from what a window saw: S before and after it,
// the blocks it folded, S right behind its last crossing (s_before when there was none) and the
// blocks folded since (a fraction when the window ended inside the crossing block).  Fewer than 64
// elements behind the crossing say too little: then the average over the window stands in.  The
// first window of a sum (s_before = 0) always takes its average: S climbs through its first
// binades inside one block, at one rate.
SEQ_HD double seq_window_rate(double s_before, double s_after, double advanced, double s_cross, double since_cross,
                              double *rate_elems) {
    double rate = advanced > 0.0 ? (s_after - s_before) / advanced : 0.0;
    *rate_elems = advanced * (double)SEQ_BLOCK_ELEMS;
    if (s_before > 0.0 && since_cross * (double)SEQ_BLOCK_ELEMS >= 64.0 && since_cross <= advanced) {
        rate = (s_after - s_cross) / since_cross;
        *rate_elems = since_cross * (double)SEQ_BLOCK_ELEMS;
    }
    return rate;
}

// ---- where a window's block maps lie -------------------------------------------------------------
// The window-end kernel gives each of its 1024 threads a run of consecutive blocks: `chunk` =
// ceil(win / 1024) of them up to 32, and longer windows in stretches of 32768 blocks, 32 per thread.
// The maps are stored transposed to that: the i-th block of thread t's run lies at slot
// i * 1024 + t (of its stretch), so that what the 64 lanes of a wave load together is contiguous
// (with the maps in block order every lane asked for a cache line of its own, and one compute unit
// took 10 us for 32768 maps).  Slots stay below win rounded up to 1024, or to 32768 in stretches.
#define SEQ_SCAN_THREADS 1024u
#define SEQ_SCAN_RUN 32u  // the longest run of blocks per thread
SEQ_HD uint32_t seq_map_slot(uint32_t block, uint32_t win) {
    if (win <= SEQ_SCAN_THREADS) return block;
    const uint32_t stretch_blocks = SEQ_SCAN_THREADS * SEQ_SCAN_RUN;
    if (win <= stretch_blocks) {
        const uint32_t chunk = (win + SEQ_SCAN_THREADS - 1u) / SEQ_SCAN_THREADS;
        return (block % chunk) * SEQ_SCAN_THREADS + block / chunk;
    }
    const uint32_t r = block % stretch_blocks;
    return (block - r) + (r % SEQ_SCAN_RUN) * SEQ_SCAN_THREADS + r / SEQ_SCAN_RUN;
}

// ---- windows that span several binades ------------------------------------------------------
// The first binades are short: S of similar terms doubles when the position doubles, so the
// first 8192 blocks hold thirteen of them, and a window per binade spends its time on launches.
// A window that starts below SEQ_MULTI_LIMIT therefore carries TWO maps per block, for the
// exponents e and e + 1 where e = seq_multi_es_lo() is the exponent that a cautious prediction
// of S gives for that block: L(i) = S0 + i * rate_lo with rate_lo = 0.9 x the growth per block
// measured over the previous window.  The true S entering block i has exponent e or e + 1
// whenever L(i) <= S < 2 L(i), i.e. for any growth between 0.9 and 1.8 times the measured one;
// the scan then walks through the binades inside one window (scan to the crossing, replay that
// block, go on with the other map) and ends the window early at the first block whose pair does
// not hold the exponent S really has.  Block 0 of a window always does (L(0) = S0).
#define SEQ_MULTI_LIMIT 8192u

SEQ_HD uint32_t seq_multi_es_lo(uint32_t s0_bits, uint32_t rate_lo_bits, uint32_t i) {
    float s0, r;
    __builtin_memcpy(&s0, &s0_bits, 4);
    __builtin_memcpy(&r, &rate_lo_bits, 4);
    const float l = __builtin_fmaf((float)i, r, s0);  // one rounding, the same wherever it is evaluated
    uint32_t b;
    __builtin_memcpy(&b, &l, 4);
    const uint32_t e = (b >> 23) & 0xffu;
    return e == 0u ? 1u : (e > 254u ? 254u : e);
}

// rate_lo as f32 bits from the growth per block of the last window (0 when there is none to trust)
SEQ_HD uint32_t seq_multi_rate_lo(double rate) {
    float r = 0.0f;
    if (rate > 0.0 && rate < 1e38) r = (float)(0.9 * rate);
    uint32_t b;
    __builtin_memcpy(&b, &r, 4);
    return b;
}

// The next window: its size, and in *multi whether it carries two maps per block.
SEQ_HD uint64_t seq_plan_window(uint64_t pos, uint64_t total_blocks, double s_now, double rate, double rate_elems,
                                uint32_t *multi) {
    if (pos == 0u) {  // S = +0 has no binade to make maps for: the first block is resolved on its own
        *multi = 0u;
        return 1u;
    }
    if (pos > 0u && pos < SEQ_MULTI_LIMIT && isfinite(s_now)) {
        // all the way to the limit: the growth measured over the first block alone is good to a few per
        // cent for terms of similar size, well inside what the pair of exponents allows (a window of a
        // few hundred blocks in between, to measure it better, cost a pair of launches for nothing)
        uint64_t win = SEQ_MULTI_LIMIT - pos;
        if (win > total_blocks - pos) win = total_blocks - pos;
        *multi = 1u;
        return win;
    }
    *multi = 0u;
    return seq_next_window(pos, total_blocks, s_now, rate, rate_elems);
}

#endif  // RONN_SEQSUM_CORE_H

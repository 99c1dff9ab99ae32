// Host replica of the device's exact sequential-sum driver (ronn_amd/csrc/ternarize.hip:
// seq_block_maps_kernel, seq_scan_replay_kernel, strict_abs_sum), built on
// the same arithmetic header.  It lets the CPU test-suite check the algorithm against
// a literal `s = s + |x|` loop on any input, without a GPU.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "../../ronn_amd/csrc/seqsum_core.h"

namespace {
constexpr int kTile = 4096;

SeqMap thread_map(const float *x, uint64_t base, uint64_t n, uint32_t es, int use_mask, float thr) {
    const float scale = seq_ulp_scale(es < 26u ? 26u : es);
    float a[16];
    for (int i = 0; i < 16; ++i) {
        uint64_t idx = base + i;
        a[i] = 0.0f;  // an element past the end or under the mask: the identity
        if (idx < n) {
            float v = std::fabs(x[idx]);
            bool take = use_mask ? (v > thr) : true;
            if (take) a[i] = v;
        }
    }
    return seq_map16(a, es, scale);
}

// The same map term by term (the form seq_map16 falls back to on a tie), for the comparison test.
SeqMap thread_map_serial(const float *a, uint32_t es) {
    SeqMap m = seq_identity();
    const float scale = seq_ulp_scale(es < 26u ? 26u : es);
    for (int i = 0; i < 16; ++i) m = seq_append_abs(m, a[i], es, scale);
    return m;
}

SeqMap block_map(const float *x, uint64_t first, uint64_t n, uint32_t es, int use_mask, float thr) {
    SeqMap lanes[256];
    for (int t = 0; t < 256; ++t) lanes[t] = thread_map(x, first + (uint64_t)t * 16, n, es, use_mask, thr);
    SeqMap waves[4];
    for (int w = 0; w < 4; ++w) {
        SeqMap v[64];
        for (int l = 0; l < 64; ++l) v[l] = lanes[w * 64 + l];
        for (int off = 1; off < 64; off <<= 1) {
            SeqMap nv[64];
            for (int l = 0; l < 64; ++l) {
                SeqMap o = (l + off < 64) ? v[l + off] : v[l];  // out-of-range shuffles return own value
                nv[l] = seq_compose(v[l], o);
            }
            for (int l = 0; l < 64; ++l) v[l] = nv[l];
        }
        waves[w] = v[0];
    }
    SeqMap t = waves[0];
    for (int w = 1; w < 4; ++w) t = seq_compose(t, waves[w]);
    return t;
}

struct ScanResult {
    uint32_t cross_block;
    uint32_t k;
};

ScanResult scan_stretch(const std::vector<SeqMap> &maps, uint32_t from, uint32_t to, uint32_t k0, SeqMap *total);

// The scan of a window: in one piece up to 32768 blocks (32 maps per thread), longer ones in
// stretches of 32768, each from the state the stretch before it ends in.
ScanResult scan(const std::vector<SeqMap> &maps, uint32_t s_bits) {
    const uint32_t nblocks = (uint32_t)maps.size();
    uint32_t es, k0;
    seq_state_split(s_bits, &es, &k0);
    SeqMap total;
    if (nblocks <= 32768u) return scan_stretch(maps, 0, nblocks, k0, &total);
    uint32_t k_in = k0;
    for (uint32_t from = 0;; from += 32768u) {
        const uint32_t to = nblocks - from > 32768u ? from + 32768u : nblocks;
        ScanResult r = scan_stretch(maps, from, to, k_in, &total);
        if (r.cross_block != 0xffffffffu || to == nblocks) return r;
        k_in = seq_apply(total, k_in);
    }
}

// Blocks [from, to) of the window from the state k0: the first block in which k reaches 2^24 (as an
// index into the window) and the k that enters it, or no block and the k after the last one.
ScanResult scan_stretch(const std::vector<SeqMap> &all_maps, uint32_t from, uint32_t to, uint32_t k0, SeqMap *total) {
    const std::vector<SeqMap> maps(all_maps.begin() + from, all_maps.begin() + to);
    const uint32_t nblocks = to - from;
    const uint32_t chunk = (nblocks + 1023u) / 1024u;
    std::vector<SeqMap> a(1024), b(1024);
    for (uint32_t t = 0; t < 1024; ++t) {
        uint32_t lo = t * chunk, hi = lo + chunk < nblocks ? lo + chunk : nblocks;
        SeqMap mine = seq_identity();
        for (uint32_t i = lo; i < hi; ++i) mine = seq_compose(mine, maps[i]);
        a[t] = mine;
    }
    std::vector<SeqMap> *src = &a, *dst = &b;
    for (uint32_t off = 1; off < 1024u; off <<= 1) {
        for (uint32_t t = 0; t < 1024; ++t) {
            SeqMap v = (*src)[t];
            if (t >= off) v = seq_compose((*src)[t - off], v);
            (*dst)[t] = v;
        }
        std::swap(src, dst);
    }
    ScanResult r{0xffffffffu, 0};
    uint32_t first = 0xffffffffu;
    std::vector<uint32_t> cand(1024, 0xffffffffu), cand_k(1024, 0), last_k(1024, 0);
    for (uint32_t t = 0; t < 1024; ++t) {
        uint32_t lo = t * chunk, hi = lo + chunk < nblocks ? lo + chunk : nblocks;
        SeqMap before = t == 0 ? seq_identity() : (*src)[t - 1];
        uint32_t k = seq_apply(before, k0);
        if (k < SEQ_K_LIMIT) {
            for (uint32_t i = lo; i < hi; ++i) {
                uint32_t k2 = seq_apply(maps[i], k);
                if (k2 >= SEQ_K_LIMIT) {
                    cand[t] = i;
                    cand_k[t] = k;
                    break;
                }
                k = k2;
            }
        }
        last_k[t] = k;
        if (cand[t] < first) first = cand[t];
    }
    for (uint32_t t = 0; t < 1024; ++t) {
        uint32_t lo = t * chunk, hi = lo + chunk < nblocks ? lo + chunk : nblocks;
        if (first != 0xffffffffu) {
            if (cand[t] == first) r = ScanResult{from + first, cand_k[t]};
        } else if (hi == nblocks && lo < hi) {
            r = ScanResult{0xffffffffu, last_k[t]};
        }
    }
    *total = (*src)[1023];
    return r;
}
}  // namespace

// Counters of the two-barrier replay below: blocks it was tried on, blocks it resolved, and blocks
// where its result differed from the general replay's (must stay 0).
static uint64_t g_once_tried = 0, g_once_used = 0, g_once_differs = 0;
extern "C" void seqsum_once_stats(uint64_t *tried, uint64_t *used, uint64_t *differs) {
    *tried = g_once_tried, *used = g_once_used, *differs = g_once_differs;
}

// The usual crossing block as the device resolves it with two barriers: the quarters' maps for the
// state's exponent and the next one, the quarter and then the chunk in which k reaches 2^24, that
// chunk replayed, the chunks behind it and the quarters behind them for the new exponent.  Returns
// false when the block is not of that kind.
static bool replay_block_once(const float *x, uint64_t n, uint64_t bbase, int use_mask, float thr, uint32_t es,
                              uint32_t k_cur, uint32_t *result_bits, uint32_t *cross_bits, uint32_t *cross_chunks) {
    if (es < 26u || es + 1u > 253u) return false;
    SeqMap m0[256], m1[256], q0[4], q1[4];
    for (int t = 0; t < 256; ++t) {
        m0[t] = thread_map(x, bbase + (uint64_t)t * 16, n, es, use_mask, thr);
        m1[t] = thread_map(x, bbase + (uint64_t)t * 16, n, es + 1u, use_mask, thr);
    }
    for (int w = 0; w < 4; ++w) {
        q0[w] = q1[w] = seq_identity();
        for (int l = 0; l < 64; ++l) {
            q0[w] = seq_compose(q0[w], m0[w * 64 + l]);
            q1[w] = seq_compose(q1[w], m1[w * 64 + l]);
        }
    }
    int q = -1;
    uint32_t kq = k_cur, k = k_cur;
    for (int w = 0; w < 4; ++w) {
        const uint32_t k2 = seq_apply(q0[w], k);
        if (q < 0 && k2 >= SEQ_K_LIMIT) q = w, kq = k;
        if (q < 0) k = k2;
    }
    if (q < 0) return false;
    int tstar = -1;
    uint32_t kl = kq;
    for (int l = 0; l < 64; ++l) {
        if (kl < SEQ_K_LIMIT && seq_apply(m0[q * 64 + l], kl) >= SEQ_K_LIMIT) {
            tstar = l;
            break;
        }
        kl = seq_apply(m0[q * 64 + l], kl);
    }
    if (tstar < 0) return false;
    const uint32_t jb = seq_state_join(es, kl);
    float s;
    std::memcpy(&s, &jb, 4);
    for (int i = 0; i < 16; ++i) {
        const uint64_t idx = bbase + (uint64_t)(q * 64 + tstar) * 16 + i;
        float av = 0.0f;
        bool take = false;
        if (idx < n) {
            av = std::fabs(x[idx]);
            take = use_mask ? (av > thr) : true;
        }
        volatile float t2 = s + (take ? av : 0.0f);
        s = t2;
    }
    uint32_t bits;
    std::memcpy(&bits, &s, 4);
    uint32_t es2, k2;
    seq_state_split(bits, &es2, &k2);
    if (((bits >> 23) & 0xffu) == 0xffu || es2 != es + 1u) return false;
    SeqMap tail = seq_identity();
    for (int l = tstar + 1; l < 64; ++l) tail = seq_compose(tail, m1[q * 64 + l]);
    uint32_t k3 = seq_apply(tail, k2);
    if (k3 >= SEQ_K_LIMIT) return false;
    for (int w = q + 1; w < 4; ++w) {
        k3 = seq_apply(q1[w], k3);
        if (k3 >= SEQ_K_LIMIT) return false;
    }
    *result_bits = seq_state_join(es + 1u, k3);
    *cross_bits = bits, *cross_chunks = (uint32_t)(q * 64 + tstar + 1);
    return true;
}

// The replay of one block (the second half of the window-end kernel): crossings inside the
// block are resolved one after another.  Returns the state after the block as f32 bits.
static uint32_t replay_block(const float *x, uint64_t n, uint64_t bbase, int use_mask, float thr,
                             uint32_t es, uint32_t k_cur, uint32_t *cross_bits, uint32_t *cross_chunks) {
    uint32_t done = 0, result_bits = 0;
    *cross_bits = seq_state_join(es, k_cur), *cross_chunks = 0;
    for (int guard = 0; guard <= 256; ++guard) {
        SeqMap cm[256], a[256], b2[256];
        for (int t = 0; t < 256; ++t)
            cm[t] = (uint32_t)t >= done ? thread_map(x, bbase + (uint64_t)t * 16, n, es, use_mask, thr)
                                        : seq_identity();
        for (int t = 0; t < 256; ++t) a[t] = cm[t];
        SeqMap *src = a, *dst = b2;
        for (int off = 1; off < 256; off <<= 1) {
            for (int t = 0; t < 256; ++t) {
                SeqMap v = src[t];
                if (t >= off) v = seq_compose(src[t - off], v);
                dst[t] = v;
            }
            std::swap(src, dst);
        }
        int tstar = -1;
        uint32_t kstar = 0;
        for (int t = 0; t < 256; ++t) {
            SeqMap before = t == 0 ? seq_identity() : src[t - 1];
            uint32_t kk = seq_apply(before, k_cur);
            if ((uint32_t)t >= done && kk < SEQ_K_LIMIT && seq_apply(cm[t], kk) >= SEQ_K_LIMIT) {
                tstar = t;
                kstar = kk;
                break;
            }
        }
        if (tstar < 0) {
            result_bits = seq_state_join(es, seq_apply(src[255], k_cur));
            break;
        }
        uint32_t jb = seq_state_join(es, kstar);
        float s;
        std::memcpy(&s, &jb, 4);
        for (int i = 0; i < 16; ++i) {
            uint64_t idx = bbase + (uint64_t)tstar * 16 + i;
            float av = 0.0f;
            bool take = false;
            if (idx < n) {
                av = std::fabs(x[idx]);
                take = use_mask ? (av > thr) : true;
            }
            volatile float t2 = s + (take ? av : 0.0f);
            s = t2;
        }
        std::memcpy(&result_bits, &s, 4);
        done = (uint32_t)tstar + 1;
        *cross_bits = result_bits, *cross_chunks = done;
        if (((result_bits >> 23) & 0xff) == 0xff) {
            for (uint64_t idx = bbase + (uint64_t)done * 16; idx < bbase + kTile && idx < n; ++idx) {
                bool take = use_mask ? (std::fabs(x[idx]) > thr) : true;
                if (take && x[idx] != x[idx]) result_bits |= 0x7fc00000u;
            }
            break;
        }
        if (done >= 256) break;
        seq_state_split(result_bits, &es, &k_cur);
    }
    return result_bits;
}

extern "C" float seqsum_host(const float *x, uint64_t n, int use_mask, float thr,
                             uint64_t *iterations, uint64_t *elements_read) {
    uint64_t iters = 0, read = 0;
    if (n == 0) {
        if (iterations) *iterations = 0;
        if (elements_read) *elements_read = 0;
        return -0.0f;
    }
    const uint64_t total_blocks = (n + kTile - 1) / kTile;
    uint64_t pos = 0;  // in blocks
    uint32_t s_bits = 0;
    double rate = 0.0, rate_elems = 0.0;
    while (pos < total_blocks) {
        if (((s_bits >> 23) & 0xff) == 0xff) break;
        uint32_t es0, k0;
        seq_state_split(s_bits, &es0, &k0);
        float s_before;
        std::memcpy(&s_before, &s_bits, 4);
        uint32_t multi = 0;
        const uint64_t win = seq_plan_window(pos, total_blocks, (double)s_before, rate, rate_elems, &multi);
        const uint32_t rate_lo = seq_multi_rate_lo(rate);
        const uint32_t nm = multi ? 2u : 1u;
        const uint64_t first = pos * kTile;
        // the maps kernel: one map per block for the state's exponent, or two for the pair that the
        // prediction gives the block
        std::vector<uint32_t> elo(win);
        std::vector<SeqMap> maps(win * nm);
        for (uint64_t b = 0; b < win; ++b) {
            elo[b] = multi ? seq_multi_es_lo(s_bits, rate_lo, (uint32_t)b) : es0;
            for (uint32_t j = 0; j < nm; ++j)
                maps[b * nm + j] = block_map(x, first + b * kTile, n, elo[b] + j, use_mask, thr);
        }
        read += win * kTile;
        // the window-end kernel: scan to the crossing, replay that block, go on in the new binade
        // while the blocks' maps hold it
        uint64_t b_cur = 0;
        uint32_t cur_bits = s_bits;
        // the last crossing of the window: S right behind its chunk, and where it was
        bool crossed = false;
        uint32_t cross_bits = s_bits, cross_chunks = 0;
        uint64_t cross_block = 0;
        for (int guard = 0; guard < 64; ++guard) {
            uint32_t es, k;
            seq_state_split(cur_bits, &es, &k);
            uint64_t range_end = b_cur;
            while (range_end < win && es >= elo[range_end] && es - elo[range_end] < nm) ++range_end;
            if (range_end == b_cur) break;
            std::vector<SeqMap> sel(range_end - b_cur);
            for (uint64_t b = b_cur; b < range_end; ++b) sel[b - b_cur] = maps[b * nm + (es - elo[b])];
            ScanResult sr = scan(sel, cur_bits);
            if (sr.cross_block == 0xffffffffu) {
                cur_bits = seq_state_join(es, sr.k);
                b_cur = range_end;
                break;
            }
            cur_bits = replay_block(x, n, first + (b_cur + sr.cross_block) * kTile, use_mask, thr, es, sr.k,
                                    &cross_bits, &cross_chunks);
            if (pos + b_cur + sr.cross_block > 0) {  // (the first block of a sum is always replayed in general)
                uint32_t once_bits, once_cross, once_chunks;
                ++g_once_tried;
                if (replay_block_once(x, n, first + (b_cur + sr.cross_block) * kTile, use_mask, thr, es, sr.k,
                                      &once_bits, &once_cross, &once_chunks)) {
                    ++g_once_used;
                    if (once_bits != cur_bits || once_cross != cross_bits || once_chunks != cross_chunks)
                        ++g_once_differs;
                }
            }
            crossed = true, cross_block = b_cur + sr.cross_block;
            b_cur += (uint64_t)sr.cross_block + 1;
            if (((cur_bits >> 23) & 0xff) == 0xff || b_cur >= win) break;
        }
        if (b_cur == 0) return NAN;  // no progress: cannot happen (block 0 holds the state's exponent)
        s_bits = cur_bits;
        float s_after;
        std::memcpy(&s_after, &s_bits, 4);
        float s_cross;
        std::memcpy(&s_cross, &cross_bits, 4);
        const double since = !crossed ? (double)b_cur
                                      : (double)(b_cur - cross_block - 1) + (double)(256u - cross_chunks) / 256.0;
        rate = seq_window_rate((double)s_before, (double)s_after, (double)b_cur, (double)s_cross,
                               since, &rate_elems);
        pos += b_cur;
        ++iters;
    }
    float s;
    std::memcpy(&s, &s_bits, 4);
    if (((s_bits >> 23) & 0xff) == 0xff && s == s && pos < total_blocks && !use_mask) {
        for (uint64_t i = pos * kTile; i < n; ++i)
            if (x[i] != x[i]) s = NAN;
    }
    if (iterations) *iterations = iters;
    if (elements_read) *elements_read = read;
    if (use_mask) {
        // nothing survived the mask: the fold never ran and keeps Rust's initial -0.0
        // (the device entry point knows this from the survivor count)
        bool any = false;
        for (uint64_t i = 0; i < n && !any; ++i) any = std::fabs(x[i]) > thr;
        if (!any) return -0.0f;
    }
    return s;
}

// The literal fold the reference performs (quantization.rs:79 / :96).
extern "C" float seqsum_literal(const float *x, uint64_t n, int use_mask, float thr) {
    volatile float s = -0.0f;
    for (uint64_t i = 0; i < n; ++i) {
        float a = std::fabs(x[i]);
        bool take = use_mask ? (a > thr) : true;
        if (take) s = s + a;
    }
    return s;
}

// seq_map16 against sixteen seq_append_abs on `count` pseudo-random groups of sixteen terms around
// the state's ulp (short mantissas, so that ties happen; zeros, huge terms, Inf and NaN among them).
// Returns the number of disagreements (both at or above the limit counts as agreement).
extern "C" uint64_t seqsum_compare_map16(uint64_t count, uint64_t seed, uint64_t *groups_with_a_tie) {
    uint64_t bad = 0, ties = 0, x = seed * 0x9E3779B97F4A7C15ull + 1;
    auto next = [&]() {
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        return x;
    };
    for (uint64_t g = 0; g < count; ++g) {
        const uint32_t es = 20u + (uint32_t)(next() % 235u);  // 20 .. 254: both term splits
        float a[16];
        for (int i = 0; i < 16; ++i) {
            uint32_t ex = es - 27u + (uint32_t)(next() % 30u);  // ulp/8 .. far above
            if (ex > 255u) ex = 0u;
            uint32_t frac = (uint32_t)(next() & 0x7fffffu);
            switch (next() % 8u) {
                case 0: frac = 0; break;
                case 1: frac &= 0x700000u; break;
                case 2: frac = 0x400000u; break;
                case 3: ex = 0; frac = 0; break;            // +0.0
                case 4: if (next() % 64u == 0) ex = 255u; break;  // Inf / NaN now and then
                default: break;
            }
            const uint32_t bits = (ex << 23) | frac;
            std::memcpy(&a[i], &bits, 4);
        }
        const float scale = seq_ulp_scale(es < 26u ? 26u : es);
        bool tie = false;
        for (int i = 0; i < 16 && es >= 26u; ++i) {
            const float v = a[i] * scale;
            if (v < 33554432.0f && v - std::floor(v) == 0.5f) tie = true;
        }
        ties += tie ? 1 : 0;
        const SeqMap want = thread_map_serial(a, es), got = seq_map16(a, es, scale);
        const bool w_over = want.d0 >= SEQ_K_LIMIT / 2 || want.d1 >= SEQ_K_LIMIT / 2;
        if (w_over) {
            if (got.d0 < SEQ_K_LIMIT / 2 || got.d1 < SEQ_K_LIMIT / 2) ++bad;
        } else if (got.d0 != want.d0 || got.d1 != want.d1) {
            ++bad;
        }
    }
    if (groups_with_a_tie) *groups_with_a_tie = ties;
    return bad;
}

// A whole block as the maps kernel's streaming form computes it (elements dealt to the threads as a
// copy would deal them, every thread's sixteen roundings summed, the sums added up) against the
// ordered form (block_map), on `count` pseudo-random blocks of 4096 terms around the state's ulp.
// The streaming form is only used when no term is a tie; returns the number of blocks in which it
// would have been used and disagrees, and in *used how many blocks it would have been used for.
extern "C" uint64_t seqsum_compare_block_forms(uint64_t count, uint64_t seed, uint64_t *used) {
    uint64_t bad = 0, fast = 0, x = seed * 0x9E3779B97F4A7C15ull + 1;
    auto next = [&]() {
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        return x;
    };
    std::vector<float> blk(kTile);
    for (uint64_t g = 0; g < count; ++g) {
        const uint32_t es = 26u + (uint32_t)(next() % 200u);
        const bool short_mantissas = next() % 4u == 0;  // ties happen in these blocks
        for (int i = 0; i < kTile; ++i) {
            // ulp/8 .. 512 ulp: the lower bits of such a term are exactly 1000...0 once in 2^3 .. 2^14 draws,
            // so some blocks hold a tie and most do not
            uint32_t ex = es - 26u + (uint32_t)(next() % 13u);
            uint32_t frac = (uint32_t)(next() & 0x7fffffu);
            if (short_mantissas && next() % 64u == 0) frac &= 0x600000u;
            if (next() % 5u == 0) { ex = 0; frac = 0; }
            const uint32_t bits = (ex << 23) | frac;
            std::memcpy(&blk[i], &bits, 4);
        }
        const float scale = seq_ulp_scale(es);
        uint64_t total = 0;
        bool any_tie = false;
        for (int t = 0; t < 256; ++t) {
            float a[16];
            for (int j = 0; j < 4; ++j)
                for (int i = 0; i < 4; ++i) a[4 * j + i] = blk[4 * (j * 256 + t) + i];
            bool tie;
            const uint32_t sum = seq_sum16(a, es, scale, &tie);
            any_tie = any_tie || tie;
            total += seq_min_u32(sum, SEQ_SAT);
        }
        if (any_tie) continue;
        ++fast;
        const uint32_t d = total > SEQ_SAT ? SEQ_SAT : (uint32_t)total;
        const SeqMap want = block_map(blk.data(), 0, kTile, es, 0, 0.0f);
        const bool w_over = want.d0 >= SEQ_K_LIMIT / 2 || want.d1 >= SEQ_K_LIMIT / 2;
        if (w_over ? d < SEQ_K_LIMIT / 2 : (want.d0 != d || want.d1 != d)) ++bad;
    }
    if (used) *used = fast;
    return bad;
}

// Compares the floating-point term split (seq_append_abs, es >= 26) with the integer one
// (seq_append) on `count` pseudo-random (map, term, exponent) triples.  Returns the number
// of disagreements: below the limit the maps must be identical; at or above it both must
// be at or above it (the exact value is never used there).
extern "C" uint64_t seqsum_compare_term_splits(uint64_t count, uint64_t seed) {
    uint64_t bad = 0, x = seed * 0x9E3779B97F4A7C15ull + 1;
    auto next = [&]() {
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        return x;
    };
    for (uint64_t i = 0; i < count; ++i) {
        const uint32_t es = 26u + (uint32_t)(next() % 229u);  // 26 .. 254
        SeqMap m;
        m.d0 = (uint32_t)(next() % 5u == 0 ? next() % (1u << 24) : next() % 64u);
        m.d1 = m.d0 + (uint32_t)(next() % 2u);
        // a term near the state's ulp, sometimes far off, sometimes special
        uint32_t ex = es - 30u + (uint32_t)(next() % 40u);  // es-30 .. es+9
        if (next() % 16u == 0) ex = (uint32_t)(next() % 256u);
        if (ex > 255u) ex = 0u;
        uint32_t frac = (uint32_t)(next() & 0x7fffffu);
        switch (next() % 8u) {
            case 0: frac = 0; break;
            case 1: frac &= 0x7f0000u; break;          // short mantissas: ties happen
            case 2: frac = 0x400000u; break;
            default: break;
        }
        const uint32_t bits = (ex << 23) | frac;
        float a;
        std::memcpy(&a, &bits, 4);
        const SeqMap want = seq_append(m, bits, es);
        const SeqMap got = seq_append_abs(m, a, es, seq_ulp_scale(es));
        const bool w_over = want.d0 >= SEQ_K_LIMIT / 2 || want.d1 >= SEQ_K_LIMIT / 2;
        if (w_over) {
            // any increment of 2^23 or more ends the binade for every k >= 2^23
            if (got.d0 < SEQ_K_LIMIT / 2 || got.d1 < SEQ_K_LIMIT / 2) ++bad;
        } else if (got.d0 != want.d0 || got.d1 != want.d1) {
            ++bad;
        }
    }
    return bad;
}

// The transposed storage of a window's maps against the runs the window-end kernel gives its
// threads: thread t's i-th block must lie at slot i * 1024 + t of its stretch, no two blocks may
// share a slot, and no slot may lie beyond the window rounded up to a stretch.  Returns the
// number of violations.
extern "C" uint64_t seqsum_check_map_slots(uint32_t win) {
    uint64_t bad = 0;
    const uint32_t stretch = SEQ_SCAN_THREADS * SEQ_SCAN_RUN;
    std::vector<uint8_t> taken((size_t)((win + stretch - 1) / stretch) * stretch, 0);
    auto claim = [&](uint32_t block, uint32_t expect) {
        const uint32_t slot = seq_map_slot(block, win);
        if (slot != expect || slot >= taken.size() || taken[slot]) ++bad;
        if (slot < taken.size()) taken[slot] = 1;
    };
    uint32_t seen = 0;
    if (win <= stretch) {
        const uint32_t chunk = (win + SEQ_SCAN_THREADS - 1) / SEQ_SCAN_THREADS;
        for (uint32_t t = 0; t < SEQ_SCAN_THREADS; ++t) {
            const uint32_t lo = t * chunk, hi = lo + chunk < win ? lo + chunk : win;
            for (uint32_t b = lo; b < hi; ++b, ++seen) claim(b, (b - lo) * SEQ_SCAN_THREADS + t);
        }
    } else {
        for (uint32_t from = 0; from < win; from += stretch) {
            const uint32_t to = win - from > stretch ? from + stretch : win;
            for (uint32_t t = 0; t < SEQ_SCAN_THREADS; ++t) {
                uint32_t lo = from + t * SEQ_SCAN_RUN;
                lo = lo < to ? lo : to;
                const uint32_t hi = lo + SEQ_SCAN_RUN < to ? lo + SEQ_SCAN_RUN : to;
                for (uint32_t b = lo; b < hi; ++b, ++seen) claim(b, from + (b - lo) * SEQ_SCAN_THREADS + t);
            }
        }
    }
    if (seen != win) ++bad;
    return bad;
}

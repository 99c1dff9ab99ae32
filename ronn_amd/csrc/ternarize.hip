// Weight/activation ternarisation: threshold and scale sums, 2-bit packing,
// dequantisation, expansion to int8 and the device-internal weight tiling.
//
// Reference: BitNetQuantizer::quantize_ternary (quantization.rs:67-109),
// pack_ternary_bits (:131-153), dequantize_ternary (:182-207),
// TernaryTensor::get_value (:275-291) in crates/ronn-providers/src/bitnet/.
#include <cmath>
#include <cstring>
#include <type_traits>

#include "common.hpp"
#include "seqsum_core.h"

namespace {

// NT: a non-temporal load, which keeps a streamed tensor from being allocated in the caches on
// its way in.  It pays when the tensor is larger than the last-level cache (8192 x 28672 f32,
// two tree passes: 0.41 -> 0.39 ms); a smaller one is still there for the second pass, and
// the windows of the exact sequential sums re-read what they have just read.
template <bool NT>
__device__ __forceinline__ float4 ld_stream(const float4 *p) {
    if constexpr (NT) {
        typedef float v4f __attribute__((ext_vector_type(4)));
        const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
        return make_float4(v.x, v.y, v.z, v.w);
    } else {
        return *p;
    }
}
constexpr uint64_t kStreamBytes = 192ull << 20;  // tensors above this size are read non-temporally

constexpr int kBlock = 256;
constexpr int kSeqTile = 4096;  // elements per block map of the sequential sum (256 x 16)
static_assert(kSeqTile == (int)SEQ_BLOCK_ELEMS, "the window policy counts elements per block");

__device__ __forceinline__ uint32_t ternary_code(float v, float threshold) {
    // quantization.rs:138-144.  NaN fails both comparisons and packs as 00 (-1).
    return fabsf(v) <= threshold ? 1u : (v > 0.0f ? 2u : 0u);
}

// ---------------------------------------------------------------------------
// pack_ternary_bits.  One thread per group of four consecutive elements makes one
// byte; four neighbouring lanes merge their bytes into the little-endian u32 that
// lane%4==0 stores.  A block covers 4096 elements in four strided passes so that
// every load instruction of a wave reads 1 KiB of consecutive floats.
// `survivors` (optional) receives the number of elements with |x| > threshold.
// ---------------------------------------------------------------------------
template <bool NT>
__global__ __launch_bounds__(kBlock) void pack_ternary_kernel(
    const float *__restrict__ x, uint64_t n, float threshold_arg, const float *__restrict__ threshold_ptr,
    uint32_t *__restrict__ packed, uint64_t n_tiles, unsigned long long *__restrict__ survivors,
    double *__restrict__ psum) {
    // (the tree-sum quantiser queues this pass behind its sum: the threshold then comes from the device)
    const float threshold = threshold_ptr ? *threshold_ptr : threshold_arg;
    __shared__ unsigned s_cnt[kBlock / 64];
    __shared__ double s_sum[kBlock / 64];
    double acc = 0.0;  // sum of the survivors' |x| (tree mode: one partial per workgroup)
    const uint64_t n_quads = (n + 3) / 4;
    const uint64_t n_words = (n + 15) / 16;
    unsigned count = 0;
    for (uint64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const uint64_t tile_quad0 = tile * (kBlock * 4);
        float4 v[4];
        bool full[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint64_t q = tile_quad0 + (uint64_t)j * kBlock + threadIdx.x;
            full[j] = (q * 4 + 3) < n;
            v[j] = full[j] ? ld_stream<NT>(reinterpret_cast<const float4 *>(x) + q)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint64_t q = tile_quad0 + (uint64_t)j * kBlock + threadIdx.x;
            uint32_t byte = 0;
            if (full[j]) {
                float e[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    byte |= ternary_code(e[i], threshold) << (2 * i);
                    const bool keep = fabsf(e[i]) > threshold;
                    count += keep ? 1u : 0u;
                    if (psum) acc += keep ? (double)fabsf(e[i]) : 0.0;
                }
            } else if (q < n_quads) {  // the single partial group at the tail
                for (int i = 0; i < 4; ++i) {
                    uint64_t idx = q * 4 + i;
                    if (idx < n) {
                        float e = x[idx];
                        byte |= ternary_code(e, threshold) << (2 * i);
                        const bool keep = fabsf(e) > threshold;
                        count += keep ? 1u : 0u;
                        if (psum) acc += keep ? (double)fabsf(e) : 0.0;
                    }
                }
            }
            uint32_t word = byte << (8 * (threadIdx.x & 3));
            word |= __shfl_xor(word, 1);
            word |= __shfl_xor(word, 2);
            if ((threadIdx.x & 3) == 0 && (q >> 2) < n_words) packed[q >> 2] = word;
        }
    }
    if (survivors) {
        // wave sum, block sum, then ONE atomic per workgroup (integer: order does not
        // matter; thousands of atomics on one address would serialise in L2)
        for (int off = 32; off > 0; off >>= 1) count += __shfl_down(count, off);
        if ((threadIdx.x & 63) == 0) s_cnt[threadIdx.x >> 6] = count;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long t = 0;
            for (int w = 0; w < kBlock / 64; ++w) t += s_cnt[w];
            if (t) atomicAdd(survivors, t);
        }
    }
    if (psum) {
        // fixed order: lanes by shuffles, waves in turn, workgroups by the final kernel
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off);
        if ((threadIdx.x & 63) == 0) s_sum[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            double t = 0.0;
            for (int w = 0; w < kBlock / 64; ++w) t += s_sum[w];
            psum[blockIdx.x] = t;
        }
    }
}

// Sum of the per-workgroup partials of the kernel above, in a fixed order.
__global__ __launch_bounds__(kBlock) void sum_partials_kernel(const double *__restrict__ psum,
                                                             int nparts, float *__restrict__ out) {
    __shared__ double s_sum[kBlock];
    double acc = 0.0;
    for (int i0 = 0; i0 < nparts; i0 += 8 * kBlock) {  // eight loads in flight per thread
        double v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = i0 + j * kBlock + (int)threadIdx.x;
            v[j] = psum[i < nparts ? i : nparts - 1];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += (i0 + j * kBlock + (int)threadIdx.x) < nparts ? v[j] : 0.0;
    }
    s_sum[threadIdx.x] = acc;
    __syncthreads();
    for (int off = kBlock / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) s_sum[threadIdx.x] += s_sum[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = (float)s_sum[0];
}

// ---------------------------------------------------------------------------
// Tree mode: deterministic f64 sum of |x| (optionally masked) and survivor count.
// ---------------------------------------------------------------------------
template <bool NT>
__global__ __launch_bounds__(kBlock) void abs_sum_tree_partial_kernel(
    const float *__restrict__ x, uint64_t n, int use_mask, float thr, double *__restrict__ psum,
    unsigned long long *__restrict__ pcnt) {
    __shared__ double s_sum[kBlock];
    __shared__ unsigned long long s_cnt[kBlock];
    double acc = 0.0;
    unsigned long long cnt = 0;
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    const uint64_t tid = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    auto add = [&](float v) {
        const float a = fabsf(v);
        const bool take = use_mask ? (a > thr) : true;
        acc += take ? (double)a : 0.0;
        cnt += take ? 1u : 0u;
    };
    // 16-byte loads, four in flight per thread; a scalar loop for what is left (or for an
    // unaligned tensor).  The order of the additions is fixed by the grid, hence deterministic.
    uint64_t done = 0;
    if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        const uint64_t n4 = n / 4;
        uint64_t i = tid;
        for (; i + 3 * stride < n4; i += 4 * stride) {
            const float4 a = ld_stream<NT>(x4 + i), b = ld_stream<NT>(x4 + i + stride),
                         c = ld_stream<NT>(x4 + i + 2 * stride), d = ld_stream<NT>(x4 + i + 3 * stride);
            add(a.x), add(a.y), add(a.z), add(a.w);
            add(b.x), add(b.y), add(b.z), add(b.w);
            add(c.x), add(c.y), add(c.z), add(c.w);
            add(d.x), add(d.y), add(d.z), add(d.w);
        }
        for (; i < n4; i += stride) {
            const float4 a = x4[i];
            add(a.x), add(a.y), add(a.z), add(a.w);
        }
        done = n4 * 4;
    }
    for (uint64_t i = done + tid; i < n; i += stride) add(x[i]);
    s_sum[threadIdx.x] = acc;
    s_cnt[threadIdx.x] = cnt;
    __syncthreads();
    for (int off = kBlock / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + off];
            s_cnt[threadIdx.x] += s_cnt[threadIdx.x + off];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        psum[blockIdx.x] = s_sum[0];
        pcnt[blockIdx.x] = s_cnt[0];
    }
}

__global__ __launch_bounds__(kBlock) void abs_sum_tree_final_kernel(
    const double *__restrict__ psum, const unsigned long long *__restrict__ pcnt, int nparts,
    float *__restrict__ out_sum, unsigned long long *__restrict__ out_cnt,
    uint64_t n = 0, float *__restrict__ out_threshold = nullptr /* (sum / n) * 0.7, quantization.rs:79 */,
    unsigned long long *__restrict__ clear = nullptr /* the packing pass's survivor counter */) {
    __shared__ double s_sum[kBlock];
    __shared__ unsigned long long s_cnt[kBlock];
    double acc = 0.0;
    unsigned long long cnt = 0;
    for (int i = threadIdx.x; i < nparts; i += kBlock) {
        acc += psum[i];
        cnt += pcnt[i];
    }
    s_sum[threadIdx.x] = acc;
    s_cnt[threadIdx.x] = cnt;
    __syncthreads();
    for (int off = kBlock / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + off];
            s_cnt[threadIdx.x] += s_cnt[threadIdx.x + off];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float sum = (float)s_sum[0];
        *out_sum = sum;
        *out_cnt = s_cnt[0];
        if (out_threshold) {
            const float mean = sum / (float)n;
            *out_threshold = mean * 0.7f;
        }
        if (clear) *clear = 0ull;
    }
}

// ---------------------------------------------------------------------------
// Strict mode: the kernels of the exact sequential sum (see seqsum_core.h).
// ---------------------------------------------------------------------------
// The state of a sum lives in device memory and drives the kernels themselves, so that several
// windows can be queued without the host in between; the kernel that ends a window mirrors it
// into pinned host memory.
struct SeqState {
    uint32_t s_bits;    // current sum S as f32 bits (S >= 0)
    uint32_t win;       // blocks in the window that starts at `pos`
    uint64_t pos;       // blocks already folded into S
    uint32_t done;      // all blocks folded, or S no longer finite: queued kernels just return
    uint32_t error;     // a window made no progress (internal error)
    uint32_t saw_nan;   // set by any_nan_kernel
    uint32_t multi;     // the window carries two maps per block (seq_plan_window)
    uint64_t fresh_from;  // blocks from here on have not been seen by any window yet
    uint32_t rate_lo;   // multi: the cautious growth of S per block (f32 bits) behind the blocks' exponents
    uint32_t thr_bits;  // a sum queued behind another one: its mask threshold (f32 bits), set on the device
    uint64_t survivors;  // packing sums only: elements above the threshold, set by the window that ends the sum
    uint32_t windows;   // windows folded so far (the host sizes the next sum's first batch by it)
    uint32_t pad;
};

// A SeqMap from another lane by a DPP move: lanes without a source (and rows outside the
// mask) read zeros, which is the identity map.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ SeqMap seq_dpp(SeqMap m) {
    SeqMap o;
    o.d0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m.d0, CTRL, ROWMASK, 0xf, true);
    o.d1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m.d1, CTRL, ROWMASK, 0xf, true);
    return o;
}

// One SeqMap per block of 4096 elements, valid for a state of biased exponent `es` - or, in a
// window that spans several binades (state->multi), two per block: for the exponents e and e + 1,
// e = seq_multi_es_lo(block), stored side by side (maps[2 * block], maps[2 * block + 1]).
// The window and the exponent come from the state; the grid strides over the window's blocks.
// With `packed` given (masked sums only: thr is the ternary threshold) the kernel also packs
// every block that no earlier window has touched - a thread's 16 elements are one 32-bit word
// of the reference's layout - and adds their survivors to this workgroup's counter: the
// scale's sum and the packing then share one pass over the tensor.
// MASK and PACK are compile-time copies of use_mask and packed != nullptr: the body is the same,
// without the run-time selects per element.
template <bool MULTI, bool MASK, bool PACK>
__device__ __forceinline__ void seq_block_maps_body(
    const float *__restrict__ x, uint64_t n, float thr,
    const SeqState &st, SeqMap *__restrict__ maps, uint32_t *__restrict__ packed,
    unsigned long long *__restrict__ count_parts, SeqMap *s_wave, unsigned *s_cnt) {
    const uint32_t win = st.win;
    const uint64_t fresh_from = st.fresh_from, pos = st.pos;
    unsigned fresh_count = 0;
    const uint64_t first = st.pos * kSeqTile;
    const uint32_t s_bits = st.s_bits, rate_lo = st.rate_lo;
    uint32_t es0, k_unused;
    seq_state_split(s_bits, &es0, &k_unused);
  for (uint32_t blk = blockIdx.x; blk < win; blk += gridDim.x) {
    const uint32_t es = MULTI ? seq_multi_es_lo(s_bits, rate_lo, blk) : es0;
    const float scale = seq_ulp_scale(es < 26u ? 26u : es);
    const float scale_b = seq_ulp_scale(es + 1u < 26u ? 26u : es + 1u);
    uint64_t base = first + (uint64_t)blk * kSeqTile + (uint64_t)threadIdx.x * 16;
    bool fresh = PACK && pos + blk >= fresh_from;
    constexpr int NW = kBlock / 64;
    // ---- whole blocks first try the streaming form ---------------------------------------------
    // Unless one of its 4096 terms is an exact tie, a block's map is the saturated sum of all its
    // roundings, however the elements are dealt to the threads (seqsum_core.h).  So the loads are
    // the coalesced ones of a copy - thread t takes the float4s t, t + 256, t + 512, t + 768 of the
    // block, non-temporally: every cache line is fetched by one instruction and read once - the
    // wave adds its sums up by DPP, and only a block that does hold a tie (or an exponent below 26,
    // where terms are split in integer arithmetic) is done again in order, below.  Packing does not
    // depend on the order of the sums: four neighbouring lanes hold the four bytes of a word.
    const uint64_t blk_first = first + (uint64_t)blk * kSeqTile;
    bool in_order = blk_first + kSeqTile > n || es < 26u;  // (the same for the whole workgroup)
    if (!in_order) {
        const float4 *x4 = reinterpret_cast<const float4 *>(x + blk_first);
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = ld_stream<true>(x4 + j * kBlock + threadIdx.x);
        // (all four loads go out before the first value is touched: short of registers, the compiler
        // had put the first load's wait and use between the first and the second load)
        __builtin_amdgcn_sched_barrier(0);
        float am[16];
        uint32_t bytes[4] = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float e[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float a = fabsf(e[i]);
                const bool take = MASK ? (a > thr) : true;
                am[4 * j + i] = take ? a : 0.0f;
                if (fresh) {
                    bytes[j] |= ternary_code(e[i], thr) << (2 * i);
                    fresh_count += take ? 1u : 0u;
                }
            }
        }
        if (fresh) {
            const int lane = threadIdx.x & 63;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int w = (int)(bytes[j] << (8 * (lane & 3)));
                w |= __builtin_amdgcn_update_dpp(0, w, 0xB1, 0xf, 0xf, true);  // quad_perm:[1,0,3,2]
                w |= __builtin_amdgcn_update_dpp(0, w, 0x4E, 0xf, 0xf, true);  // quad_perm:[2,3,0,1]
                // (non-temporal: the words are not read again here, and fewer dirty lines are left to the
                // launch's end - 6 us of the packing sum at 235 M elements)
                if ((lane & 3) == 0)
                    __builtin_nontemporal_store((uint32_t)w, &packed[(blk_first >> 4) + j * (kBlock / 4) + (threadIdx.x >> 2)]);
            }
            fresh = false;  // (a second pass over this block packs nothing)
        }
        bool tie_a = false, tie_b = false;
        uint32_t sum_a = seq_min_u32(seq_sum16(am, es, scale, &tie_a), SEQ_SAT), sum_b = 0;
        if (MULTI) sum_b = seq_min_u32(seq_sum16(am, es + 1u, scale_b, &tie_b), SEQ_SAT);
        auto wave_add = [](uint32_t u) {  // <= 2^25 per lane: a wave's total stays at or below 2^31
            int sum = (int)u;
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x111, 0xf, 0xf, true);  // row_shr:1
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x112, 0xf, 0xf, true);  // row_shr:2
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x114, 0xf, 0xf, true);  // row_shr:4
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x118, 0xf, 0xf, true);  // row_shr:8
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x142, 0xa, 0xf, true);  // row_bcast15
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x143, 0xc, 0xf, true);  // row_bcast31
            return seq_min_u32((uint32_t)sum, SEQ_SAT);  // lane 63 holds the wave's
        };
        sum_a = wave_add(sum_a);
        if (MULTI) sum_b = wave_add(sum_b);
        const bool wave_tie = __ballot(tie_a || tie_b) != 0ull;
        if ((threadIdx.x & 63) == 63) {
            SeqMap t;
            t.d0 = sum_a;
            t.d1 = sum_b | (wave_tie ? 0x80000000u : 0u);  // (sums stay below 2^26)
            s_wave[threadIdx.x >> 6] = t;
        }
        __syncthreads();
        uint32_t tot_a = 0, tot_b = 0, any_tie = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const SeqMap t = s_wave[w];
            tot_a += t.d0;
            tot_b += t.d1 & 0x7fffffffu;
            any_tie |= t.d1 & 0x80000000u;
        }
        in_order = any_tie != 0;
        if (!in_order && threadIdx.x == 0) {
            tot_a = seq_min_u32(tot_a, SEQ_SAT);
            tot_b = seq_min_u32(tot_b, SEQ_SAT);
            if (MULTI) {
                reinterpret_cast<uint4 *>(maps)[blk] = make_uint4(tot_a, tot_a, tot_b, tot_b);
            } else {
                SeqMap t;
                t.d0 = t.d1 = tot_a;
                maps[seq_map_slot(blk, win)] = t;
            }
        }
        __syncthreads();  // s_wave is rewritten by the next block, or below
        if (!in_order) continue;
    }
    // ---- in order: a thread's sixteen consecutive elements, the wave's maps composed left to right
    uint32_t word = 0;
    float am[16];  // |x| of the elements that count, +0.0 (the identity as a term) for the others
    if (base + 16 <= n) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = reinterpret_cast<const float4 *>(x + base)[j];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float e[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = fabsf(e[i]);
                bool take = MASK ? (a > thr) : true;
                am[4 * j + i] = take ? a : 0.0f;
                if (fresh) {
                    word |= ternary_code(e[i], thr) << (2 * (4 * j + i));
                    fresh_count += take ? 1u : 0u;
                }
            }
        }
        if (fresh) packed[base >> 4] = word;
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) am[i] = 0.0f;
        for (int i = 0; i < 16; ++i) {
            uint64_t idx = base + i;
            if (idx < n) {
                float e = x[idx];
                float a = fabsf(e);
                bool take = MASK ? (a > thr) : true;
                am[i] = take ? a : 0.0f;
                if (fresh) {
                    word |= ternary_code(e, thr) << (2 * i);
                    fresh_count += take ? 1u : 0u;
                }
            }
        }
        if (fresh && base < n) packed[base >> 4] = word;  // tail bits stay zero
    }
    SeqMap m = seq_map16(am, es, scale), mb = seq_identity();
    if (MULTI) mb = seq_map16(am, es + 1u, scale_b);
    // ordered reduction of the wave by DPP moves (each lane absorbs what lies to its left):
    // lane 63 ends up with the map of all 1024 elements
    // (maps that do not depend on the parity of k - all of them unless a term is an exact tie -
    // compose by adding their increments, in any order: one DPP add per step)
    auto wave_fold = [](SeqMap v) {
        if (__ballot(v.d0 != v.d1) == 0ull) {
            int sum = (int)v.d0;  // <= 2^25 per lane: a wave's total stays below 2^31
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x111, 0xf, 0xf, true);  // row_shr:1
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x112, 0xf, 0xf, true);  // row_shr:2
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x114, 0xf, 0xf, true);  // row_shr:4
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x118, 0xf, 0xf, true);  // row_shr:8
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x142, 0xa, 0xf, true);  // row_bcast15
            sum += __builtin_amdgcn_update_dpp(0, sum, 0x143, 0xc, 0xf, true);  // row_bcast31
            v.d0 = v.d1 = seq_min_u32((uint32_t)sum, SEQ_SAT);
            return v;
        }
        v = seq_compose(seq_dpp<0x111, 0xf>(v), v);  // row_shr:1
        v = seq_compose(seq_dpp<0x112, 0xf>(v), v);  // row_shr:2
        v = seq_compose(seq_dpp<0x114, 0xf>(v), v);  // row_shr:4
        v = seq_compose(seq_dpp<0x118, 0xf>(v), v);  // row_shr:8
        v = seq_compose(seq_dpp<0x142, 0xa>(v), v);  // row_bcast15
        v = seq_compose(seq_dpp<0x143, 0xc>(v), v);  // row_bcast31
        return v;
    };
    m = wave_fold(m);
    if (MULTI) mb = wave_fold(mb);
    if ((threadIdx.x & 63) == 63) {
        s_wave[threadIdx.x >> 6] = m;
        if (MULTI) s_wave[NW + (threadIdx.x >> 6)] = mb;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        SeqMap t = s_wave[0];
        for (int w = 1; w < NW; ++w) t = seq_compose(t, s_wave[w]);
        if (MULTI) {
            SeqMap u = s_wave[NW];
            for (int w = 1; w < NW; ++w) u = seq_compose(u, s_wave[NW + w]);
            reinterpret_cast<uint4 *>(maps)[blk] = make_uint4(t.d0, t.d1, u.d0, u.d1);
        } else {
            maps[seq_map_slot(blk, win)] = t;
        }
    }
    __syncthreads();  // s_wave is rewritten in the next turn
  }
    if (PACK) {
        // one plain read-modify-write per workgroup and launch: slot blockIdx.x belongs to
        // this workgroup alone, and launches are ordered by the stream
        for (int off = 32; off > 0; off >>= 1) fresh_count += __shfl_down(fresh_count, off);
        if ((threadIdx.x & 63) == 0) s_cnt[threadIdx.x >> 6] = fresh_count;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned t = 0;
            for (int w = 0; w < kBlock / 64; ++w) t += s_cnt[w];
            if (t) count_parts[blockIdx.x] += t;
        }
    }
}

// (seven waves per SIMD: left to itself the compiler takes 83 registers for the two forms of the body,
// five waves per SIMD, and the long windows lose what the streaming loads gain)
__global__ __launch_bounds__(kBlock, 7) void seq_block_maps_kernel(
    const float *__restrict__ x, uint64_t n, int use_mask, float thr_arg, int thr_from_state,
    const SeqState *__restrict__ state, SeqMap *__restrict__ maps, uint32_t *__restrict__ packed,
    unsigned long long *__restrict__ count_parts) {
    __shared__ SeqMap s_wave[2 * (kBlock / 64)];
    __shared__ unsigned s_cnt[kBlock / 64];
    // the whole state in one scalar round trip (asked for field by field, `done`, `multi` and the
    // window each cost a dependent one before the first load of data could go out)
    asm volatile("" : : "s"(x), "s"(n), "s"(use_mask), "s"(thr_arg), "s"(state), "s"(maps), "s"(packed),
                 "s"(count_parts));
    const SeqState st = *state;
    asm volatile("" : : "s"(st.s_bits), "s"(st.win), "s"(st.pos), "s"(st.done), "s"(st.multi), "s"(st.fresh_from),
                 "s"(st.rate_lo));
    if (st.done) return;
    const float thr = thr_from_state ? __uint_as_float(st.thr_bits) : thr_arg;
    // (in the ordered form plain loads also in long windows: a thread's four loads share their cache
    // lines, and non-temporal ones fetched each line four times)
    auto run = [&](auto multi) {
        constexpr bool M = decltype(multi)::value;
        if (packed != nullptr)  // packing goes with a masked sum (thr is the ternary threshold)
            seq_block_maps_body<M, true, true>(x, n, thr, st, maps, packed, count_parts, s_wave, s_cnt);
        else if (use_mask)
            seq_block_maps_body<M, true, false>(x, n, thr, st, maps, packed, count_parts, s_wave, s_cnt);
        else
            seq_block_maps_body<M, false, false>(x, n, thr, st, maps, packed, count_parts, s_wave, s_cnt);
    };
    if (st.multi)
        run(std::true_type{});
    else
        run(std::false_type{});
}

// The state before the first window (one launch instead of a fill and a copy from the host): S = +0,
// nothing folded, the first window `win0` blocks long; the per-workgroup survivor counters cleared.
__global__ __launch_bounds__(kBlock) void seq_init_kernel(SeqState *__restrict__ state, uint32_t win0,
                                                         unsigned long long *__restrict__ count_parts, int n_parts) {
    if (count_parts)
        for (int i = threadIdx.x; i < n_parts; i += kBlock) count_parts[i] = 0;
    if (threadIdx.x == 0) {
        SeqState z;
        z.s_bits = 0, z.win = win0, z.pos = 0, z.done = 0, z.error = 0, z.saw_nan = 0, z.multi = 0;
        z.fresh_from = 0, z.rate_lo = 0, z.thr_bits = 0, z.survivors = 0, z.windows = 0, z.pad = 0;
        *state = z;
    }
}

// The state of a sum that is queued behind another one without the host in between: the masked sum
// of the quantiser, whose threshold is (S / n) * 0.7 of the sum before it (quantization.rs:79).  If
// that sum is not complete when this kernel runs (its batch of windows was too short, or S left the
// finite range), the follower is marked done with error 2: its kernels return at once and the host
// runs it the ordinary way afterwards.
__global__ __launch_bounds__(kBlock) void seq_chain_init_kernel(const SeqState *__restrict__ prev,
                                                               SeqState *__restrict__ state, uint64_t n,
                                                               uint64_t total_blocks,
                                                               unsigned long long *__restrict__ count_parts,
                                                               int n_parts) {
    if (count_parts)
        for (int i = threadIdx.x; i < n_parts; i += kBlock) count_parts[i] = 0;
    if (threadIdx.x == 0) {
        const SeqState p = *prev;
        const bool complete = p.done && !p.error && p.pos >= total_blocks && ((p.s_bits >> 23) & 0xffu) != 0xffu;
        SeqState z;
        z.s_bits = 0, z.win = 1u, z.pos = 0, z.done = complete ? 0u : 1u, z.error = complete ? 0u : 2u;
        z.saw_nan = 0, z.multi = 0, z.fresh_from = 0, z.rate_lo = 0, z.survivors = 0, z.windows = 0, z.pad = 0;
        const float mean = __uint_as_float(p.s_bits) / (float)n;
        z.thr_bits = __float_as_uint(mean * 0.7f);
        *state = z;
    }
}

// Inclusive ordered scan of a wave's maps (lane l ends with the composition of lanes 0..l).  Maps that
// do not depend on the parity of k - all of them unless a term was an exact tie - are plain
// increments, and composing increments is adding them and saturating once at the end (the sum of 64
// saturated increments stays below 2^31): one DPP add per step instead of a composition of ten
// instructions.  The choice is made per wave, so all lanes take the same path.
__device__ __forceinline__ SeqMap seq_wave_inclusive(SeqMap m) {
    if (__ballot(m.d0 != m.d1) == 0ull) {
        int sum = (int)m.d0;
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x111, 0xf, 0xf, true);  // row_shr:1
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x112, 0xf, 0xf, true);  // row_shr:2
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x114, 0xf, 0xf, true);  // row_shr:4
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x118, 0xf, 0xf, true);  // row_shr:8
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x142, 0xa, 0xf, true);  // row_bcast15: rows 1, 3 absorb the row before
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x143, 0xc, 0xf, true);  // row_bcast31: rows 2, 3 absorb rows 0-1
        m.d0 = m.d1 = seq_min_u32((uint32_t)sum, SEQ_SAT);
        return m;
    }
    m = seq_compose(seq_dpp<0x111, 0xf>(m), m);  // row_shr:1
    m = seq_compose(seq_dpp<0x112, 0xf>(m), m);  // row_shr:2
    m = seq_compose(seq_dpp<0x114, 0xf>(m), m);  // row_shr:4
    m = seq_compose(seq_dpp<0x118, 0xf>(m), m);  // row_shr:8
    m = seq_compose(seq_dpp<0x142, 0xa>(m), m);  // row_bcast15
    m = seq_compose(seq_dpp<0x143, 0xc>(m), m);  // row_bcast31
    return m;
}

// Ordered scans of SeqMaps without a barrier per step: inside a wave by shuffles (lane l
// absorbs what lies to its left), across the waves through one LDS slot per wave.  Returns the
// composition of everything BEFORE this thread, and in *total the composition of all; NW = waves
// that carry values (the others pass the identity).  One __syncthreads inside: every thread of
// the workgroup must call it, and s_w must not be touched again before the next barrier.
template <int NW>
__device__ __forceinline__ SeqMap seq_block_before(SeqMap m, SeqMap *s_w, SeqMap *total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // inclusive scan of the wave: inside rows of 16 lanes, then across the rows
    m = seq_wave_inclusive(m);
    if (lane == 63 && wave < NW) s_w[wave] = m;
    const SeqMap ex = seq_dpp<0x138, 0xf>(m);  // wave_shr:1: exclusive inside the wave, lane 0 reads the identity
    __syncthreads();
    // the waves' totals, one per lane of the first row, scanned the same way (four steps instead
    // of a chain of NW compositions); lane w - 1 then holds everything before wave w
    static_assert(NW <= 16, "the waves' totals must fit one row of lanes");
    SeqMap v = seq_identity();
    if (lane < NW) v = s_w[lane];
    if (__ballot(v.d0 != v.d1) == 0ull) {  // plain increments (see seq_wave_inclusive): at most 16 x 2^25
        int sum = (int)v.d0;
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x111, 0xf, 0xf, true);  // row_shr:1
        sum += __builtin_amdgcn_update_dpp(0, sum, 0x112, 0xf, 0xf, true);  // row_shr:2
        if (NW > 4) sum += __builtin_amdgcn_update_dpp(0, sum, 0x114, 0xf, 0xf, true);  // row_shr:4
        if (NW > 8) sum += __builtin_amdgcn_update_dpp(0, sum, 0x118, 0xf, 0xf, true);  // row_shr:8
        v.d0 = v.d1 = seq_min_u32((uint32_t)sum, SEQ_SAT);
    } else {
        v = seq_compose(seq_dpp<0x111, 0xf>(v), v);  // row_shr:1
        v = seq_compose(seq_dpp<0x112, 0xf>(v), v);  // row_shr:2
        if (NW > 4) v = seq_compose(seq_dpp<0x114, 0xf>(v), v);  // row_shr:4
        if (NW > 8) v = seq_compose(seq_dpp<0x118, 0xf>(v), v);  // row_shr:8
    }
    const int w_uni = __builtin_amdgcn_readfirstlane(wave);
    SeqMap pre = seq_identity(), tot;
    tot.d0 = (uint32_t)__builtin_amdgcn_readlane((int)v.d0, NW - 1);
    tot.d1 = (uint32_t)__builtin_amdgcn_readlane((int)v.d1, NW - 1);
    if (w_uni > 0) {
        pre.d0 = (uint32_t)__builtin_amdgcn_readlane((int)v.d0, w_uni - 1);
        pre.d1 = (uint32_t)__builtin_amdgcn_readlane((int)v.d1, w_uni - 1);
    }
    *total = tot;
    return seq_compose(pre, ex);
}

// Resolves one block of 4096 elements from the state (es, k_cur) that enters it, called by all
// 1024 threads of the window-end kernel.  The block's 256 chunks of 16 elements are mapped
// (threads 0..255, one chunk each) and scanned from the entering state; the one chunk in which
// k reaches 2^24 is replayed with ordinary f32 additions, which moves S into a new binade; the
// chunks after it are mapped again for that binade, and so on to the end of the block.  Early
// blocks cross several binades (S doubles every few elements at first), later ones at most one.
// Only the first four waves work: the other twelve share their SIMDs, and every instruction
// they issue delays the four (a turn of the loop took 5,300 cycles with all sixteen running the
// same code), so they only keep the barriers and read the loop's conditions from LDS.
// Returns the state after the block as f32 bits (possibly +Inf or NaN) - in the first four waves;
// the same value is left in *s_bits_now for the others, who read it behind a barrier of the
// caller's.  s_w, s_first and s_bits_now are LDS scratch; the caller puts a barrier before it
// touches them again.
__device__ __forceinline__ uint32_t seq_replay_block(const float *__restrict__ x, uint64_t n, uint64_t block_base,
                                                     int use_mask, float thr, uint32_t es, uint32_t k_cur,
                                                     SeqMap *s_w, unsigned *s_first, uint32_t *s_bits_now,
                                                     float *s_head /* 512 floats */,
                                                     uint32_t *s_cross /* [0]: S behind the block's last crossing
                                                                          chunk, [1]: chunks folded up to there */,
                                                     uint32_t *__restrict__ packed = nullptr /* pack this block too */,
                                                     unsigned *s_survivors = nullptr /* LDS, zeroed: += its survivors */) {
    const uint32_t t = threadIdx.x;
    constexpr int NW = kBlock / 64;
    const bool worker = __builtin_amdgcn_readfirstlane((int)(t >> 6)) < NW;  // wave-uniform
    // A sum that starts at zero doubles every few elements: crossed binade by binade, the first
    // 512 elements cost nine turns of the loop below.  They are added one after the other instead
    // (that IS the fold, so it is exact whatever the state; 2 us for the 512 additions).
    const bool head = es == 1u && k_cur == 0u;
    if (!worker) {
        // the barriers of the worker waves, in the same order, and their exits
        if (head) {
            __syncthreads();  // (h1) head elements in LDS
            __syncthreads();  // (h2) head folded
            if (((*s_bits_now >> 23) & 0xffu) == 0xffu) {
                __syncthreads();  // (h3) NaN behind an Inf
                return 0u;
            }
        }
        for (int guard = 0; guard <= kBlock; ++guard) {
            __syncthreads();  // (1) wave totals written
            __syncthreads();  // (2) crossing chunk known
            const uint32_t tstar = *s_first;
            if (tstar == 0xffffffffu) break;
            __syncthreads();  // (3) chunk replayed
            const uint32_t bits = *s_bits_now;
            if (((bits >> 23) & 0xffu) == 0xffu) {
                __syncthreads();  // (4) NaN behind an Inf
                break;
            }
            if (tstar + 1u >= (uint32_t)kBlock) break;
        }
        return 0u;
    }
    const uint64_t base = block_base + (uint64_t)t * 16;
    float a[16];
    uint32_t word = 0;  // the thread's sixteen elements as one packed word (only when packing)
    if (base + 16 <= n && (reinterpret_cast<uintptr_t>(x + base) & 15u) == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 v = reinterpret_cast<const float4 *>(x + base)[j];
            a[4 * j] = fabsf(v.x), a[4 * j + 1] = fabsf(v.y), a[4 * j + 2] = fabsf(v.z), a[4 * j + 3] = fabsf(v.w);
            if (packed)
                word |= (ternary_code(v.x, thr) | ternary_code(v.y, thr) << 2 | ternary_code(v.z, thr) << 4 |
                         ternary_code(v.w, thr) << 6) << (8 * j);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) a[i] = 0.0f;
        for (int i = 0; i < 16; ++i) {
            const uint64_t idx = base + i;
            if (idx < n) {
                const float v = x[idx];
                a[i] = fabsf(v);
                if (packed) word |= ternary_code(v, thr) << (2 * i);
            }
        }
    }
    if (packed) {
        if (base < n) packed[base >> 4] = word;  // tail bits stay zero
        unsigned mine = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) mine += a[i] > thr ? 1u : 0u;  // (elements past the end are +0.0; a NaN is no survivor)
        if (mine) atomicAdd(s_survivors, mine);
    }
    // a skipped element adds +0.0, which leaves any S >= 0 (and NaN/Inf) unchanged, and as a
    // term of a map it is the identity
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = (!use_mask || a[i] > thr) ? a[i] : 0.0f;
    const int lane = t & 63, wave = t >> 6;
    uint32_t done = 0;  // chunks [0, done) are already folded into (es, k_cur)
    uint32_t result_bits = 0;
    uint32_t cross_bits = seq_state_join(es, k_cur), cross_done = 0;  // the last crossing so far: none
    if (head) {
        constexpr uint32_t kHeadChunks = 32;
        if (t < kHeadChunks) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s_head[t * 16 + i] = a[i];
        }
        __syncthreads();  // (h1)
        if (t == 0) {
            float sum = __uint_as_float(seq_state_join(es, k_cur));
            for (uint32_t i = 0; i < kHeadChunks * 16; i += 4) {
                const float4 v = *reinterpret_cast<const float4 *>(s_head + i);
                sum = sum + v.x;
                sum = sum + v.y;
                sum = sum + v.z;
                sum = sum + v.w;
            }
            *s_bits_now = __float_as_uint(sum);
        }
        __syncthreads();  // (h2)
        result_bits = *s_bits_now;
        done = kHeadChunks;
        if (((result_bits >> 23) & 0xffu) == 0xffu) {
            // as below: +Inf turns into NaN if a NaN follows inside this block
            bool nan_after = false;
            if (t >= done) {
#pragma unroll
                for (int i = 0; i < 16; ++i) nan_after |= (a[i] != a[i]);
            }
            if (nan_after) atomicOr(s_bits_now, 0x7fc00000u);
            __syncthreads();  // (h3)
            return *s_bits_now;  // (already in LDS for the other waves)
        }
        seq_state_split(result_bits, &es, &k_cur);
        cross_bits = result_bits, cross_done = done;
    }
    for (int guard = 0; guard <= kBlock; ++guard) {
        SeqMap m = seq_identity();
        if (t >= done) m = seq_map16(a, es, seq_ulp_scale(es < 26u ? 26u : es));
        if (t == 0) *s_first = 0xffffffffu;
        // inclusive scan of the wave, the waves' totals through LDS
        const SeqMap inc = seq_wave_inclusive(m);
        if (lane == 63) s_w[wave] = inc;
        const SeqMap ex = seq_dpp<0x138, 0xf>(inc);  // wave_shr:1: exclusive inside the wave
        __syncthreads();  // (1)
        SeqMap pre = seq_identity(), all = seq_identity();
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const SeqMap sw = s_w[w];
            if (w < wave) pre = seq_compose(pre, sw);
            all = seq_compose(all, sw);
        }
        const SeqMap before = seq_compose(pre, ex);
        const uint32_t k = seq_apply(before, k_cur);
        const bool crosses = t >= done && k < SEQ_K_LIMIT && seq_apply(m, k) >= SEQ_K_LIMIT;
        if (crosses) atomicMin(s_first, t);
        const uint32_t k_end = seq_apply(all, k_cur);  // state after the block if no crossing
        __syncthreads();  // (2)
        const uint32_t tstar = *s_first;
        if (tstar == 0xffffffffu) {
            result_bits = seq_state_join(es, k_end);
            break;
        }
        if (t == tstar) {
            float sum = __uint_as_float(seq_state_join(es, k));
#pragma unroll
            for (int i = 0; i < 16; ++i) sum = sum + a[i];
            *s_bits_now = __float_as_uint(sum);
        }
        __syncthreads();  // (3)
        result_bits = *s_bits_now;
        done = tstar + 1;
        cross_bits = result_bits, cross_done = done;
        if (((result_bits >> 23) & 0xffu) == 0xffu) {
            // S is +Inf or NaN.  +Inf turns into NaN if a NaN follows inside this block.
            bool nan_after = false;
            if (t >= done) {
#pragma unroll
                for (int i = 0; i < 16; ++i) nan_after |= (a[i] != a[i]);
            }
            if (nan_after) atomicOr(s_bits_now, 0x7fc00000u);  // Inf | quiet bit = NaN
            __syncthreads();  // (4)
            result_bits = *s_bits_now;
            break;
        }
        if (done >= (uint32_t)kBlock) break;
        seq_state_split(result_bits, &es, &k_cur);
        // (no barrier here: s_first was last read before barrier (3), s_w before (2), and
        // s_bits_now is written again only behind the next turn's barrier (2))
    }
    // For the waves that only kept the barriers the result is left in LDS (the caller puts a
    // barrier before reading it).  The store cannot overtake a read: with no crossing in this turn
    // nobody has read s_bits_now since the last turn's barrier (3), two barriers ago; on the other
    // exits it holds this very value already.
    if (t == 0) {
        *s_bits_now = result_bits;
        s_cross[0] = cross_bits, s_cross[1] = cross_done;  // (read by thread 0 only, or behind the caller's barrier)
    }
    return result_bits;
}

// The usual case of a crossing block, resolved with two barriers instead of five: S leaves its binade
// once inside the block and ends one binade up.  The four working waves map their quarter of the
// block for BOTH exponents at once (a map does not depend on the state, only on the exponent), so
// that after one exchange of the quarters' maps the wave that holds the crossing can finish alone:
// it finds the crossing chunk among its lanes, lets that lane add its sixteen terms, composes the
// maps of its remaining lanes for the new exponent and walks through the quarters behind it.
// Returns false (the same in every thread, nothing but LDS scratch touched) when the block is not
// of that kind - a second crossing, a jump over a binade, an overflow: seq_replay_block then does
// it in general.  Results as there: *s_bits_now, s_cross[0..1], valid after the last barrier inside.
__device__ __forceinline__ bool seq_replay_block_once(const float *__restrict__ x, uint64_t n, uint64_t block_base,
                                                      int use_mask, float thr, uint32_t es, uint32_t k_cur,
                                                      SeqMap *s_w /* 8 slots */, uint32_t *s_bits_now,
                                                      uint32_t *s_cross, unsigned *s_ok) {
    if (es < 26u || es + 1u > 253u) return false;  // (uniform: below 26 terms are split in integer arithmetic)
    const uint32_t t = threadIdx.x;
    constexpr int NW = kBlock / 64;
    const int wave = __builtin_amdgcn_readfirstlane((int)(t >> 6));
    if (wave >= NW) {
        __syncthreads();  // (A) the quarters' maps
        __syncthreads();  // (B) the result
        return *s_ok != 0u;
    }
    const uint64_t base = block_base + (uint64_t)t * 16;
    float a[16];
    if (base + 16 <= n && (reinterpret_cast<uintptr_t>(x + base) & 15u) == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 v = reinterpret_cast<const float4 *>(x + base)[j];
            a[4 * j] = fabsf(v.x), a[4 * j + 1] = fabsf(v.y), a[4 * j + 2] = fabsf(v.z), a[4 * j + 3] = fabsf(v.w);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) a[i] = 0.0f;
        for (int i = 0; i < 16; ++i) {
            const uint64_t idx = base + i;
            if (idx < n) a[i] = fabsf(x[idx]);
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) a[i] = (!use_mask || a[i] > thr) ? a[i] : 0.0f;
    const SeqMap m0 = seq_map16(a, es, seq_ulp_scale(es));
    const SeqMap m1 = seq_map16(a, es + 1u, seq_ulp_scale(es + 1u));
    const SeqMap inc0 = seq_wave_inclusive(m0);
    const int lane = t & 63;
    // the quarter's map for the new exponent: lane 63 of the scan of all its lanes
    const SeqMap inc1 = seq_wave_inclusive(m1);
    if (lane == 63) {
        s_w[wave] = inc0;
        s_w[NW + wave] = inc1;
    }
    if (t == 0) *s_ok = 0u;
    __syncthreads();  // (A)
    // the quarter in which k reaches 2^24, and the k that enters it (the same in every thread)
    int q = -1;
    uint32_t kq = k_cur, k = k_cur;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const uint32_t k2 = seq_apply(s_w[w], k);
        if (q < 0 && k2 >= SEQ_K_LIMIT) q = w, kq = k;
        if (q < 0) k = k2;
    }
    if (wave == q) {
        const SeqMap ex0 = seq_dpp<0x138, 0xf>(inc0);  // wave_shr:1: what lies before the lane, lane 0 the identity
        const uint32_t kl = seq_apply(ex0, kq);
        const bool crosses = kl < SEQ_K_LIMIT && seq_apply(m0, kl) >= SEQ_K_LIMIT;
        const unsigned long long where = __ballot(crosses);
        bool ok = where != 0ull;
        const int tstar = ok ? __builtin_ctzll(where) : 0;
        // the crossing chunk, replayed by its lane with ordinary f32 additions
        float sum = __uint_as_float(seq_state_join(es, kl));
#pragma unroll
        for (int i = 0; i < 16; ++i) sum = sum + a[i];
        const uint32_t bits = (uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(sum), tstar);
        uint32_t es2, k2;
        seq_state_split(bits, &es2, &k2);
        ok = ok && ((bits >> 23) & 0xffu) != 0xffu && es2 == es + 1u;
        // the lanes behind it, for the new exponent
        SeqMap rest = lane > tstar ? m1 : seq_identity();
        rest = seq_wave_inclusive(rest);
        SeqMap tail;
        tail.d0 = (uint32_t)__builtin_amdgcn_readlane((int)rest.d0, 63);
        tail.d1 = (uint32_t)__builtin_amdgcn_readlane((int)rest.d1, 63);
        uint32_t k3 = seq_apply(tail, k2);
        ok = ok && k3 < SEQ_K_LIMIT;
        // and the quarters behind this one
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            if (w > q && ok) {
                k3 = seq_apply(s_w[NW + w], k3);
                ok = k3 < SEQ_K_LIMIT;
            }
        }
        if (lane == 0 && ok) {
            *s_bits_now = seq_state_join(es + 1u, k3);
            s_cross[0] = bits, s_cross[1] = (uint32_t)q * 64u + (uint32_t)tstar + 1u;
            *s_ok = 1u;
        }
    }
    __syncthreads();  // (B)
    return *s_ok != 0u;
}

// One workgroup of 1024 threads ends a window.
// (1) Scan: walks the block maps of the window from the true state and finds the first
//     block in which k reaches 2^24.
// (2) Replay: resolves that block.  Its 256 chunks of 16 elements are mapped (threads
//     0..255, one chunk each) and scanned from the state entering the block; the one chunk
//     in which k reaches 2^24 is replayed with ordinary f32 additions, which moves S into a
//     new binade; the chunks after it are mapped again for that binade, and so on to the
//     end of the block.  Early blocks cross several binades (S doubles every few elements
//     at first), later ones at most one.
// A window with two maps per block (state->multi) repeats (1) and (2): after the replay S is in a
// new binade, for which the blocks that follow carry their other map, and so on until the window
// ends or a block's pair does not hold the exponent S has.
// The new state goes to device memory (for the next window's kernels) and to the pinned
// host mailbox (the host reads it after synchronising: it sizes the next window).
__global__ __launch_bounds__(1024) void seq_scan_replay_kernel(
    const SeqMap *__restrict__ maps, const float *__restrict__ x, uint64_t n, uint64_t total_blocks,
    int use_mask, float thr_arg, int thr_from_state, SeqState *__restrict__ state, SeqState *__restrict__ host_copy,
    int mirror /* the last launch of a batch: the host reads the state after it */,
    unsigned long long *__restrict__ count_parts /* packing sums: the maps kernels' survivor counters */,
    int n_parts, uint32_t *__restrict__ packed /* packing sums: the packed words (the first block is packed here) */) {
    extern __shared__ uint4 s_maps[];  // SEQ_MULTI_LIMIT units: the maps of a window with two per block
    __shared__ SeqMap s_w[16];
    __shared__ unsigned s_first;
    __shared__ uint32_t s_cross_block, s_cross_k;
    __shared__ uint32_t s_bits_now;
    __shared__ unsigned long long s_min64;
    __shared__ uint32_t s_edge[64];
    __shared__ unsigned long long s_cnt64[16];
    __shared__ unsigned s_cnt0;
    __shared__ __attribute__((aligned(16))) float s_head[512];
    __shared__ uint32_t s_cross[2];
    __shared__ unsigned s_once;
    const uint32_t t = threadIdx.x;
    // Windows of up to 1024 blocks (most of them) have one map per thread: it is requested
    // here, before the state is known, so that the two round trips overlap (the buffer holds
    // at least 1024 maps).
    const SeqMap spec = maps[t];
    // the whole state in the same round trip (field by field, `done`, the window, `multi` and its
    // rate each cost a dependent one)
    const SeqState st0 = *state;
    // (all values are named here so that every load is issued before any is waited for)
    asm volatile("" : : "v"(spec.d0), "v"(spec.d1), "s"(st0.done), "s"(st0.win), "s"(st0.pos), "s"(st0.s_bits),
                 "s"(st0.multi), "s"(st0.rate_lo), "s"(st0.fresh_from));
    const uint32_t done0 = st0.done;
    if (done0) {
        if (mirror && t == 0) *host_copy = *state;
        return;
    }
    const float thr = thr_from_state ? __uint_as_float(st0.thr_bits) : thr_arg;
    const uint32_t nblocks = st0.win;
    const uint64_t pos0 = st0.pos;
    const uint64_t first = pos0 * kSeqTile;
    const uint32_t bits0 = st0.s_bits;
    uint32_t es, k0;
    seq_state_split(bits0, &es, &k0);
    // ends the window: the state after `advanced` blocks, the next window's size from the
    // growth of S over this one, mirrored to the host
    // The window that folds the last block also adds up the survivor counters of the packing pass
    // (all maps kernels have run by then): called by every thread with the same `advanced`, before
    // finish(); the total is valid in thread 0.
    unsigned long long survivors_total = 0;
    auto count_survivors = [&](uint32_t advanced) {
        if (count_parts == nullptr || pos0 + advanced < total_blocks) return;
        unsigned long long acc = 0;
        for (int i = (int)t; i < n_parts; i += 1024) acc += count_parts[i];
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off);
        if ((t & 63u) == 0) s_cnt64[t >> 6] = acc;
        __syncthreads();
        if (t == 0) {
            unsigned long long sum = 0;
            for (int w = 0; w < 16; ++w) sum += s_cnt64[w];
            survivors_total = sum;
        }
    };
    // (cross_bits: S right behind the window's last crossing, since_cross: the blocks folded since, a
    // fraction inside the crossing block; bits0 and `advanced` for a window without a crossing)
    auto finish = [&](uint32_t bits, uint32_t advanced, uint32_t cross_bits, double since_cross) {
        const uint64_t pos = pos0 + advanced;
        const bool finite = ((bits >> 23) & 0xffu) != 0xffu;
        const double s_before = (double)__uint_as_float(bits0), s_after = (double)__uint_as_float(bits);
        double rate_elems = 0.0;
        const double rate = seq_window_rate(s_before, s_after, (double)advanced, (double)__uint_as_float(cross_bits),
                                            since_cross, &rate_elems);
        SeqState next;
        next.s_bits = bits;
        next.pos = pos;
        next.error = (advanced == 0 || advanced > nblocks) ? 1u : 0u;
        next.done = (pos >= total_blocks || !finite || next.error) ? 1u : 0u;
        uint32_t next_multi = 0u;
        next.win = next.done ? 0u : (uint32_t)seq_plan_window(pos, total_blocks, s_after, rate, rate_elems, &next_multi);
        next.multi = next.done ? 0u : next_multi;
        next.rate_lo = seq_multi_rate_lo(rate);
        next.saw_nan = 0;
        next.thr_bits = st0.thr_bits;
        next.windows = st0.windows + 1u;
        next.pad = 0;
        next.survivors = survivors_total;
        const uint64_t seen = pos0 + nblocks, before = st0.fresh_from;
        next.fresh_from = seen > before ? seen : before;
        *state = next;
        if (mirror) *host_copy = next;  // a store to pinned host memory: only when somebody will look
    };

    // ---- the first block of a sum: S = +0 has no binade to make maps for; the block is replayed at
    // once (no maps launch runs before this one), and packed here when the sum goes with packing
    if (pos0 == 0 && bits0 == 0u && nblocks == 1u) {
        if (t == 0) s_cnt0 = 0;
        __syncthreads();
        const uint32_t result_bits = seq_replay_block(x, n, 0, use_mask, thr, 1u, 0u, s_w, &s_first, &s_bits_now, s_head,
                                                      s_cross, count_parts ? packed : nullptr, &s_cnt0);
        __syncthreads();
        if (t == 0 && count_parts) count_parts[n_parts - 1] = s_cnt0;  // the last slot is this block's
        __syncthreads();
        count_survivors(1);
        if (t == 0) finish(result_bits, 1, bits0, 1.0);
        return;
    }

    // ---- a window with two maps per block: through as many binades as the maps hold ---------
    if (st0.multi) {
        // at most SEQ_MULTI_LIMIT blocks: eight per thread, loaded once (both maps of a block are
        // one 16-byte load)
        const uint32_t rate_lo = st0.rate_lo;
        if (nblocks > SEQ_MULTI_LIMIT) {  // not a window the plan makes: reported as an internal error
            if (t == 0) finish(bits0, 0, bits0, 0.0);
            return;
        }
        // The window's maps go to LDS once (both maps of a block are one 16-byte unit): kept in
        // registers across the replays they did not fit and were spilled.
        for (uint32_t b = t; b < nblocks; b += 1024u) s_maps[b] = reinterpret_cast<const uint4 *>(maps)[b];
        __syncthreads();
        // s_edge[i]: the first block of the window whose lower exponent exceeds es0 + i (nblocks if
        // there is none).  The exponents never fall along the window, so this is the first b with
        // S0 + b * rate_lo >= 2^(e+1-127): guessed by a division, settled with the predicate itself.
        constexpr uint32_t kEdges = 64;
        const uint32_t es0 = es;
        if (t < kEdges) {
            const uint32_t e = es0 + t, a = 0u, z = nblocks;
            const float s0 = __uint_as_float(bits0), r = __uint_as_float(rate_lo);
            uint32_t g = a;
            if (e + 1u <= 254u && r > 0.0f) {
                const float edge = __uint_as_float((e + 1u) << 23);
                const float q = (edge - s0) / r;
                g = q <= (float)a ? a : (q >= (float)z ? z : (uint32_t)q);
            }
            int steps = 0;
            while (g > a && seq_multi_es_lo(bits0, rate_lo, g - 1u) > e && steps < 8) --g, ++steps;
            while (g < z && !(seq_multi_es_lo(bits0, rate_lo, g) > e) && steps < 16) ++g, ++steps;
            const bool settled = (g == a || !(seq_multi_es_lo(bits0, rate_lo, g - 1u) > e)) &&
                                 (g == z || seq_multi_es_lo(bits0, rate_lo, g) > e);
            if (!settled) {  // the guess was far off (a rate next to nothing): bisect
                uint32_t lo2 = a, hi2 = z;
                while (lo2 < hi2) {
                    const uint32_t mid = lo2 + ((hi2 - lo2) >> 1);
                    if (seq_multi_es_lo(bits0, rate_lo, mid) > e) hi2 = mid; else lo2 = mid + 1u;
                }
                g = lo2;
            }
            s_edge[t] = g;
        }
        __syncthreads();
        uint32_t b_cur = 0, cur_bits = bits0;
        uint32_t cross_bits = bits0, cross_block = 0, cross_chunks = 0;  // the last crossing
        bool crossed = false;
        for (int guard = 0; guard < 48; ++guard) {
            uint32_t k_in;
            seq_state_split(cur_bits, &es, &k_in);
            // The blocks from b_cur on whose pair holds `es` reach up to the first one whose lower
            // exponent exceeds es - provided the pair of b_cur itself is not below es; among them,
            // those before b_eq stand for es with their second map, the others with their first.
            if (es - es0 >= kEdges) break;  // further than the table reaches: the next window starts here
            const uint32_t range_end = s_edge[es - es0];
            const uint32_t b_eq = es == es0 ? 0u : s_edge[es - es0 - 1u];  // first block whose lower exponent is es
            // b_cur's pair must hold es: its lower exponent is es (b_cur >= b_eq) or es - 1
            const uint32_t b_lowest = es - es0 >= 2u ? s_edge[es - es0 - 2u] : 0u;  // first block with es - 1
            if (b_cur >= range_end || b_cur < b_lowest) break;  // the prediction has lost S
            // the range in equal shares (at most eight blocks per thread)
            const uint32_t chunk = (range_end - b_cur + 1023u) / 1024u;
            const uint32_t lo = b_cur + t * chunk;
            const uint32_t hi = lo + chunk < range_end ? lo + chunk : range_end;
            auto pick = [&](uint32_t b) {
                const uint4 mm = s_maps[b];
                SeqMap r;
                r.d0 = b < b_eq ? mm.z : mm.x;
                r.d1 = b < b_eq ? mm.w : mm.y;
                return r;
            };
            SeqMap mine = seq_identity();
            for (uint32_t b2 = lo; b2 < hi; ++b2) mine = seq_compose(mine, pick(b2));
            if (t == 0) s_min64 = ~0ull;
            SeqMap all;
            const SeqMap before = seq_block_before<16>(mine, s_w, &all);
            uint32_t k = seq_apply(before, k_in);
            if (k < SEQ_K_LIMIT) {
                for (uint32_t b2 = lo; b2 < hi; ++b2) {
                    const uint32_t k2 = seq_apply(pick(b2), k);
                    if (k2 >= SEQ_K_LIMIT) {
                        // the first crossing block and the k that enters it, as one 64-bit minimum
                        atomicMin(&s_min64, ((unsigned long long)b2 << 32) | k);
                        break;
                    }
                    k = k2;
                }
            }
            __syncthreads();
            const unsigned long long first_cross = s_min64;
            if (first_cross == ~0ull) {
                // no crossing up to range_end: the state there is what all maps of the range give
                cur_bits = seq_state_join(es, seq_apply(all, k_in));
                b_cur = range_end;
                break;  // the window is through, or the next block's pair does not hold es
            }
            const uint32_t cb = (uint32_t)(first_cross >> 32), k_cb = (uint32_t)first_cross;
            if (!seq_replay_block_once(x, n, first + (uint64_t)cb * kSeqTile, use_mask, thr, es, k_cb, s_w, &s_bits_now,
                                       s_cross, &s_once)) {
                __syncthreads();  // (s_once was read)
                (void)seq_replay_block(x, n, first + (uint64_t)cb * kSeqTile, use_mask, thr, es, k_cb, s_w, &s_first,
                                       &s_bits_now, s_head, s_cross);
            }
            __syncthreads();  // the result is in LDS; s_w and s_min64 are rewritten in the next turn
            cur_bits = s_bits_now;
            cross_bits = s_cross[0], cross_chunks = s_cross[1], cross_block = cb, crossed = true;
            b_cur = cb + 1u;
            if (((cur_bits >> 23) & 0xffu) == 0xffu || b_cur >= nblocks) break;
        }
        count_survivors(b_cur);
        // blocks folded since the last crossing: the rest of its block and the whole ones behind it
        const double since = !crossed
                                 ? (double)b_cur
                                 : (double)(b_cur - cross_block - 1u) + (double)((uint32_t)kBlock - cross_chunks) / kBlock;
        if (t == 0) finish(cur_bits, b_cur, cross_bits, since);
        return;
    }

    // ---- (1) scan -----------------------------------------------------------------------
    {
        const uint32_t chunk = (nblocks + 1023u) / 1024u;
        uint32_t lo = t * chunk;
        uint32_t hi = lo + chunk < nblocks ? lo + chunk : nblocks;
        // A thread's maps are loaded once, all loads in flight, and kept in registers for
        // both walks (composition, then the search for the crossing): up to 32 of them.  A window of
        // more than 32768 blocks is walked in stretches of that many, each from the state the one
        // before it ends in, up to the stretch that holds the crossing (in batches of eight per thread,
        // one round trip to memory after the other, 45,000 blocks took 36 us; so they take 8).
        // Spare slots re-read the chunk's last map and are skipped.
        SeqMap mine = seq_identity();
        uint32_t k = 0, cand = 0xffffffffu, cand_k = 0;
        uint32_t k_in = k0;  // the state that enters the stretch
        SeqMap stretch = seq_identity();  // the map of the whole stretch
        const SeqMap *run_maps = maps + t;  // the thread's run: every 1024th slot from here (seq_map_slot)
        if (t == 0) s_first = 0xffffffffu;
        auto walk_cached = [&](auto size_tag) {
            constexpr int C = decltype(size_tag)::value;
            SeqMap mm[C];
            if constexpr (C == 1) {
                mm[0] = spec;
            } else {
#pragma unroll
                for (int i = 0; i < C; ++i) mm[i] = run_maps[(uint32_t)i * SEQ_SCAN_THREADS];  // (slots past the run are skipped)
            }
#pragma unroll
            for (int i = 0; i < C; ++i)
                if (lo + i < hi) mine = seq_compose(mine, mm[i]);
            const SeqMap before = seq_block_before<16>(mine, s_w, &stretch);
            k = seq_apply(before, k_in);
            if (k < SEQ_K_LIMIT) {
#pragma unroll
                for (int i = 0; i < C; ++i) {
                    if (lo + i < hi && cand == 0xffffffffu) {
                        const uint32_t k2 = seq_apply(mm[i], k);
                        if (k2 >= SEQ_K_LIMIT) {
                            cand = lo + i;
                            cand_k = k;
                        } else {
                            k = k2;
                        }
                    }
                }
            }
        };
        if (chunk == 1u) {
            walk_cached(std::integral_constant<int, 1>{});
        } else if (chunk <= 8u) {
            walk_cached(std::integral_constant<int, 8>{});
        } else if (chunk <= 32u) {
            walk_cached(std::integral_constant<int, 32>{});
        } else {
            constexpr uint32_t kStretch = SEQ_SCAN_THREADS * SEQ_SCAN_RUN;
            for (uint32_t from = 0; from < nblocks; from += kStretch) {
                const uint32_t to = nblocks - from > kStretch ? from + kStretch : nblocks;
                lo = from + t * SEQ_SCAN_RUN;
                lo = lo < to ? lo : to;
                hi = lo + SEQ_SCAN_RUN < to ? lo + SEQ_SCAN_RUN : to;
                run_maps = maps + from + t;
                mine = seq_identity();
                walk_cached(std::integral_constant<int, 32>{});
                if (to == nblocks) break;  // the last stretch: its crossing, or the end of the window, is settled below
                if (cand != 0xffffffffu) atomicMin(&s_first, cand);
                __syncthreads();  // (also: s_w is rewritten by the next stretch)
                if (s_first != 0xffffffffu) break;
                k_in = seq_apply(stretch, k_in);
            }
        }
        if (cand != 0xffffffffu) atomicMin(&s_first, cand);
        __syncthreads();
        const uint32_t first_cross = s_first;
        if (first_cross != 0xffffffffu) {
            if (cand == first_cross) {
                s_cross_block = first_cross;
                s_cross_k = cand_k;
            }
        } else if (hi == nblocks && lo < hi) {
            // this thread owns the last block of the window: k is the state after it
            s_cross_block = 0xffffffffu;
            s_cross_k = k;
        }
        __syncthreads();
    }
    const uint32_t cb = s_cross_block;
    uint32_t k_cur = s_cross_k;
    if (cb == 0xffffffffu) {
        count_survivors(nblocks);
        if (t == 0) finish(seq_state_join(es, k_cur), nblocks, bits0, (double)nblocks);
        return;
    }

    // ---- (2) replay of block cb
    uint32_t result_bits;
    if (seq_replay_block_once(x, n, first + (uint64_t)cb * kSeqTile, use_mask, thr, es, k_cur, s_w, &s_bits_now, s_cross,
                              &s_once)) {
        result_bits = s_bits_now;
    } else {
        __syncthreads();  // (s_once was read)
        result_bits = seq_replay_block(x, n, first + (uint64_t)cb * kSeqTile, use_mask, thr, es, k_cur, s_w, &s_first,
                                       &s_bits_now, s_head, s_cross);
    }
    count_survivors(cb + 1);
    if (t == 0) finish(result_bits, cb + 1, s_cross[0], (double)((uint32_t)kBlock - s_cross[1]) / kBlock);
}

__global__ __launch_bounds__(kBlock) void any_nan_kernel(const float *__restrict__ x,
                                                         uint64_t first, uint64_t n,
                                                         SeqState *__restrict__ state) {
    uint64_t stride = (uint64_t)gridDim.x * kBlock;
    bool found = false;
    for (uint64_t i = first + (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        found |= (x[i] != x[i]);
    if (found) atomicOr(&state->saw_nan, 1u);
}

// ---------------------------------------------------------------------------
// dequantize_ternary, get_value expansion, weight tiling
// ---------------------------------------------------------------------------
__device__ __forceinline__ int ternary_value(uint32_t code) {
    // quantization.rs:285-290: 00 -> -1, 01 -> 0, 10 -> +1, 11 -> 0
    return code == 0u ? -1 : (code == 2u ? 1 : 0);
}

__global__ __launch_bounds__(kBlock) void dequantize_ternary_kernel(
    const uint8_t *__restrict__ packed, uint64_t n, float scale, float *__restrict__ out) {
    uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        uint32_t code = (packed[i >> 2] >> ((i & 3) * 2)) & 3u;
        out[i] = code == 0u ? -scale : (code == 2u ? scale : 0.0f);
    }
}

// One block per row: q[r, c] = get_value(r*cols + c), zero beyond cols; rowsum[r].
__global__ __launch_bounds__(kBlock) void unpack_ternary_i8_kernel(
    const uint8_t *__restrict__ packed, uint64_t cols, uint64_t pitch, int8_t *__restrict__ q,
    int32_t *__restrict__ rowsum) {
    __shared__ int s_sum[kBlock];
    const uint64_t r = blockIdx.x;
    int acc = 0;
    for (uint64_t c = threadIdx.x; c < pitch; c += kBlock) {
        int v = 0;
        if (c < cols) {
            uint64_t i = r * cols + c;
            v = ternary_value((packed[i >> 2] >> ((i & 3) * 2)) & 3u);
        }
        q[r * pitch + c] = (int8_t)v;
        acc += v;
    }
    s_sum[threadIdx.x] = acc;
    __syncthreads();
    for (int off = kBlock / 2; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off) s_sum[threadIdx.x] += s_sum[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0 && rowsum) rowsum[r] = s_sum[0];
}

// "packed" [K,N] -> "tiled": u32 word ((q * KB + kb) * 4 + c) holds column 4q+c, k-block kb;
// see the header for the bit layout inside a word.
__global__ __launch_bounds__(kBlock) void tile_weights_kernel(
    const uint8_t *__restrict__ packed, uint64_t K, uint64_t N, uint64_t kblocks, uint64_t n_words,
    uint32_t *__restrict__ tiled) {
    uint64_t w = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (w >= n_words) return;
    const uint64_t q = w / (kblocks * 4), rem = w % (kblocks * 4);
    const uint64_t kb = rem >> 2, n = q * 4 + (rem & 3);
    uint32_t word = 0;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint64_t k = kb * 16 + 4 * s + b;
            uint32_t code = 1u;  // padding is a zero weight
            if (k < K && n < N) {
                uint64_t i = k * N + n;
                code = (packed[i >> 2] >> ((i & 3) * 2)) & 3u;
                if (code == 3u) code = 1u;  // invalid pattern reads as zero
            }
            word |= code << (8 * b + 2 * s);
        }
    }
    tiled[w] = word;
}

// Device scalars used by the reductions, at the start of the context workspace.
struct ReduceScratch {
    SeqState seq;
    SeqState seq_next;  // the sum queued behind `seq`
    unsigned long long survivors;
    float tree_sum;
    float tree_threshold;  // the tree-sum quantiser: the threshold its packing pass reads
    unsigned long long tree_cnt;
    float pack_sum;  // ... and the survivors' sum of that pass
    uint32_t pad0;
};
constexpr size_t kScratchHeader = 256;
static_assert(sizeof(ReduceScratch) <= kScratchHeader, "scratch header too small");
constexpr int kTreeParts = 2048;

inline bool is_finite_bits(uint32_t b) { return ((b >> 23) & 0xffu) != 0xffu; }

constexpr size_t kSeqScanLds = (size_t)SEQ_MULTI_LIMIT * 16;  // dynamic LDS of the window-end kernel

// Exact sequential sum (optionally masked) of |x| over n elements.
int pack_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, float threshold, uint8_t *d_packed,
                 uint64_t *h_survivors, float *h_survivor_sum);

// One sum as the window kernels see it.
struct SeqRun {
    int use_mask;
    float thr;
    int thr_from_state;  // the kernels take the threshold from the device state instead of thr
    SeqState *d_state, *h_state;
    uint32_t *d_packed;
    unsigned long long *count_parts;
};

// A second sum queued behind the first without the host in between: the quantiser's masked sum,
// whose threshold (S / n) * 0.7 the device derives from the first sum's result.  `ran` is false
// when the chain broke (the first sum needed another look by the host, or left the finite range):
// the caller then runs the second sum the ordinary way.
struct SeqFollower {
    uint8_t *d_packed;
    float *h_sum;
    uint64_t *h_survivors;
    bool ran;
};

// With d_packed given (use_mask must be set, thr is the ternary threshold) the same pass also
// packs the tensor and counts the survivors into *h_survivors.
int strict_abs_sum(rbn_ctx *ctx, const float *d_x, uint64_t n, int use_mask, float thr,
                   float *h_sum, uint8_t *d_packed = nullptr, uint64_t *h_survivors = nullptr,
                   SeqFollower *follower = nullptr) {
    if (follower) follower->ran = false;
    if (n == 0) {
        *h_sum = -0.0f;  // Rust's empty f32 sum
        if (h_survivors) *h_survivors = 0;
        return RBN_OK;
    }
    constexpr int kMapGrid = 8192;
    const uint64_t total_blocks = (n + kSeqTile - 1) / kSeqTile;
    void *ws = nullptr;
    // at least 1024 map slots: the window-end kernel reads slot threadIdx.x before it knows the window
    // and two per block for the windows that span several binades
    // and a stretch more than blocks: the maps of a window are stored transposed (seq_map_slot), in
    // slots up to the window rounded up to a stretch, and the window-end kernel loads a thread's
    // whole run of slots whatever the window
    const uint64_t map_slots = (total_blocks > 2 * SEQ_MULTI_LIMIT ? total_blocks : 2 * SEQ_MULTI_LIMIT) +
                               SEQ_SCAN_THREADS * SEQ_SCAN_RUN;
    RBN_CHECK(rbn_workspace(ctx, kScratchHeader + map_slots * sizeof(SeqMap) + (kMapGrid + 1) * 8, &ws));
    ReduceScratch *scr = (ReduceScratch *)ws;
    SeqMap *maps = (SeqMap *)((char *)ws + kScratchHeader);
    unsigned long long *parts_mem = (unsigned long long *)((char *)ws + kScratchHeader + map_slots * sizeof(SeqMap));
    if (!ctx->seq_scan_prepared) {  // (once per context: the call costs the host a few microseconds)
        RBN_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(seq_scan_replay_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSeqScanLds));
        ctx->seq_scan_prepared = true;
    }
    SeqRun main_run{use_mask, thr, 0, &scr->seq, (SeqState *)ctx->mailbox, (uint32_t *)d_packed,
                    d_packed ? parts_mem : nullptr};
    memset(main_run.h_state, 0, sizeof(SeqState));
    seq_init_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(
        main_run.d_state, 1u /* the first window is the first block */, main_run.count_parts, kMapGrid + 1);
    // Windows are queued in batches: the kernels take each window from the device state and
    // return at once when the sum is complete, so the host only looks in between batches and
    // sizes the next one by the binades S still has to climb (a window ends where S leaves
    // its binade).
    const unsigned grid = (unsigned)(total_blocks < (uint64_t)kMapGrid ? total_blocks : (uint64_t)kMapGrid);
    auto queue_batch = [&](const SeqRun &r, int batch, bool first_batch) {
        for (int i = 0; i < batch; ++i) {
            // (the very first window is the first block from S = +0: the window-end kernel replays it
            // without maps, so no maps launch goes before it)
            if (!(first_batch && i == 0))
                seq_block_maps_kernel<<<dim3(grid), dim3(kBlock), 0, ctx->stream>>>(
                    d_x, n, r.use_mask, r.thr, r.thr_from_state, r.d_state, maps, r.d_packed, r.count_parts);
            seq_scan_replay_kernel<<<dim3(1), dim3(1024), kSeqScanLds, ctx->stream>>>(
                maps, d_x, n, total_blocks, r.use_mask, r.thr, r.thr_from_state, r.d_state, r.h_state,
                i == batch - 1, r.count_parts, kMapGrid + 1, r.d_packed);
        }
    };
    // Looks at the state the last batch left and queues batches until the sum is complete.
    auto run_to_end = [&](const SeqRun &r) -> int {
        for (;;) {
            if (r.h_state->error)
                return rbn_fail(RBN_ERR_HIP, "sequential-sum scan made no progress (internal error)");
            if (r.h_state->done) return RBN_OK;
            // S grows by about s_now * (blocks left / blocks done) more: one window per doubling
            const double done_blocks = (double)r.h_state->pos, left = (double)(total_blocks - r.h_state->pos);
            const double growth = 1.0 + left / (done_blocks > 1.0 ? done_blocks : 1.0);
            int batch = (int)(log2(growth) + 1.5);
            batch = batch < 1 ? 1 : (batch > 16 ? 16 : batch);
            queue_batch(r, batch, false);
            RBN_HIP(hipGetLastError());
            RBN_HIP(hipStreamSynchronize(ctx->stream));
        }
    };
    // first batch: the binades of the first SEQ_MULTI_LIMIT blocks take two windows (the first
    // block, and one that carries a pair of maps per block); after them S of similar terms climbs one
    // binade per doubling of the position; plus one more (a window that ends early, or a spare
    // pair of launches returns at once: 4 us; another look by the host costs 10-25 us)
    int batch = 4;
    for (uint64_t b = total_blocks / SEQ_MULTI_LIMIT; b > 1; b >>= 1) ++batch;
    // ... unless the context has just summed a tensor of this size: sums that stall (rounding eats the
    // terms in the highest binades) and windows sized by a good rate need fewer, and a pair of
    // launches that finds the sum complete still costs 6 us.  One spare beyond what the last
    // sums of this size took; a sum that needs more costs a look by the host.
    if (ctx->seq_seen_blocks == total_blocks && ctx->seq_seen_windows > 0 && ctx->seq_seen_windows + 1 < batch)
        batch = ctx->seq_seen_windows + 1;
    int windows_taken = 0;
    queue_batch(main_run, batch, true);
    SeqRun next_run{};
    if (follower) {
        next_run = SeqRun{1, 0.0f, 1, &scr->seq_next, (SeqState *)((char *)ctx->mailbox + 256),
                          (uint32_t *)follower->d_packed, parts_mem};
        memset(next_run.h_state, 0, sizeof(SeqState));
        seq_chain_init_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(
            main_run.d_state, next_run.d_state, n, total_blocks, next_run.count_parts, kMapGrid + 1);
        queue_batch(next_run, batch, true);
    }
    RBN_HIP(hipGetLastError());
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    RBN_CHECK(run_to_end(main_run));
    SeqState *h_state = main_run.h_state;
    windows_taken = (int)h_state->windows;
    const uint32_t s_bits = h_state->s_bits;
    const uint64_t pos = h_state->pos;
    float s;
    memcpy(&s, &s_bits, 4);
    if (!is_finite_bits(s_bits) && s == s && pos < total_blocks && !use_mask) {
        // S is +Inf: it stays +Inf unless a NaN follows (masked sums never take a NaN).
        any_nan_kernel<<<dim3(1024), dim3(kBlock), 0, ctx->stream>>>(d_x, pos * kSeqTile, n,
                                                                     &scr->seq);
        RBN_HIP(hipGetLastError());
        RBN_HIP(hipMemcpyAsync(h_state, &scr->seq, sizeof(SeqState), hipMemcpyDeviceToHost,
                               ctx->stream));
        RBN_HIP(hipStreamSynchronize(ctx->stream));
        if (h_state->saw_nan) s = NAN;
    }
    *h_sum = s;
    if (d_packed) {
        if (pos < total_blocks) {
            // the sum left the finite range before the end: the windows stopped there, so
            // pack (and count) with the plain kernel
            RBN_CHECK(pack_ternary(ctx, d_x, n, thr, d_packed, h_survivors, nullptr));
        } else if (h_survivors) {
            *h_survivors = h_state->survivors;  // added up by the window that folded the last block
        }
    }
    if (follower) {
        SeqState *h_next = next_run.h_state;
        // the threshold the device derived must be the host's own (same two IEEE operations)
        volatile float mean = s / (float)n;
        volatile float host_thr = mean * 0.7f;
        float thr_f = host_thr;
        uint32_t host_thr_bits;
        memcpy(&host_thr_bits, &thr_f, 4);
        const bool chained = !(h_next->done && h_next->error == 2u) && h_next->thr_bits == host_thr_bits &&
                             is_finite_bits(s_bits) && pos >= total_blocks;
        if (chained) {
            RBN_CHECK(run_to_end(next_run));
            float s_next;
            memcpy(&s_next, &h_next->s_bits, 4);
            *follower->h_sum = s_next;
            if (h_next->pos < total_blocks)
                RBN_CHECK(pack_ternary(ctx, d_x, n, thr_f, follower->d_packed, follower->h_survivors, nullptr));
            else
                *follower->h_survivors = h_next->survivors;
            follower->ran = true;
            if ((int)h_next->windows > windows_taken) windows_taken = (int)h_next->windows;
        }
    }
    ctx->seq_seen_blocks = total_blocks;
    ctx->seq_seen_windows = windows_taken;
    return RBN_OK;
}

int tree_abs_sum(rbn_ctx *ctx, const float *d_x, uint64_t n, int use_mask, float thr,
                 float *h_sum, uint64_t *h_count) {
    if (n == 0) {
        *h_sum = -0.0f;
        if (h_count) *h_count = 0;
        return RBN_OK;
    }
    void *ws = nullptr;
    RBN_CHECK(rbn_workspace(ctx, kScratchHeader + kTreeParts * 16, &ws));
    ReduceScratch *scr = (ReduceScratch *)ws;
    double *psum = (double *)((char *)ws + kScratchHeader);
    unsigned long long *pcnt = (unsigned long long *)(psum + kTreeParts);
    uint64_t want = (n + kSeqTile - 1) / kSeqTile;
    int parts = (int)(want < (uint64_t)kTreeParts ? want : (uint64_t)kTreeParts);
    if (n * 4 > kStreamBytes)
        abs_sum_tree_partial_kernel<true><<<dim3(parts), dim3(kBlock), 0, ctx->stream>>>(d_x, n, use_mask,
                                                                                        thr, psum, pcnt);
    else
        abs_sum_tree_partial_kernel<false><<<dim3(parts), dim3(kBlock), 0, ctx->stream>>>(d_x, n, use_mask,
                                                                                         thr, psum, pcnt);
    abs_sum_tree_final_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(
        psum, pcnt, parts, &scr->tree_sum, &scr->tree_cnt);
    RBN_HIP(hipGetLastError());
    char *mb = (char *)ctx->mailbox;
    RBN_HIP(hipMemcpyAsync(mb, &scr->tree_sum, 4, hipMemcpyDeviceToHost, ctx->stream));
    RBN_HIP(hipMemcpyAsync(mb + 8, &scr->tree_cnt, 8, hipMemcpyDeviceToHost, ctx->stream));
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    memcpy(h_sum, mb, 4);
    if (h_count) memcpy(h_count, mb + 8, 8);
    return RBN_OK;
}

// pack + survivor count (count returned through the mailbox when h_survivors != NULL) and,
// when h_survivor_sum != NULL, the survivors' sum of |x| as a deterministic f64 tree (the
// tree mode's scale rides on the packing pass; the strict mode's cannot)
constexpr int kPackGrid = 8192;
int pack_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, float threshold, uint8_t *d_packed,
                 uint64_t *h_survivors, float *h_survivor_sum) {
    if (n == 0) {
        if (h_survivors) *h_survivors = 0;
        if (h_survivor_sum) *h_survivor_sum = -0.0f;
        return RBN_OK;
    }
    unsigned long long *d_cnt = nullptr;
    double *d_psum = nullptr;
    ReduceScratch *scr = nullptr;
    if (h_survivors || h_survivor_sum) {
        void *ws = nullptr;
        RBN_CHECK(rbn_workspace(ctx, kScratchHeader + (size_t)kPackGrid * sizeof(double), &ws));
        scr = (ReduceScratch *)ws;
        d_cnt = &scr->survivors;
        if (h_survivor_sum) d_psum = (double *)((char *)ws + kScratchHeader);
        memset(ctx->mailbox, 0, 8);
        RBN_HIP(hipMemcpyAsync(d_cnt, ctx->mailbox, 8, hipMemcpyHostToDevice, ctx->stream));
    }
    uint64_t tiles = (n + kSeqTile - 1) / kSeqTile;
    if (tiles > 0x7fffffffull) return rbn_fail(RBN_ERR_UNSUPPORTED, "tensor too large");
    const unsigned grid = (unsigned)(tiles < (uint64_t)kPackGrid ? tiles : (uint64_t)kPackGrid);
    if (n * 4 > kStreamBytes)
        pack_ternary_kernel<true><<<dim3(grid), dim3(kBlock), 0, ctx->stream>>>(
            d_x, n, threshold, nullptr, (uint32_t *)d_packed, tiles, d_cnt, d_psum);
    else
        pack_ternary_kernel<false><<<dim3(grid), dim3(kBlock), 0, ctx->stream>>>(
            d_x, n, threshold, nullptr, (uint32_t *)d_packed, tiles, d_cnt, d_psum);
    if (d_psum)
        sum_partials_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(d_psum, (int)grid, &scr->tree_sum);
    RBN_HIP(hipGetLastError());
    if (scr) {
        char *mb = (char *)ctx->mailbox;
        RBN_HIP(hipMemcpyAsync(mb, d_cnt, 8, hipMemcpyDeviceToHost, ctx->stream));
        if (d_psum) RBN_HIP(hipMemcpyAsync(mb + 8, &scr->tree_sum, 4, hipMemcpyDeviceToHost, ctx->stream));
        RBN_HIP(hipStreamSynchronize(ctx->stream));
        if (h_survivors) memcpy(h_survivors, mb, 8);
        if (h_survivor_sum) memcpy(h_survivor_sum, mb + 8, 4);
    }
    return RBN_OK;
}

// The tree-sum quantiser in one queue: sum, threshold on the device, packing pass with the
// survivors' count and sum, one look by the host at the end.  *chained is false when the device's
// threshold is not the host's own (sum / n) * 0.7 bit for bit: the caller then packs again the
// ordinary way.
int tree_quantize_chained(rbn_ctx *ctx, const float *d_x, uint64_t n, uint8_t *d_packed, float *h_sum,
                          uint64_t *h_survivors, float *h_survivor_sum, bool *chained) {
    *chained = false;
    const uint64_t tiles = (n + kSeqTile - 1) / kSeqTile;
    if (n == 0 || tiles > 0x7fffffffull) return RBN_OK;
    void *ws = nullptr;
    RBN_CHECK(rbn_workspace(ctx, kScratchHeader + kTreeParts * 16 + (size_t)kPackGrid * sizeof(double), &ws));
    ReduceScratch *scr = (ReduceScratch *)ws;
    double *psum = (double *)((char *)ws + kScratchHeader);
    unsigned long long *pcnt = (unsigned long long *)(psum + kTreeParts);
    double *pack_psum = (double *)((char *)ws + kScratchHeader + kTreeParts * 16);
    const int parts = (int)(tiles < (uint64_t)kTreeParts ? tiles : (uint64_t)kTreeParts);
    const unsigned grid = (unsigned)(tiles < (uint64_t)kPackGrid ? tiles : (uint64_t)kPackGrid);
    const bool stream = n * 4 > kStreamBytes;
    if (stream)
        abs_sum_tree_partial_kernel<true><<<dim3(parts), dim3(kBlock), 0, ctx->stream>>>(d_x, n, 0, 0.0f, psum, pcnt);
    else
        abs_sum_tree_partial_kernel<false><<<dim3(parts), dim3(kBlock), 0, ctx->stream>>>(d_x, n, 0, 0.0f, psum, pcnt);
    abs_sum_tree_final_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(
        psum, pcnt, parts, &scr->tree_sum, &scr->tree_cnt, n, &scr->tree_threshold, &scr->survivors);
    if (stream)
        pack_ternary_kernel<true><<<dim3(grid), dim3(kBlock), 0, ctx->stream>>>(
            d_x, n, 0.0f, &scr->tree_threshold, (uint32_t *)d_packed, tiles, &scr->survivors, pack_psum);
    else
        pack_ternary_kernel<false><<<dim3(grid), dim3(kBlock), 0, ctx->stream>>>(
            d_x, n, 0.0f, &scr->tree_threshold, (uint32_t *)d_packed, tiles, &scr->survivors, pack_psum);
    sum_partials_kernel<<<dim3(1), dim3(kBlock), 0, ctx->stream>>>(pack_psum, (int)grid, &scr->pack_sum);
    RBN_HIP(hipGetLastError());
    char *mb = (char *)ctx->mailbox;
    constexpr size_t kBack = offsetof(ReduceScratch, pad0) - offsetof(ReduceScratch, survivors);  // survivors .. pack_sum
    RBN_HIP(hipMemcpyAsync(mb, &scr->survivors, kBack, hipMemcpyDeviceToHost, ctx->stream));
    RBN_HIP(hipStreamSynchronize(ctx->stream));
    ReduceScratch back;
    memcpy(&back.survivors, mb, kBack);
    *h_sum = back.tree_sum;
    volatile float mean = back.tree_sum / (float)n;
    volatile float want = mean * 0.7f;
    float want_f = want;
    if (memcmp(&want_f, &back.tree_threshold, 4) != 0) return RBN_OK;
    *h_survivors = back.survivors;
    *h_survivor_sum = back.pack_sum;
    *chained = true;
    return RBN_OK;
}

int check_f32_ptr(const float *p, const char *name) {
    RBN_REQUIRE(p != nullptr, "%s is NULL", name);
    RBN_REQUIRE(((uintptr_t)p & 15u) == 0, "%s must be 16-byte aligned", name);
    return RBN_OK;
}

}  // namespace

extern "C" {

int rbn_abs_sum_f32(rbn_ctx *ctx, const float *d_x, uint64_t n, int mode, int use_mask,
                    float mask_threshold, float *h_sum, uint64_t *h_count) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_sum != nullptr, "h_sum is NULL");
    RBN_REQUIRE(mode == RBN_SUM_STRICT_SEQ || mode == RBN_SUM_TREE, "unknown sum mode %d", mode);
    if (n > 0) RBN_CHECK(check_f32_ptr(d_x, "d_x"));
    if (mode == RBN_SUM_TREE)
        return tree_abs_sum(ctx, d_x, n, use_mask, mask_threshold, h_sum, h_count);
    RBN_CHECK(strict_abs_sum(ctx, d_x, n, use_mask, mask_threshold, h_sum));
    uint64_t count = n;
    if (use_mask) {
        float unused;
        RBN_CHECK(tree_abs_sum(ctx, d_x, n, 1, mask_threshold, &unused, &count));
        if (count == 0) *h_sum = -0.0f;  // the fold never ran: Rust's empty f32 sum
    }
    if (h_count) *h_count = count;
    return RBN_OK;
}

int rbn_pack_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, float threshold,
                     uint8_t *d_packed) {
    RBN_ENTER(ctx);
    if (n == 0) return RBN_OK;
    RBN_CHECK(check_f32_ptr(d_x, "d_x"));
    RBN_REQUIRE(d_packed && ((uintptr_t)d_packed & 3u) == 0, "d_packed must be 4-byte aligned");
    return pack_ternary(ctx, d_x, n, threshold, d_packed, nullptr, nullptr);
}

int rbn_quantize_ternary(rbn_ctx *ctx, const float *d_x, uint64_t n, int mode, uint8_t *d_packed,
                         float *h_scale, float *h_threshold, uint64_t *h_survivors) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_scale && h_threshold, "h_scale / h_threshold is NULL");
    RBN_REQUIRE(mode == RBN_SUM_STRICT_SEQ || mode == RBN_SUM_TREE, "unknown sum mode %d", mode);
    if (n > 0) {
        RBN_CHECK(check_f32_ptr(d_x, "d_x"));
        RBN_REQUIRE(d_packed && ((uintptr_t)d_packed & 3u) == 0,
                    "d_packed must be 4-byte aligned");
    }
    // quantization.rs:79: (sum / n as f32) * 0.7
    float sum = 0.0f;
    uint64_t survivors = 0;
    float nz_sum = 0.0f;
    bool tree_chained = false;
    if (mode == RBN_SUM_TREE) {
        RBN_CHECK(tree_quantize_chained(ctx, d_x, n, d_packed, &sum, &survivors, &nz_sum, &tree_chained));
        if (!tree_chained) RBN_CHECK(tree_abs_sum(ctx, d_x, n, 0, 0.0f, &sum, nullptr));
    }
    SeqFollower masked{d_packed, &nz_sum, &survivors, false};
    if (mode != RBN_SUM_TREE)
        RBN_CHECK(strict_abs_sum(ctx, d_x, n, 0, 0.0f, &sum, nullptr, nullptr, &masked));
    volatile float mean = sum / (float)n;
    volatile float threshold = mean * 0.7f;
    // quantization.rs:100 (pack) and the survivor count of :82-91
    // (one pass in either mode: the survivors' sum, their count and the packed words)
    if (mode == RBN_SUM_TREE) {
        if (!tree_chained) RBN_CHECK(pack_ternary(ctx, d_x, n, threshold, d_packed, &survivors, &nz_sum));
    } else if (!masked.ran)
        RBN_CHECK(strict_abs_sum(ctx, d_x, n, 1, threshold, &nz_sum, d_packed, &survivors));
    // quantization.rs:93-97
    float scale = 1.0f;
    if (survivors != 0) {
        volatile float sc = nz_sum / (float)survivors;
        scale = sc;
    }
    *h_scale = scale;
    *h_threshold = threshold;
    if (h_survivors) *h_survivors = survivors;
    return RBN_OK;
}

int rbn_dequantize_ternary(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t n, float scale,
                           float *d_out) {
    RBN_ENTER(ctx);
    if (n == 0) return RBN_OK;
    RBN_REQUIRE(d_packed && d_out, "null pointer in rbn_dequantize_ternary");
    uint64_t blocks = (n + kBlock - 1) / kBlock;
    if (blocks > 65536) blocks = 65536;
    dequantize_ternary_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream>>>(
        d_packed, n, scale, d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_unpack_ternary_i8(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t rows, uint64_t cols,
                          uint64_t pitch, int8_t *d_q, int32_t *d_rowsum) {
    RBN_ENTER(ctx);
    if (rows == 0) return RBN_OK;
    RBN_REQUIRE(d_packed && d_q, "null pointer in rbn_unpack_ternary_i8");
    RBN_REQUIRE(pitch >= cols && pitch > 0, "pitch %llu smaller than cols %llu",
                (unsigned long long)pitch, (unsigned long long)cols);
    RBN_REQUIRE(rows <= 0x7fffffffull, "too many rows");
    unpack_ternary_i8_kernel<<<dim3((unsigned)rows), dim3(kBlock), 0, ctx->stream>>>(
        d_packed, cols, pitch, d_q, d_rowsum);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_tile_weights(rbn_ctx *ctx, const uint8_t *d_packed, uint64_t K, uint64_t N,
                     uint32_t *d_tiled) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(K > 0 && N > 0, "K and N must be positive");
    RBN_REQUIRE(d_packed && d_tiled, "null pointer in rbn_tile_weights");
    RBN_REQUIRE(((uintptr_t)d_tiled & 15u) == 0, "d_tiled must be 16-byte aligned");
    uint64_t kblocks = rbn_kpad(K) / 16;
    uint64_t n_words = kblocks * rbn_npad(N);
    uint64_t blocks = (n_words + kBlock - 1) / kBlock;
    RBN_REQUIRE(blocks <= 0x7fffffffull, "weight matrix too large");
    tile_weights_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream>>>(
        d_packed, K, N, kblocks, n_words, d_tiled);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

}  // extern "C"

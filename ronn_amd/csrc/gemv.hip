// Decode-regime ternary GEMV: out[m,n] = ((float)acc * act_scale[m]) * w_scale with
// acc = sum_k q[m,k] * w[k,n] in int32, for M <= 16 tokens.
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (inner loop :161-165,
// epilogue :168).
//
// The kernel is bound by HBM.  Design, each point measured on an MI355X:
//  * One wavefront owns one quad of four adjacent columns.  In the tiled layout a
//    quad's weights are contiguous along k (16 bytes per 16 k), so every load
//    instruction of a wave reads 1 KiB of consecutive memory and a workgroup reads
//    a few consecutive KiB: the access pattern of a plain streaming read.
//  * Lanes split k.  The partial sums of a wave meet through six DPP additions
//    (quad_perm, row_ror, row_bcast); nothing crosses waves unless the matrix has too
//    few columns to fill the chip, in which case KS waves share a quad's k range and
//    meet through LDS.  Global memory is never used for partial sums.
//  * Activations are issued to the memory pipe BEFORE the weights (the vector-memory
//    counter retires in order) and staged in LDS once per workgroup, so the weight
//    stream is the only traffic of any size.
//  * Weights are stored as code = value + 1 in {0,1,2}.  Two VALU operations split a
//    word into two registers of eight 4-bit codes ((w & 0x33333333),
//    ((w >> 2) & 0x33333333)); the activations are staged as 4-bit planes
//    (a = 16 * hi + lo, hi signed, lo unsigned) so that v_dot8_i32_i4 and
//    v_dot8_u32_u4 consume them directly: 3 + 4 VALU operations per 16 weights
//    instead of 7 + 4 with byte-wise v_dot4.  sum q*w = sum q*code - sum q; the
//    per-token sum of q is subtracted once in the epilogue.  All of it is
//    integer-exact.
#include "common.hpp"
#include <hip/hip_ext.h>

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kLdsBudget = 48 * 1024;  // bytes of staged activations per workgroup

template <int CTRL, int ROWMASK>
__device__ __forceinline__ int dpp_add(int v) {
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROWMASK, 0xf, false);
}

// Sum over the 64 lanes of a wave; the total is valid in lane 63.
__device__ __forceinline__ int wave_total_lane63(int v) {
    v = dpp_add<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x124, 0xf>(v);  // row_ror:4
    v = dpp_add<0x128, 0xf>(v);  // row_ror:8   -> every lane holds its row's total
    v = dpp_add<0x142, 0xA>(v);  // row_bcast15 -> rows 1 and 3 add rows 0 and 2
    v = dpp_add<0x143, 0xC>(v);  // row_bcast31 -> rows 2 and 3 add row 1
    return v;
}

// int8 x16 (k = 0..15 of one 16-k block, natural order) -> the four 4-bit planes that
// pair with the even/odd 2-bit fields of a tiled weight word:
//   .x high nibbles, k order (0,8,1,9,2,10,3,11)   .y low nibbles, same order
//   .z high nibbles, k order (4,12,5,13,6,14,7,15) .w low nibbles, same order
__device__ __forceinline__ uint4 to_nibble_planes(uint4 a) {
    uint4 p;
    p.x = ((a.x >> 4) & 0x0F0F0F0Fu) | (a.z & 0xF0F0F0F0u);
    p.y = (a.x & 0x0F0F0F0Fu) | ((a.z & 0x0F0F0F0Fu) << 4);
    p.z = ((a.y >> 4) & 0x0F0F0F0Fu) | (a.w & 0xF0F0F0F0u);
    p.w = (a.y & 0x0F0F0F0Fu) | ((a.w & 0x0F0F0F0Fu) << 4);
    return p;
}

// Weights are read once per launch: a non-temporal load keeps them from being allocated in the
// caches on their way in (headline shape 4.32 -> 4.02 us, 8192 x 28672 12.0 -> 10.8 us).
__device__ __forceinline__ uint4 ld_w(const uint4 *p) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// MT tokens, KS waves per column quad, L weight loads in flight per lane and round.
// EXACT: the k-blocks fit one pass and are a multiple of 64 * L, so no index of the
// loop needs a clamp and no block a mask.
// `block` is the workgroup's index inside its problem (blockIdx.x for a single GEMV).
template <int MT, int KS, int L, bool EXACT>
__device__ __forceinline__ void gemv_body(
    const uint4 *__restrict__ q4,         // [M][KB]: 16 int8 each
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint4 *__restrict__ w4,         // [nquads][KB]
    float w_scale, int M, int KB, int KC /* k-blocks staged per pass */, int N, int nquads,
    int vec_store /* N % 4 == 0 and the outputs are 16-byte aligned */,
    int32_t *__restrict__ acc_out, float *__restrict__ out, const int block) {
    constexpr int QPB = kWaves / KS;  // quads per workgroup
    extern __shared__ uint4 s_a[];  // MT * KC staged activation blocks (4-bit planes)
    __shared__ int s_part[KS > 1 ? kWaves * MT * 4 : 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int quad_local = wave / KS, slice = wave % KS;
    int quad = block * QPB + quad_local;
    const bool active = quad < nquads;
    quad = active ? quad : nquads - 1;
    const uint4 *wq = w4 + (size_t)quad * KB;

    // epilogue scalars, fetched while the weights are in flight (spare token rows repeat the last)
    int rs_m[MT];
    float as_m[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        rs_m[m] = rowsum[min(m, M - 1)];
        as_m[m] = act_scale[min(m, M - 1)];
    }

    int hi[MT][4], lo[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            hi[m][c] = 0;
            lo[m][c] = 0;
        }

    for (int kc = 0; kc < KB; kc += KC) {
        const int kc_len = min(KC, KB - kc);
        // this wave's k range inside the pass
        const int sl_len = (kc_len + KS - 1) / KS;
        const int sl_lo = kc + slice * sl_len;
        const int sl_hi = min(sl_lo + sl_len, kc + kc_len);

        // (1) activations first, (2) the first round of weights, then the LDS hand-over.
        // Every load below is unconditional (indices are clamped, never branched on) so
        // that the compiler keeps them back to back and waits with vmcnt(L), not vmcnt(0).
        const int n_stage = MT * kc_len;  // uint4 entries: [m][kb - kc]
        constexpr int kPre = MT * KS * L / 4 < 1 ? 1 : (MT * KS * L / 4 > 4 ? 4 : MT * KS * L / 4);
        uint4 stage[kPre];
#pragma unroll
        for (int j = 0; j < kPre; ++j) {
            const int e = min(tid + j * kThreads, n_stage - 1);
            const int m = MT == 1 ? 0 : min(e / kc_len, M - 1);  // spare token rows repeat the last
            const int kb = kc + (MT == 1 ? e : e % kc_len);
            stage[j] = q4[(size_t)m * KB + kb];
        }
        __builtin_amdgcn_sched_barrier(0);
        uint4 w[L];
#pragma unroll
        for (int it = 0; it < L; ++it) {
            const int kb = sl_lo + it * 64 + lane;
            // a lane past its slice re-reads its first block (a cache hit) and adds 0
            w[it] = ld_w(wq + (EXACT || kb < sl_hi ? kb : min(sl_lo + lane, KB - 1)));
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kc != 0) __syncthreads();  // everyone is done reading the previous pass
#pragma unroll
        for (int j = 0; j < kPre; ++j) {
            const int e = tid + j * kThreads;
            if (e < n_stage) s_a[e] = to_nibble_planes(stage[j]);
        }
        for (int e = tid + kPre * kThreads; e < n_stage; e += kThreads) {
            const int m = min(e / kc_len, M - 1), kb = kc + e % kc_len;
            s_a[e] = to_nibble_planes(q4[(size_t)m * KB + kb]);
        }
        __syncthreads();

        // One round: expand L loaded blocks and accumulate.  Beyond the slice the codes are
        // forced to 0, so the lane adds q * 0.
        auto consume = [&](const uint4(&wr)[L], int r0) {
#pragma unroll
            for (int it = 0; it < L; ++it) {
                const int kb = r0 + it * 64 + lane;
                const uint32_t keep = EXACT || kb < sl_hi ? 0x33333333u : 0u;
                const int a_idx = EXACT ? kb : min(kb, sl_hi - 1) - kc;
                const uint32_t ww[4] = {wr[it].x, wr[it].y, wr[it].z, wr[it].w};
                uint32_t ev[4], od[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    ev[c] = ww[c] & keep;
                    od[c] = (ww[c] >> 2) & keep;
                }
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const uint4 a = s_a[m * kc_len + a_idx];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        hi[m][c] = __builtin_amdgcn_sdot8((int)a.x, (int)ev[c], hi[m][c], false);
                        lo[m][c] = (int)__builtin_amdgcn_udot8(a.y, ev[c], (uint32_t)lo[m][c], false);
                        hi[m][c] = __builtin_amdgcn_sdot8((int)a.z, (int)od[c], hi[m][c], false);
                        lo[m][c] = (int)__builtin_amdgcn_udot8(a.w, od[c], (uint32_t)lo[m][c], false);
                    }
                }
            }
        };
        // Rounds with a successor prefetch it before consuming; the last round has nothing
        // else in flight, so its blocks are consumed as they arrive (vmcnt L-1, L-2, ...).
        int r0 = sl_lo;
        while (r0 + 64 * L < sl_hi) {
            uint4 wn[L];
#pragma unroll
            for (int it = 0; it < L; ++it) {
                const int kb = r0 + 64 * L + it * 64 + lane;
                wn[it] = ld_w(wq + (EXACT || kb < sl_hi ? kb : min(sl_lo + lane, KB - 1)));
            }
            consume(w, r0);
#pragma unroll
            for (int it = 0; it < L; ++it) w[it] = wn[it];
            r0 += 64 * L;
        }
        if (r0 < sl_hi) consume(w, r0);
    }

    // wave totals (lane 63), then across the KS waves of a quad if any
    int tot[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) tot[m][c] = wave_total_lane63(hi[m][c] * 16 + lo[m][c]);

    if (KS == 1) {
        if (lane == 63 && active) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m >= M) break;
                const int rs = rs_m[m];
                const float as = as_m[m];
                if (vec_store) {
                    // one 16-byte store per token instead of four: the stores sit at the very end
                    // of the launch, where each instruction's round trip is exposed
                    int t4[4];
                    float r4[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        t4[c] = tot[m][c] - rs;
                        const float r = (float)t4[c] * as;  // kernels.rs:168, left to right
                        r4[c] = r * w_scale;
                    }
                    const size_t at = (size_t)m * N + (size_t)quad * 4;
                    if (quad * 4 < N) {  // quads of the column padding write nothing
                        if (acc_out) *(int4 *)(acc_out + at) = make_int4(t4[0], t4[1], t4[2], t4[3]);
                        *(float4 *)(out + at) = make_float4(r4[0], r4[1], r4[2], r4[3]);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int n = quad * 4 + c;
                        if (n < N) {
                            const int total = tot[m][c] - rs;
                            if (acc_out) acc_out[(size_t)m * N + n] = total;
                            float r = (float)total * as;  // kernels.rs:168, left to right
                            r = r * w_scale;
                            out[(size_t)m * N + n] = r;
                        }
                    }
                }
            }
        }
    } else {
        if (lane == 63) {
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int c = 0; c < 4; ++c) s_part[(wave * MT + m) * 4 + c] = tot[m][c];
        }
        __syncthreads();
        for (int idx = tid; idx < QPB * MT * 4; idx += kThreads) {
            const int ql = idx / (MT * 4), m = (idx / 4) % MT, c = idx % 4;
            const int qd = block * QPB + ql;
            const int n = qd * 4 + c;
            if (qd < nquads && m < M && n < N) {
                int total = 0;
#pragma unroll
                for (int s = 0; s < KS; ++s) total += s_part[((ql * KS + s) * MT + m) * 4 + c];
                total -= rowsum[m];
                if (acc_out) acc_out[(size_t)m * N + n] = total;
                float r = (float)total * act_scale[m];  // kernels.rs:168, left to right
                r = r * w_scale;
                out[(size_t)m * N + n] = r;
            }
        }
    }
}

template <int MT, int KS, int L, bool EXACT>
__global__ __launch_bounds__(kThreads) void gemv_t2_i8_kernel(
    const uint4 *__restrict__ q4, const float *__restrict__ act_scale, const int32_t *__restrict__ rowsum,
    const uint4 *__restrict__ w4, float w_scale, int M, int KB, int KC, int N, int nquads, int vec_store,
    int32_t *__restrict__ acc_out, float *__restrict__ out) {
    gemv_body<MT, KS, L, EXACT>(q4, act_scale, rowsum, w4, w_scale, M, KB, KC, N, nquads, vec_store, acc_out,
                                out, (int)blockIdx.x);
}

// Several independent GEMVs of one shape in one launch: workgroup b works on problem
// b / blocks_per_problem.  The problems' pointers travel in the kernel arguments (a workgroup
// reads its own with scalar loads), so nothing has to be uploaded before the launch.  Back to
// back in one grid the problems overlap: the next one's first loads are in flight while the
// previous one's last waves reduce and store, which a launch of its own cannot do.
struct GroupArgs {
    rbn_gemv_problem p[RBN_GEMV_GROUP_MAX];
};

template <int MT, int KS, int L, bool EXACT>
__global__ __launch_bounds__(kThreads) void gemv_t2_i8_grouped_kernel(
    const GroupArgs g, int blocks_per_problem, int M, int KB, int KC, int N, int nquads, int vec_store) {
    const int p = __builtin_amdgcn_readfirstlane((int)blockIdx.x / blocks_per_problem);
    const int block = (int)blockIdx.x - p * blocks_per_problem;
    const rbn_gemv_problem &d = g.p[p];
    gemv_body<MT, KS, L, EXACT>((const uint4 *)d.d_q, d.d_act_scale, d.d_rowsum, (const uint4 *)d.d_tiled,
                                d.w_scale, M, KB, KC, N, nquads, vec_store, d.d_acc, d.d_out, block);
}

struct Args {
    const GroupArgs *group = nullptr;  // set: a grouped launch of `count` problems
    int count = 1;
    const uint4 *q4;
    const float *act_scale;
    const int32_t *rowsum;
    const uint4 *w4;
    float w_scale;
    int M, KB, KC, N, nquads, vec_store;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    int32_t *acc;
    float *out;
};

template <int MT, int KS, int L>
void launch(hipStream_t stream, const Args &a) {
    constexpr int QPB = kWaves / KS;
    const int blocks = (a.nquads + QPB - 1) / QPB;
    dim3 grid((unsigned)blocks);
    const size_t lds = (size_t)MT * a.KC * 16;
    const bool exact = KS == 1 && MT <= 4 && a.KC == a.KB && a.KB % (64 * L) == 0;
    if (a.group) {
        dim3 ggrid((unsigned)(blocks * a.count));
        if constexpr (KS == 1 && MT <= 4) {
            if (exact) {
                gemv_t2_i8_grouped_kernel<MT, KS, L, true><<<ggrid, dim3(kThreads), lds, stream>>>(
                    *a.group, blocks, a.M, a.KB, a.KC, a.N, a.nquads, a.vec_store);
                return;
            }
        }
        gemv_t2_i8_grouped_kernel<MT, KS, L, false><<<ggrid, dim3(kThreads), lds, stream>>>(
            *a.group, blocks, a.M, a.KB, a.KC, a.N, a.nquads, a.vec_store);
        return;
    }
    // with events given the launch records the kernel's own begin and end timestamps in them
    auto go = [&](auto kernel) {
        if (a.ev_begin)
            hipExtLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, stream, a.ev_begin, a.ev_end, 0, a.q4,
                                  a.act_scale, a.rowsum, a.w4, a.w_scale, a.M, a.KB, a.KC, a.N, a.nquads,
                                  a.vec_store, a.acc, a.out);
        else
            kernel<<<grid, dim3(kThreads), lds, stream>>>(a.q4, a.act_scale, a.rowsum, a.w4, a.w_scale, a.M,
                                                         a.KB, a.KC, a.N, a.nquads, a.vec_store, a.acc, a.out);
    };
    if constexpr (KS == 1 && MT <= 4) {
        if (exact) {
            go(gemv_t2_i8_kernel<MT, KS, L, true>);
            return;
        }
    }
    go(gemv_t2_i8_kernel<MT, KS, L, false>);
}

template <int MT, int KS>
void launch_l(hipStream_t stream, const Args &a, int loads) {
    // one or two tokens with 8 to 15 loads per lane to cover a wave's share (K around 8192): all
    // eight in flight at once instead of two rounds of four (8192 x 28672: 12.6 -> 12.1 us; two
    // tokens at 8192 x 8192: 6.6 -> 6.0 us; with 16 and more, rounds of four stay ahead)
    if constexpr (MT <= 2) {
        if (loads >= 8 && loads < 16) {
            launch<MT, KS, 8>(stream, a);
            return;
        }
    }
    if (loads <= 1)
        launch<MT, KS, 1>(stream, a);
    else if (loads <= 2 || MT >= 8)
        launch<MT, KS, 2>(stream, a);
    else
        launch<MT, KS, 4>(stream, a);
}

template <int MT>
void launch_ks(hipStream_t stream, const Args &a, int ks) {
    // weight loads per lane needed to cover one wave's share of a pass
    const int sl_len = ((a.KC + ks - 1) / ks + 63) / 64;
    if (ks == 4)
        launch_l<MT, 4>(stream, a, sl_len);
    else if (ks == 2)
        launch_l<MT, 2>(stream, a, sl_len);
    else
        launch_l<MT, 1>(stream, a, sl_len);
}

}  // namespace

static void shape_and_launch(hipStream_t stream, Args &a);

static int gemv_impl(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale, const int32_t *d_rowsum,
                     const uint32_t *d_tiled, float w_scale, uint64_t M, uint64_t K, uint64_t N,
                     int32_t *d_acc, float *d_out, float *h_kernel_us) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(M > 0 && K > 0 && N > 0, "M, K and N must be positive");
    RBN_REQUIRE(M <= RBN_GEMV_MAX_M, "rbn_gemv_t2_i8 takes M <= %d (got %llu)", RBN_GEMV_MAX_M,
                (unsigned long long)M);
    RBN_REQUIRE(d_q && d_act_scale && d_rowsum && d_tiled && d_out, "null pointer in rbn_gemv_t2_i8");
    RBN_REQUIRE((((uintptr_t)d_q | (uintptr_t)d_tiled) & 15u) == 0,
                "d_q and d_tiled must be 16-byte aligned");
    RBN_REQUIRE(K <= (1ull << 30) && N <= (1ull << 30), "dimension too large");
    Args a;
    a.q4 = (const uint4 *)d_q;
    a.act_scale = d_act_scale;
    a.rowsum = d_rowsum;
    a.w4 = (const uint4 *)d_tiled;
    a.w_scale = w_scale;
    a.M = (int)M;
    a.KB = (int)(rbn_kpad(K) / 16);
    a.N = (int)N;
    a.nquads = (int)(rbn_npad(N) / 4);
    a.acc = d_acc;
    a.out = d_out;
    if (h_kernel_us) {
        a.ev_begin = ctx->ev_start;
        a.ev_end = ctx->ev_stop;
    }
    a.vec_store = N % 4 == 0 && (((uintptr_t)d_out | (uintptr_t)d_acc) & 15u) == 0;
    shape_and_launch(ctx->stream, a);
    RBN_HIP(hipGetLastError());
    if (h_kernel_us) {
        float ms = 0.0f;
        RBN_HIP(hipEventSynchronize(ctx->ev_stop));
        RBN_HIP(hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop));
        *h_kernel_us = ms * 1000.0f;
    }
    return RBN_OK;
}

// Picks the launch shape for a.M, a.KB, a.nquads (a.KC is set here) and launches.
static void shape_and_launch(hipStream_t stream, Args &a) {
    const int M = a.M;
    const int mt = M == 1 ? 1 : M == 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    // k-blocks whose staged activations fit the LDS budget in one pass
    const int kc_cap = kLdsBudget / 16 / mt;
    a.KC = a.KB < kc_cap ? a.KB : kc_cap;
    // Waves per quad: enough wavefronts to cover the chip (256 CUs x 4 SIMDs, a few waves
    // each) without shrinking a wave's share of k below one round.  One token tolerates
    // shorter shares than several (measured crossovers).
    int ks = 1;
    if (M == 1) {
        if (a.nquads <= 1024 && a.KB >= 640)
            ks = 4;
        else if (a.nquads <= 1024 && a.KB >= 320)
            ks = 2;
    } else {
        // (a share of 128-159 k-blocks only when the waves would otherwise be few)
        while (ks < 4 && (long long)a.nquads * ks < 2048 &&
               (a.KB / (ks * 2) >= 160 || (a.KB / (ks * 2) >= 128 && (long long)a.nquads * ks < 1024)))
            ks *= 2;
    }
    switch (mt) {
        case 1: launch_ks<1>(stream, a, ks); break;
        case 2: launch_ks<2>(stream, a, ks); break;
        case 4: launch_ks<4>(stream, a, ks); break;
        case 8: launch_ks<8>(stream, a, ks); break;
        default: launch_ks<16>(stream, a, ks); break;
    }
}

extern "C" int rbn_gemv_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                              const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                              uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out) {
    return gemv_impl(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc, d_out, nullptr);
}

extern "C" int rbn_gemv_t2_i8_kernel_time(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                          const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                                          uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out,
                                          float *h_kernel_us) {
    if (ctx && !h_kernel_us) {
        RBN_ENTER(ctx);
        return rbn_fail(RBN_ERR_INVALID, "h_kernel_us is NULL");
    }
    return gemv_impl(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc, d_out, h_kernel_us);
}

extern "C" int rbn_gemv_t2_i8_grouped(rbn_ctx *ctx, const rbn_gemv_problem *h_problems, uint64_t count,
                                      uint64_t M, uint64_t K, uint64_t N) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_problems != nullptr, "h_problems is NULL");
    RBN_REQUIRE(count >= 1 && count <= RBN_GEMV_GROUP_MAX, "rbn_gemv_t2_i8_grouped takes 1 to %d problems (got %llu)",
                RBN_GEMV_GROUP_MAX, (unsigned long long)count);
    RBN_REQUIRE(M > 0 && K > 0 && N > 0, "M, K and N must be positive");
    RBN_REQUIRE(M <= RBN_GEMV_MAX_M, "rbn_gemv_t2_i8_grouped takes M <= %d (got %llu)", RBN_GEMV_MAX_M,
                (unsigned long long)M);
    RBN_REQUIRE(K <= (1ull << 30) && N <= (1ull << 30), "dimension too large");
    GroupArgs g;
    bool vec = N % 4 == 0;
    for (uint64_t i = 0; i < count; ++i) {
        const rbn_gemv_problem &p = h_problems[i];
        RBN_REQUIRE(p.d_q && p.d_act_scale && p.d_rowsum && p.d_tiled && p.d_out,
                    "null pointer in problem %llu of rbn_gemv_t2_i8_grouped", (unsigned long long)i);
        RBN_REQUIRE((((uintptr_t)p.d_q | (uintptr_t)p.d_tiled) & 15u) == 0,
                    "d_q and d_tiled of problem %llu must be 16-byte aligned", (unsigned long long)i);
        vec = vec && (((uintptr_t)p.d_out | (uintptr_t)p.d_acc) & 15u) == 0;
        g.p[i] = p;
    }
    for (uint64_t i = count; i < RBN_GEMV_GROUP_MAX; ++i) g.p[i] = h_problems[count - 1];
    Args a;
    a.group = &g;
    a.count = (int)count;
    a.q4 = nullptr;
    a.act_scale = nullptr;
    a.rowsum = nullptr;
    a.w4 = nullptr;
    a.w_scale = 0.0f;
    a.M = (int)M;
    a.KB = (int)(rbn_kpad(K) / 16);
    a.N = (int)N;
    a.nquads = (int)(rbn_npad(N) / 4);
    a.acc = nullptr;
    a.out = nullptr;
    a.vec_store = vec;
    RBN_REQUIRE((uint64_t)a.nquads * count < (1ull << 31), "too many workgroups");
    shape_and_launch(ctx->stream, a);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

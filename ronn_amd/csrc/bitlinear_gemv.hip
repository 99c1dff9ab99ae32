// One-token BitLinear in a single launch: RMSNorm (optionally of SwiGLU(gate, up)), per-token
// absmax int8 quantisation, ternary GEMV, fused dequantisation, optional residual add.
//
//   v      = x                         or  silu(gate) * up
//   y      = (v * gamma) * rsqrt(mean(v^2) + eps)
//   g      = max(max|y|, 1e-5);  q = clamp(rne(y * (127/g)), -128, 127);  s = g / 127
//   out[n] = [residual[n] +] ((float)(sum_k q[k] * w[k,n]) * s) * w_scale
//
// The matmul and its epilogue are BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (epilogue order :168); the
// normalisation and the int8 activations have no counterpart in the reference.
//
// Why one launch: at one token every kernel of a decoder layer is a few microseconds and
// the gap between two dependent launches costs as much again, so the normalisation is
// recomputed by every workgroup of the GEMV (the row is a few KiB in L2) while its first
// weight loads are already in flight, instead of running as a launch of its own.  The GEMV
// part is the decode kernel of gemv.hip: one wave per column quad, lanes split k, 4-bit
// planes of the activations in LDS, v_dot8, DPP reduction.
#include "common.hpp"

namespace {

constexpr int kMaxK = 8192;  // activations staged in LDS: 16 bytes per 16 k

template <int CTRL, int ROWMASK>
__device__ __forceinline__ int dpp_add(int v) {
    return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROWMASK, 0xf, false);
}
// Sum over the 64 lanes of a wave; the total is valid in lane 63.
__device__ __forceinline__ int wave_total_lane63(int v) {
    v = dpp_add<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x124, 0xf>(v);  // row_ror:4
    v = dpp_add<0x128, 0xf>(v);  // row_ror:8
    v = dpp_add<0x142, 0xA>(v);  // row_bcast15
    v = dpp_add<0x143, 0xC>(v);  // row_bcast31
    return v;
}
// The same walk for floats (a fixed order, so every workgroup gets the same bits) and for
// the maximum of non-negative floats; lanes outside a step's row mask see 0.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROWMASK, 0xf, false));
}
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v += dpp_f<0xB1, 0xf>(v);
    v += dpp_f<0x4E, 0xf>(v);
    v += dpp_f<0x124, 0xf>(v);
    v += dpp_f<0x128, 0xf>(v);
    v += dpp_f<0x142, 0xA>(v);
    v += dpp_f<0x143, 0xC>(v);
    return v;
}
__device__ __forceinline__ float wave_max_lane63(float v) {  // v >= 0
    v = fmaxf(v, dpp_f<0xB1, 0xf>(v));
    v = fmaxf(v, dpp_f<0x4E, 0xf>(v));
    v = fmaxf(v, dpp_f<0x124, 0xf>(v));
    v = fmaxf(v, dpp_f<0x128, 0xf>(v));
    v = fmaxf(v, dpp_f<0x142, 0xA>(v));
    v = fmaxf(v, dpp_f<0x143, 0xC>(v));
    return v;
}

// int8 x16 (natural k order) -> the four 4-bit planes that pair with the even/odd 2-bit
// fields of a tiled weight word (see gemv.hip).
__device__ __forceinline__ uint4 to_nibble_planes(uint4 a) {
    uint4 p;
    p.x = ((a.x >> 4) & 0x0F0F0F0Fu) | (a.z & 0xF0F0F0F0u);
    p.y = (a.x & 0x0F0F0F0Fu) | ((a.z & 0x0F0F0F0Fu) << 4);
    p.z = ((a.y >> 4) & 0x0F0F0F0Fu) | (a.w & 0xF0F0F0F0u);
    p.w = (a.y & 0x0F0F0F0Fu) | ((a.w & 0x0F0F0F0Fu) << 4);
    return p;
}

// Weights are read once per launch: non-temporal loads (see gemv.hip).
__device__ __forceinline__ uint4 ld_w(const uint4 *p) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// KS waves per column quad, L weight loads in flight per lane and round, SWIGLU input,
// W waves per workgroup, NB blocks of 16 activations per thread (K <= 1024 * W * NB).
template <int KS, int L, bool SWIGLU, int W, int NB>
__global__ __launch_bounds__(W * 64) void bitlinear_gemv_kernel(
    const float *__restrict__ x,        // [K], or gate|up [2K] with SWIGLU
    const float *__restrict__ gamma,    // [K]
    float eps, const uint4 *__restrict__ w4,  // [nquads][KB]
    float w_scale, int K, int KB, int N, int nquads,
    int vec /* N % 4 == 0, residual and out 16-byte aligned */, const float *residual, float *out) {
    constexpr int kWaves = W, kThreads = W * 64;
    constexpr int QPB = kWaves / KS;
    extern __shared__ uint4 s_a[];  // KB staged activation blocks (4-bit planes)
    __shared__ float s_ss[kWaves], s_mx[kWaves];
    __shared__ int s_redi[kWaves];
    __shared__ int s_part[KS > 1 ? kWaves * 4 : 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int quad_local = wave / KS, slice = wave % KS;
    int quad = blockIdx.x * QPB + quad_local;
    const bool active = quad < nquads;
    quad = active ? quad : nquads - 1;
    const uint4 *wq = w4 + (size_t)quad * KB;
    const int kreal = K >> 4;  // K % 16 == 0: blocks that hold activations (the rest is padding)

    // this wave's k range
    const int sl_len = (KB + KS - 1) / KS;
    const int sl_lo = slice * sl_len;
    const int sl_hi = min(sl_lo + sl_len, KB);

    // (1) the row and the gains, (2) the first round of weights: all loads unconditional
    // (indices clamped), back to back
    float v[NB][16], gm[NB][16];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int kb = min(tid + b * kThreads, kreal - 1);
        const float4 *xr = reinterpret_cast<const float4 *>(x) + kb * 4;
        const float4 *gr = reinterpret_cast<const float4 *>(gamma) + kb * 4;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float4 a = xr[c], g4 = gr[c];
            v[b][4 * c] = a.x, v[b][4 * c + 1] = a.y, v[b][4 * c + 2] = a.z, v[b][4 * c + 3] = a.w;
            gm[b][4 * c] = g4.x, gm[b][4 * c + 1] = g4.y, gm[b][4 * c + 2] = g4.z, gm[b][4 * c + 3] = g4.w;
        }
        if (SWIGLU) {
            const float4 *ur = reinterpret_cast<const float4 *>(x + K) + kb * 4;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float4 u = ur[c];
                const float uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float g = v[b][4 * c + e];
                    v[b][4 * c + e] = (g / (1.0f + __expf(-g))) * uu[e];
                }
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 w[L];
#pragma unroll
    for (int it = 0; it < L; ++it) {
        const int kb = sl_lo + it * 64 + lane;
        w[it] = ld_w(wq + (kb < sl_hi ? kb : min(sl_lo + lane, KB - 1)));
    }
    // The residual the epilogue adds, requested behind the weights (one broadcast read per
    // wave) instead of at the very end, where its round trip would be exposed.
    float4 res4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float res1 = 0.0f;
    if (residual) {
        if (KS == 1) {
            if (vec) res4 = *reinterpret_cast<const float4 *>(residual + (size_t)min(quad * 4, N - 4));
        } else if (tid < QPB * 4) {
            res1 = residual[min((int)blockIdx.x * QPB * 4 + tid, N - 1)];
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // One pass gives both statistics: sum v^2, and max |v * gamma| - rounding is monotone, so
    // max_k |fl(t_k * r)| = fl(max_k |t_k| * r) for the positive factor r = inv_rms.  Every
    // workgroup computes the same values in the same order.
    float ss = 0.0f, mx = 0.0f;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const bool mine = tid + b * kThreads < kreal;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float a = mine ? v[b][e] : 0.0f;
            ss += a * a;
            v[b][e] = a * gm[b][e];
            mx = fmaxf(mx, fabsf(v[b][e]));
        }
    }
    ss = wave_sum_lane63(ss);
    mx = wave_max_lane63(mx);
    if (lane == 63) {
        s_ss[wave] = ss;
        s_mx[wave] = mx;
    }
    __syncthreads();
    ss = 0.0f, mx = 0.0f;
#pragma unroll
    for (int i = 0; i < kWaves; i += 4) {
        ss += (s_ss[i] + s_ss[i + 1]) + (s_ss[i + 2] + s_ss[i + 3]);
        mx = fmaxf(mx, fmaxf(fmaxf(s_mx[i], s_mx[i + 1]), fmaxf(s_mx[i + 2], s_mx[i + 3])));
    }
    const float inv_rms = 1.0f / sqrtf(ss / (float)K + eps);
    const float gmax = fmaxf(mx * inv_rms, 1e-5f);
    const float inv = 127.0f / gmax;
    const float act_scale = gmax / 127.0f;
    int qsum = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int kb = tid + b * kThreads;
        uint32_t pk[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t word = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float y = v[b][4 * c + e] * inv_rms;
                float r = rintf(y * inv);  // round half to even
                r = fminf(fmaxf(r, -128.0f), 127.0f);
                const int qi = (int)r;
                qsum += qi;
                word |= (uint32_t)(qi & 0xff) << (8 * e);
            }
            pk[c] = word;
        }
        if (kb < KB) s_a[kb] = to_nibble_planes(make_uint4(pk[0], pk[1], pk[2], pk[3]));  // zeros in the padding
    }
    qsum = wave_total_lane63(qsum);
    if (lane == 63) s_redi[wave] = qsum;
    __syncthreads();
    int rowsum = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) rowsum += s_redi[i];

    int hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
    auto consume = [&](const uint4(&wr)[L], int r0) {
#pragma unroll
        for (int it = 0; it < L; ++it) {
            const int kb = r0 + it * 64 + lane;
            const uint32_t keep = kb < sl_hi ? 0x33333333u : 0u;
            const uint4 a = s_a[min(kb, sl_hi - 1)];
            const uint32_t ww[4] = {wr[it].x, wr[it].y, wr[it].z, wr[it].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t ev = ww[c] & keep, od = (ww[c] >> 2) & keep;
                hi[c] = __builtin_amdgcn_sdot8((int)a.x, (int)ev, hi[c], false);
                lo[c] = (int)__builtin_amdgcn_udot8(a.y, ev, (uint32_t)lo[c], false);
                hi[c] = __builtin_amdgcn_sdot8((int)a.z, (int)od, hi[c], false);
                lo[c] = (int)__builtin_amdgcn_udot8(a.w, od, (uint32_t)lo[c], false);
            }
        }
    };
    int r0 = sl_lo;
    while (r0 + 64 * L < sl_hi) {
        uint4 wn[L];
#pragma unroll
        for (int it = 0; it < L; ++it) {
            const int kb = r0 + 64 * L + it * 64 + lane;
            wn[it] = ld_w(wq + (kb < sl_hi ? kb : min(sl_lo + lane, KB - 1)));
        }
        consume(w, r0);
#pragma unroll
        for (int it = 0; it < L; ++it) w[it] = wn[it];
        r0 += 64 * L;
    }
    if (r0 < sl_hi) consume(w, r0);

    int tot[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) tot[c] = wave_total_lane63(hi[c] * 16 + lo[c]);

    auto value = [&](int total) {
        total -= rowsum;
        const float r = (float)total * act_scale;  // kernels.rs:168, left to right
        return r * w_scale;
    };
    if (KS == 1) {
        if (lane == 63 && active) {
            if (vec) {
                // one 16-byte store: the stores end the launch, every instruction's round trip counts
                if (quad * 4 < N) {  // quads of the column padding write nothing
                    float4 r = make_float4(value(tot[0]), value(tot[1]), value(tot[2]), value(tot[3]));
                    if (residual) r = make_float4(res4.x + r.x, res4.y + r.y, res4.z + r.z, res4.w + r.w);
                    *reinterpret_cast<float4 *>(out + (size_t)quad * 4) = r;
                }
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int n = quad * 4 + c;
                    if (n < N) {
                        const float r = value(tot[c]);
                        out[n] = residual ? residual[n] + r : r;
                    }
                }
            }
        }
    } else {
        if (lane == 63) {
#pragma unroll
            for (int c = 0; c < 4; ++c) s_part[wave * 4 + c] = tot[c];
        }
        __syncthreads();
        if (tid < QPB * 4) {
            const int ql = tid >> 2, c = tid & 3;
            const int qd = blockIdx.x * QPB + ql, n = qd * 4 + c;
            if (qd < nquads && n < N) {
                int total = 0;
#pragma unroll
                for (int s = 0; s < KS; ++s) total += s_part[(ql * KS + s) * 4 + c];
                const float r = value(total);
                out[n] = residual ? res1 + r : r;
            }
        }
    }
}

struct Args {
    const float *x, *gamma;
    float eps;
    const uint4 *w4;
    float w_scale;
    int K, KB, N, nquads, vec;
    const float *residual;
    float *out;
};

template <int KS, int L, bool SWIGLU, int W>
void launch_w(hipStream_t stream, const Args &a) {
    constexpr int QPB = W / KS;
    dim3 grid((unsigned)((a.nquads + QPB - 1) / QPB));
    if (a.K <= 1024 * W)
        bitlinear_gemv_kernel<KS, L, SWIGLU, W, 1><<<grid, dim3(W * 64), (size_t)a.KB * 16, stream>>>(
            a.x, a.gamma, a.eps, a.w4, a.w_scale, a.K, a.KB, a.N, a.nquads, a.vec, a.residual, a.out);
    else
        bitlinear_gemv_kernel<KS, L, SWIGLU, W, 2><<<grid, dim3(W * 64), (size_t)a.KB * 16, stream>>>(
            a.x, a.gamma, a.eps, a.w4, a.w_scale, a.K, a.KB, a.N, a.nquads, a.vec, a.residual, a.out);
}

template <int KS, int L, bool SWIGLU>
void launch(hipStream_t stream, const Args &a) {
    // Every workgroup repeats the normalisation of the whole row: eight waves halve that
    // work per thread and the number of workgroups re-reading the row.  It pays for long
    // rows (K > 4096: one block per thread again; 6912 x 2560 8.3 -> 5.6 us); at K = 2560
    // four waves are faster whatever the width (a decode step with 2560 x 13824 and
    // 2560 x 32000 on eight waves: 0.737 ms, on four: 0.731 ms).
    if (a.K > 4096)
        launch_w<KS, L, SWIGLU, 8>(stream, a);
    else
        launch_w<KS, L, SWIGLU, 4>(stream, a);
}

template <int KS, bool SWIGLU>
void launch_l(hipStream_t stream, const Args &a) {
    const int loads = ((a.KB + KS - 1) / KS + 63) / 64;  // per lane, to cover a wave's share
    if (loads <= 1)
        launch<KS, 1, SWIGLU>(stream, a);
    else if (loads <= 2)
        launch<KS, 2, SWIGLU>(stream, a);
    else
        launch<KS, 4, SWIGLU>(stream, a);
}

template <bool SWIGLU>
void launch_ks(hipStream_t stream, const Args &a) {
    // waves per quad: as in the plain GEMV, enough wavefronts for the chip without
    // shrinking a wave's share of k below one round
    int ks = 1;
    while (ks < 4 && (long long)a.nquads * ks < 2048 && a.KB / (ks * 2) >= 128) ks *= 2;
    if (ks == 4)
        launch_l<4, SWIGLU>(stream, a);
    else if (ks == 2)
        launch_l<2, SWIGLU>(stream, a);
    else
        launch_l<1, SWIGLU>(stream, a);
}

}  // namespace

extern "C" int rbn_bitlinear_gemv_f32(rbn_ctx *ctx, const float *d_x, const float *d_gate_up,
                                      const float *d_gamma, float eps, const uint32_t *d_tiled,
                                      float w_scale, uint64_t K, uint64_t N, const float *d_residual,
                                      float *d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE((d_x != nullptr) != (d_gate_up != nullptr),
                "rbn_bitlinear_gemv_f32 takes either d_x or d_gate_up");
    RBN_REQUIRE(d_gamma && d_tiled && d_out, "null pointer in rbn_bitlinear_gemv_f32");
    RBN_REQUIRE(K >= 16 && K % 16 == 0 && K <= (uint64_t)kMaxK,
                "rbn_bitlinear_gemv_f32 takes K %% 16 == 0, 16 <= K <= %d (got %llu)", kMaxK,
                (unsigned long long)K);
    RBN_REQUIRE(N > 0 && N <= (1ull << 30), "bad N in rbn_bitlinear_gemv_f32");
    const float *src = d_x ? d_x : d_gate_up;
    RBN_REQUIRE((((uintptr_t)src | (uintptr_t)d_gamma | (uintptr_t)d_tiled) & 15u) == 0,
                "inputs must be 16-byte aligned");
    Args a;
    a.x = src;
    a.gamma = d_gamma;
    a.eps = eps;
    a.w4 = (const uint4 *)d_tiled;
    a.w_scale = w_scale;
    a.K = (int)K;
    a.KB = (int)(rbn_kpad(K) / 16);
    a.N = (int)N;
    a.nquads = (int)(rbn_npad(N) / 4);
    a.residual = d_residual;
    a.out = d_out;
    a.vec = N % 4 == 0 && (((uintptr_t)d_residual | (uintptr_t)d_out) & 15u) == 0;
    if (d_gate_up)
        launch_ks<true>(ctx->stream, a);
    else
        launch_ks<false>(ctx->stream, a);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

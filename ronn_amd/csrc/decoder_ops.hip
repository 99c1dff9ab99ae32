// Building blocks of a BitNet-style decoder around the ternary matmuls: embedding lookup,
// RMSNorm fused with the per-token int8 quantisation (and the residual add), rotary
// embedding + f16 K/V cache store, attention over the f16 cache, SwiGLU, arg-max.
//
// None of this exists in the reference (crates/ronn-providers/src/bitnet/ holds only the
// quantiser, the matmul kernels and the provider); the formulas are the usual LLaMA /
// BitNet-b1.58 ones and are pinned by the numpy model in tests/decoder_model.py.
// Everything is stream-ordered and takes the current position from device memory, so a
// whole decode step can be captured once in a HIP graph and replayed.
#include <hip/hip_fp16.h>

#include "common.hpp"

namespace {

constexpr int kBlock = 256;

// Wave-wide reductions on the DPP cross-lane path (a few cycles per step, against a trip
// through the LDS crossbar for a shuffle): quad_perm, row_ror within rows of 16 lanes,
// row_bcast across rows; the total arrives in lane 63 and is read back as a wave-uniform
// value.  Lanes outside a step's row mask see `old`.  All 64 lanes must be active.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ int dpp_i(int old, int v) {
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROWMASK, 0xf, false);
}
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_f(float old, float v) {
    return __int_as_float(dpp_i<CTRL, ROWMASK>(__float_as_int(old), __float_as_int(v)));
}
__device__ __forceinline__ float wave_sum_f(float v) {
    v += dpp_f<0xB1, 0xf>(0.0f, v);   // quad_perm [1,0,3,2]
    v += dpp_f<0x4E, 0xf>(0.0f, v);   // quad_perm [2,3,0,1]
    v += dpp_f<0x124, 0xf>(0.0f, v);  // row_ror:4
    v += dpp_f<0x128, 0xf>(0.0f, v);  // row_ror:8
    v += dpp_f<0x142, 0xA>(0.0f, v);  // row_bcast15
    v += dpp_f<0x143, 0xC>(0.0f, v);  // row_bcast31
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ float wave_max_f(float v) {
    v = fmaxf(v, dpp_f<0xB1, 0xf>(v, v));
    v = fmaxf(v, dpp_f<0x4E, 0xf>(v, v));
    v = fmaxf(v, dpp_f<0x124, 0xf>(v, v));
    v = fmaxf(v, dpp_f<0x128, 0xf>(v, v));
    v = fmaxf(v, dpp_f<0x142, 0xA>(v, v));
    v = fmaxf(v, dpp_f<0x143, 0xC>(v, v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ int wave_sum_i(int v) {
    v += dpp_i<0xB1, 0xf>(0, v);
    v += dpp_i<0x4E, 0xf>(0, v);
    v += dpp_i<0x124, 0xf>(0, v);
    v += dpp_i<0x128, 0xf>(0, v);
    v += dpp_i<0x142, 0xA>(0, v);
    v += dpp_i<0x143, 0xC>(0, v);
    return __builtin_amdgcn_readlane(v, 63);
}

// x[m, :] = table[tokens[m], :]
__global__ __launch_bounds__(kBlock) void embed_kernel(const float *__restrict__ table,
                                                       const int32_t *__restrict__ tokens, int H,
                                                       int vocab, float *__restrict__ x) {
    const int m = blockIdx.x;
    int tok = tokens[m];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    const float *src = table + (size_t)tok * H;
    for (int i = threadIdx.x; i < H; i += kBlock) x[(size_t)m * H + i] = src[i];
}

// One workgroup of 1024 threads per token:
//   x = silu(gate) * up   when gate_up is given (SwiGLU computed on the way in), else
//   x += delta            when delta is given (written back: the residual stream)
//   y = (x * gamma) * rsqrt(mean(x^2) + eps)
//   g = max(max|y|, 1e-5); q = clamp(rne(y * (127/g)), -128, 127); scale = g/127; rowsum = sum q
// With one token the kernel is a chain of memory round trips, so every load (row, delta,
// gains) is issued before the first reduction and the row stays in registers.
constexpr int kNormThreads = 1024;
constexpr int kPer = 8;  // H <= 8192
__global__ __launch_bounds__(kNormThreads) void rmsnorm_quant_kernel(
    float *__restrict__ x, const float *__restrict__ delta, const float *__restrict__ gate_up,
    const float *__restrict__ gamma, float eps, int H, int pitch, int8_t *__restrict__ q,
    float *__restrict__ act_scale, int32_t *__restrict__ rowsum) {
    __shared__ float s_red[kNormThreads / 64], s_redm[kNormThreads / 64];
    __shared__ int s_redi[kNormThreads / 64];
    const int m = blockIdx.x, tid = threadIdx.x;
    float v[kPer], gm[kPer];
    if (gate_up) {
        const float *gu = gate_up + (size_t)m * 2 * H;
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int i = tid + j * kNormThreads;
            const float g = i < H ? gu[i] : 0.0f, u = i < H ? gu[H + i] : 0.0f;
            gm[j] = i < H ? gamma[i] : 0.0f;
            v[j] = (g / (1.0f + __expf(-g))) * u;
        }
    } else {
        float *row = x + (size_t)m * H;
        const float *drow = delta ? delta + (size_t)m * H : nullptr;
        float dv[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int i = tid + j * kNormThreads;
            v[j] = i < H ? row[i] : 0.0f;
            dv[j] = (drow && i < H) ? drow[i] : 0.0f;
            gm[j] = i < H ? gamma[i] : 0.0f;
        }
        if (drow) {
#pragma unroll
            for (int j = 0; j < kPer; ++j) {
                const int i = tid + j * kNormThreads;
                v[j] += dv[j];
                if (i < H) row[i] = v[j];
            }
        }
    }
    // one pass for both statistics: sum x^2 and max |x * gamma| (rounding is monotone, so
    // max_k |fl(t_k * r)| = fl(max_k |t_k| * r) for r = inv_rms > 0)
    float ss = 0.0f, mx = 0.0f;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        ss += v[j] * v[j];
        v[j] *= gm[j];
        mx = fmaxf(mx, fabsf(v[j]));
    }
    ss = wave_sum_f(ss);
    mx = wave_max_f(mx);
    if ((tid & 63) == 0) {
        s_red[tid >> 6] = ss;
        s_redm[tid >> 6] = mx;
    }
    __syncthreads();
    ss = 0.0f, mx = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormThreads / 64; ++w) {
        ss += s_red[w];
        mx = fmaxf(mx, s_redm[w]);
    }
    const float inv_rms = 1.0f / sqrtf(ss / (float)H + eps);
    const float gmax = fmaxf(mx * inv_rms, 1e-5f);
#pragma unroll
    for (int j = 0; j < kPer; ++j) v[j] *= inv_rms;
    const float inv = 127.0f / gmax;
    int sum = 0;
    int8_t *qrow = q + (size_t)m * pitch;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
        const int i = tid + j * kNormThreads;
        if (i < pitch) {
            float r = rintf(v[j] * inv);  // round half to even; v is 0 in the padding
            r = fminf(fmaxf(r, -128.0f), 127.0f);
            qrow[i] = (int8_t)(int)r;
            sum += (int)r;
        }
    }
    sum = wave_sum_i(sum);
    if ((tid & 63) == 0) s_redi[tid >> 6] = sum;
    __syncthreads();
    if (tid == 0) {
        int tot = 0;
#pragma unroll
        for (int w = 0; w < kNormThreads / 64; ++w) tot += s_redi[w];
        act_scale[m] = gmax / 127.0f;
        rowsum[m] = tot;
    }
}

// qkv: [M][3 * heads * hd] f32 (q | k | v).  Rotates q in place by the angle
// pos * theta^(-2i/hd) on the pairs (i, i + hd/2), rotates k the same way on its way into
// the cache, and stores k and v as f16 at position pos = *pos0 + m of the caches
// [heads][max_seq][hd].
__global__ __launch_bounds__(kBlock) void rope_kv_store_kernel(
    float *__restrict__ qkv, const int32_t *__restrict__ pos0, int heads, int hd, float theta,
    __half *__restrict__ kcache, __half *__restrict__ vcache, int max_seq) {
    const int m = blockIdx.x;
    const int pos = pos0[0] + m;
    const int HD = heads * hd, half = hd >> 1;
    float *qrow = qkv + (size_t)m * 3 * HD;
    // A thread keeps one pair index i (its angle is computed once) and walks the heads:
    // `groups` threads share an i and take every groups-th head.
    const int groups = kBlock >= half ? kBlock / half : 1;
    const int group = kBlock >= half ? (int)threadIdx.x / half : 0;
    if (group >= groups) return;  // left-over threads when half does not divide the block
    for (int i = (int)threadIdx.x % half; i < half; i += kBlock) {  // one pass unless half > kBlock
        const float freq = powf(theta, -2.0f * (float)i / (float)hd);
        float sn, cs;
        sincosf((float)pos * freq, &sn, &cs);
        for (int h = group; h < heads; h += groups) {
            float *qh = qrow + h * hd, *kh = qrow + HD + h * hd;
            const float *vh = qrow + 2 * HD + h * hd;
            const float q0 = qh[i], q1 = qh[i + half];
            qh[i] = q0 * cs - q1 * sn;
            qh[i + half] = q1 * cs + q0 * sn;
            const float k0 = kh[i], k1 = kh[i + half];
            const float r0 = k0 * cs - k1 * sn, r1 = k1 * cs + k0 * sn;
            if (pos < max_seq) {
                const size_t c = ((size_t)h * max_seq + pos) * hd;
                kcache[c + i] = __float2half_rn(r0);
                kcache[c + i + half] = __float2half_rn(r1);
                vcache[c + i] = __float2half_rn(vh[i]);
                vcache[c + i + half] = __float2half_rn(vh[i + half]);
            }
        }
    }
}

// Attention of token m (position p = *pos0 + m) and head h over cache positions 0..p.
// One workgroup per (m, h); hd == 128.  Each wave takes every kWaves-th block of 64 keys:
// scores with one key per lane (the key row is read as 16 x 16 bytes), online softmax,
// then P.V with two dimensions per lane; the waves' (max, sum, out) meet through LDS.
template <int kWaves>
__global__ __launch_bounds__(kWaves * 64) void attention_kernel(
    const float *__restrict__ qkv, const int32_t *__restrict__ pos0, int heads,
    const __half *__restrict__ kcache, const __half *__restrict__ vcache, int max_seq,
    float *__restrict__ out) {
    constexpr int hd = 128;
    __shared__ float s_q[hd];
    __shared__ float s_p[kWaves][64];
    __shared__ float s_m[kWaves], s_l[kWaves];
    __shared__ float s_o[kWaves][hd];
    const int m = blockIdx.x / heads, h = blockIdx.x - m * heads;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int HD = heads * hd;
    int p = pos0[0] + m;
    if (p >= max_seq) p = max_seq - 1;
    const int nkeys = p + 1;
    const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
    if (tid < hd) s_q[tid] = qkv[(size_t)m * 3 * HD + h * hd + tid] * scale;
    __syncthreads();

    const __half *kh = kcache + (size_t)h * max_seq * hd;
    const __half *vh = vcache + (size_t)h * max_seq * hd;
    float run_max = -INFINITY, run_sum = 0.0f, o0 = 0.0f, o1 = 0.0f;
    for (int t0 = wave * 64; t0 < nkeys; t0 += kWaves * 64) {
        // One round trip per block: the lane's key row (16 x 16 bytes) and its two columns
        // of all 64 value rows are requested together; rows past the end repeat the last
        // one and get probability 0.
        const int last = nkeys - 1 - t0;  // >= 0
        const int t = t0 + min(lane, last);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kh + (size_t)t * hd);
        uint4 kr[hd / 8];
#pragma unroll
        for (int c = 0; c < hd / 8; ++c) kr[c] = krow[c];
        __half2 vr[64];
#pragma unroll
        for (int j = 0; j < 64; ++j)
            vr[j] = *reinterpret_cast<const __half2 *>(vh + (size_t)(t0 + min(j, last)) * hd + 2 * lane);
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < hd / 8; ++c) {
            const __half2 *h2 = reinterpret_cast<const __half2 *>(&kr[c]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float2 f = __half22float2(h2[e]);
                acc = fmaf(f.x, s_q[c * 8 + 2 * e], acc);
                acc = fmaf(f.y, s_q[c * 8 + 2 * e + 1], acc);
            }
        }
        const float s = lane <= last ? acc : -INFINITY;
        const float blk_max = wave_max_f(s);
        const float new_max = fmaxf(run_max, blk_max);
        const float corr = __expf(run_max - new_max);  // 0 on the first block
        const float pr = lane <= last ? __expf(s - new_max) : 0.0f;
        run_sum = run_sum * corr + wave_sum_f(pr);
        run_max = new_max;
        o0 *= corr;
        o1 *= corr;
        s_p[wave][lane] = pr;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            const float pj = s_p[wave][j];
            const float2 v = __half22float2(vr[j]);
            o0 = fmaf(pj, v.x, o0);
            o1 = fmaf(pj, v.y, o1);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if (lane == 0) {
        s_m[wave] = run_max;
        s_l[wave] = run_sum;
    }
    s_o[wave][2 * lane] = o0;
    s_o[wave][2 * lane + 1] = o1;
    __syncthreads();
    if (tid < hd) {
        float gmax = -INFINITY;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) gmax = fmaxf(gmax, s_m[w]);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float c = s_m[w] == -INFINITY ? 0.0f : __expf(s_m[w] - gmax);
            num += c * s_o[w][tid];
            den += c * s_l[w];
        }
        out[(size_t)m * HD + h * hd + tid] = num / den;
    }
}

// Attention of a prompt on the f16 matrix cores: one workgroup per (block of 32 tokens, head),
// its four waves take every fourth block of 32 keys, keep an online softmax each and meet
// through LDS at the end.  hd == 128.
//  * Scores transposed, S^T = K . Q^T (v_mfma_f32_32x32x16_f16, A = 32 keys x 16 dims read as
//    one 16-byte piece of a key row per lane, B = Q^T): a lane then holds ONE token (column
//    lane % 32) and 16 of the 32 keys, so the softmax is lane-local but for one exchange with
//    lane ^ 32.  The same lane layout comes out of O^T = V^T . P^T, so the running rescale of
//    O is lane-local too, and P^T is already in B-operand form: MFMA step s multiplies the
//    lane's own probabilities 8s .. 8s+7, i.e. keys 8(2s + e/4) + 4(lane/32) + e%4.
//  * V^T . P^T needs values with the key index contiguous per lane: the wave stages its 32
//    value rows in LDS (row pitch 136 halves: the two lane halves read rows four apart, on
//    disjoint banks) and gathers the eight keys of a slot set with 16-bit reads.
//  * f32-grade accuracy from f16 matrix cores: K and V are f16 already; q (scaled) and the
//    probabilities go in as hi + lo f16 pairs, two MFMAs each, accumulated in f32.
//  * Rows past the last key of the prompt are never loaded (indices clamp to it: everything
//    up to there has been written), so masked keys multiply finite values by zero.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int kVPitch = 136;  // halves per staged value row
__global__ __launch_bounds__(256) void attention_mfma_kernel(
    const float *__restrict__ qkv, const int32_t *__restrict__ pos0, int M, int heads,
    const __half *__restrict__ kcache, const __half *__restrict__ vcache, int max_seq,
    float *__restrict__ out) {
    constexpr int hd = 128;
    __shared__ __attribute__((aligned(16))) _Float16 s_v[4][32 * kVPitch];  // later: the exchange
    __shared__ float s_ml[4][2][64];
    const int nqb = (M + 31) >> 5;
    const int qb = nqb - 1 - (int)(blockIdx.x / heads);  // the long blocks first
    const int h = blockIdx.x % heads;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, g = lane >> 5;
    const int HD = heads * hd;
    const int p0 = pos0[0];
    const int m = min(qb * 32 + j, M - 1);            // this lane's token (clamped: never stored twice)
    const int pj = min(p0 + m, max_seq - 1);          // its position = its last key
    const int last_key = min(p0 + M - 1, max_seq - 1);  // last row of the caches that is known to be written
    const int blk_keys = min(p0 + qb * 32 + 31, last_key) + 1;
    const int nkb = (blk_keys + 31) >> 5;

    // Q^T operand: dims 16 kk + 8 g + e of token j, scaled, as f16 hi + lo
    v8h qhi[8], qlo[8];
    {
        const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
        const float *qrow = qkv + (size_t)m * 3 * HD + h * hd + 8 * g;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const float4 a = *reinterpret_cast<const float4 *>(qrow + 16 * kk);
            const float4 b = *reinterpret_cast<const float4 *>(qrow + 16 * kk + 4);
            const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float v = f[e] * scale;
                const _Float16 hi = (_Float16)v;
                qhi[kk][e] = hi;
                qlo[kk][e] = (_Float16)(v - (float)hi);
            }
        }
    }

    const __half *kh = kcache + (size_t)h * max_seq * hd;
    const __half *vh = vcache + (size_t)h * max_seq * hd;
    _Float16 *sv = s_v[wave];
    float run_max = -INFINITY, run_sum = 0.0f;
    v16f ot[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) ot[nt][r] = 0.0f;

    for (int kb = wave; kb < nkb; kb += 4) {
        const int t0 = kb * 32;
        // key rows (A operand of the scores) and the staging of the value rows
        const uint4 *krow = reinterpret_cast<const uint4 *>(kh + (size_t)min(t0 + j, last_key) * hd + 8 * g);
        uint4 kr[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) kr[kk] = krow[2 * kk];
        uint4 vstage[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int idx = c * 64 + lane, row = idx >> 4, col = idx & 15;
            vstage[c] = *reinterpret_cast<const uint4 *>(vh + (size_t)min(t0 + row, last_key) * hd + 8 * col);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int idx = c * 64 + lane, row = idx >> 4, col = idx & 15;
            *reinterpret_cast<uint4 *>(sv + row * kVPitch + 8 * col) = vstage[c];
        }
        // S^T: keys 8b + 4g + r (register 4b + r) of token j
        v16f st;
#pragma unroll
        for (int r = 0; r < 16; ++r) st[r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const v8h ka = __builtin_bit_cast(v8h, kr[kk]);
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qhi[kk], st, 0, 0, 0);
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka, qlo[kk], st, 0, 0, 0);
        }
        float blk_max = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int t = t0 + 8 * (r >> 2) + 4 * g + (r & 3);
            st[r] = t <= pj ? st[r] : -INFINITY;
            blk_max = fmaxf(blk_max, st[r]);
        }
        blk_max = fmaxf(blk_max, __shfl_xor(blk_max, 32));
        const float new_max = fmaxf(run_max, blk_max);
        const float ref = new_max == -INFINITY ? 0.0f : new_max;  // nothing valid yet: all p = 0
        const float corr = __expf(run_max - ref);
        float psum = 0.0f;
        v8h phi[2], plo[2];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float pr = __expf(st[r] - ref);
            psum += pr;
            const _Float16 hi = (_Float16)pr;
            phi[r >> 3][r & 7] = hi;
            plo[r >> 3][r & 7] = (_Float16)(pr - (float)hi);
        }
        psum += __shfl_xor(psum, 32);
        run_sum = run_sum * corr + psum;
        run_max = new_max;
        // O^T: dims 32 nt + (8b + 4g + r) of token j
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) ot[nt][r] *= corr;
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                v8h vt;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    vt[e] = sv[(8 * (2 * s2 + (e >> 2)) + 4 * g + (e & 3)) * kVPitch + 32 * nt + j];
                ot[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt, phi[s2], ot[nt], 0, 0, 0);
                ot[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt, plo[s2], ot[nt], 0, 0, 0);
            }
        }
    }

    // The four waves' states meet pairwise: 1 -> 0 and 3 -> 2, then 2 -> 0.  The exchange
    // area reuses the value staging (everybody is past its loop after the first barrier).
    float *xch = reinterpret_cast<float *>(&s_v[0][0]);  // 2 x 64 registers x 64 lanes
    auto publish = [&](int slot) {
        float *dst = xch + slot * (64 * 64);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dst[(nt * 16 + r) * 64 + lane] = ot[nt][r];
        s_ml[slot][0][lane] = run_max;
        s_ml[slot][1][lane] = run_sum;
    };
    auto merge = [&](int slot) {
        const float *src = xch + slot * (64 * 64);
        const float m2 = s_ml[slot][0][lane], l2 = s_ml[slot][1][lane];
        const float mx = fmaxf(run_max, m2);
        const float ref = mx == -INFINITY ? 0.0f : mx;
        const float c1 = __expf(run_max - ref), c2 = __expf(m2 - ref);
        run_sum = c1 * run_sum + c2 * l2;
        run_max = mx;
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) ot[nt][r] = c1 * ot[nt][r] + c2 * src[(nt * 16 + r) * 64 + lane];
    };
    static_assert(sizeof(s_v) >= 2 * 64 * 64 * sizeof(float), "the exchange area must fit the staging");
    __syncthreads();
    if (wave & 1) publish(wave >> 1);
    __syncthreads();
    if (!(wave & 1)) merge(wave >> 1);
    __syncthreads();
    if (wave == 2) publish(0);
    __syncthreads();
    if (wave != 0) return;
    merge(0);
    if (qb * 32 + j >= M) return;  // a clamped duplicate of the last token
    const float inv = 1.0f / run_sum;
    float *orow = out + (size_t)m * HD + h * hd + 4 * g;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int b = 0; b < 4; ++b)
            *reinterpret_cast<float4 *>(orow + 32 * nt + 8 * b) =
                make_float4(ot[nt][4 * b] * inv, ot[nt][4 * b + 1] * inv, ot[nt][4 * b + 2] * inv,
                            ot[nt][4 * b + 3] * inv);
}

// Decoding one token: rotary embedding, cache store and attention in one launch, spread
// over kSplits workgroups per head so that many CUs pull the cache at once.
//  * Every workgroup rotates q (and the new k) itself; split 0 also writes the new k and v
//    row to the cache.  The new row is taken from LDS, never re-read from memory.
//  * Keys go to the 4 * kSplits waves of a head in blocks of 16; inside a block four lanes
//    share a key (32 dimensions each) for the scores and every lane owns two dimensions
//    for P.V, so a block is one round trip of 20 loads per lane.
//  * The workgroups of a head publish (max, sum, out[128]) as device-scope stores, draw a
//    ticket, and the last one combines and writes the result: no second launch, nobody waits.
constexpr int kSplits = 12;
constexpr int kPartial = 132;  // floats per partial: out[128], max, sum, padding
__global__ __launch_bounds__(256) void attention_decode_kernel(
    const float *__restrict__ qkv, const int32_t *__restrict__ pos, int heads, float theta,
    __half *__restrict__ kcache, __half *__restrict__ vcache, int max_seq,
    float *__restrict__ partials, unsigned *__restrict__ tickets, float *__restrict__ out) {
    constexpr int hd = 128, half = 64;
    __shared__ float s_q[hd], s_knew[hd], s_vnew[hd];
    __shared__ float s_m[4], s_l[4];
    __shared__ float s_o[4][hd];
    __shared__ int s_last;
    const int h = blockIdx.x / kSplits, sp = blockIdx.x - h * kSplits;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int HD = heads * hd;
    int p = pos[0];
    if (p >= max_seq) p = max_seq - 1;
    const int nkeys = p + 1;
    const float scale = 0.08838834764831845f;  // 1 / sqrt(128)
    // The first block's keys and values do not depend on q: their loads go out before the
    // rotary prologue and the barrier, whose latency they then cover.
    const __half *kh = kcache + (size_t)h * max_seq * hd;
    const __half *vh = vcache + (size_t)h * max_seq * hd;
    const int kidx = lane >> 2, sub = lane & 3;
    uint4 kr[4];
    __half2 vr[16];
    auto load_block = [&](int b) {
        const int t0 = b * 16, last = max(nkeys - 1 - t0, 0);
        const int t = t0 + min(kidx, last);
        const uint4 *krow = reinterpret_cast<const uint4 *>(kh + (size_t)t * hd + sub * 32);
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const v4u kv = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(krow + c));
            kr[c] = make_uint4(kv.x, kv.y, kv.z, kv.w);
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const unsigned vv = __builtin_nontemporal_load(
                reinterpret_cast<const unsigned *>(vh + (size_t)(t0 + min(j, last)) * hd + 2 * lane));
            vr[j] = *reinterpret_cast<const __half2 *>(&vv);
        }
    };
    int b = sp * 4 + wave;
    bool have = b * 16 < nkeys;
    load_block(have ? b : 0);
    __builtin_amdgcn_sched_barrier(0);

    if (tid < half) {
        const int i = tid;
        const float freq = powf(theta, -2.0f * (float)i / (float)hd);
        float sn, cs;
        sincosf((float)p * freq, &sn, &cs);
        const float *qh = qkv + h * hd, *kn = qh + HD, *vn = qh + 2 * HD;
        const float q0 = qh[i], q1 = qh[i + half], k0 = kn[i], k1 = kn[i + half];
        s_q[i] = (q0 * cs - q1 * sn) * scale;
        s_q[i + half] = (q1 * cs + q0 * sn) * scale;
        const __half ka = __float2half_rn(k0 * cs - k1 * sn), kb = __float2half_rn(k1 * cs + k0 * sn);
        const __half va = __float2half_rn(vn[i]), vb = __float2half_rn(vn[i + half]);
        s_knew[i] = __half2float(ka);
        s_knew[i + half] = __half2float(kb);
        s_vnew[i] = __half2float(va);
        s_vnew[i + half] = __half2float(vb);
        if (sp == 0) {
            const size_t c = ((size_t)h * max_seq + p) * hd;
            kcache[c + i] = ka;
            kcache[c + i + half] = kb;
            vcache[c + i] = va;
            vcache[c + i + half] = vb;
        }
    }
    __syncthreads();

    float run_max = -INFINITY, run_sum = 0.0f, o0 = 0.0f, o1 = 0.0f;
    while (have) {
        const int t0 = b * 16, last = nkeys - 1 - t0;  // last >= 0
        const int t = t0 + min(kidx, last);
        float acc = 0.0f;
        const bool fresh = t == p;  // the row this launch adds: take it from LDS
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const __half2 *h2 = reinterpret_cast<const __half2 *>(&kr[c]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int d = sub * 32 + c * 8 + 2 * e;
                float2 f = __half22float2(h2[e]);
                if (fresh) f = make_float2(s_knew[d], s_knew[d + 1]);
                acc = fmaf(f.x, s_q[d], acc);
                acc = fmaf(f.y, s_q[d + 1], acc);
            }
        }
        acc += dpp_f<0xB1, 0xf>(0.0f, acc);  // the four lanes of a key
        acc += dpp_f<0x4E, 0xf>(0.0f, acc);
        const float s = kidx <= last ? acc : -INFINITY;
        const float new_max = fmaxf(run_max, wave_max_f(s));
        const float corr = __expf(run_max - new_max);  // 0 on the first block
        const float pr = kidx <= last ? __expf(s - new_max) : 0.0f;
        run_sum = run_sum * corr + wave_sum_f(sub == 0 ? pr : 0.0f);
        run_max = new_max;
        o0 *= corr;
        o1 *= corr;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pr), 4 * j));
            // rows past the end were clamped loads of memory that may hold anything
            float2 v = j <= last ? __half22float2(vr[j]) : make_float2(0.0f, 0.0f);
            if (t0 + j == p) v = make_float2(s_vnew[2 * lane], s_vnew[2 * lane + 1]);
            o0 = fmaf(pj, v.x, o0);
            o1 = fmaf(pj, v.y, o1);
        }
        b += 4 * kSplits;
        have = b * 16 < nkeys;
        if (have) load_block(b);
    }
    if (lane == 0) {
        s_m[wave] = run_max;
        s_l[wave] = run_sum;
    }
    s_o[wave][2 * lane] = o0;
    s_o[wave][2 * lane + 1] = o1;
    __syncthreads();
    float *mine = partials + ((size_t)h * kSplits + sp) * kPartial;
    if (tid < hd) {
        float gmax = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float c = s_m[w] == -INFINITY ? 0.0f : __expf(s_m[w] - gmax);
            num += c * s_o[w][tid];
            den += c * s_l[w];
        }
        __hip_atomic_store(mine + tid, num, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) {
            __hip_atomic_store(mine + hd, gmax, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(mine + hd + 1, den, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // published once the stores have completed (vmcnt(0): this wave's; the barrier:
    // everybody's); then one thread draws the ticket
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(&tickets[h], 1u);
        const int is_last = ticket == (unsigned)kSplits - 1;
        if (is_last) atomicExch(&tickets[h], 0u);  // ready for the next launch
        s_last = is_last;
    }
    __syncthreads();
    if (!s_last || tid >= hd) return;
    const float *all = partials + (size_t)h * kSplits * kPartial;
    float ms[kSplits], gmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < kSplits; ++i) {
        ms[i] = __hip_atomic_load(all + i * kPartial + hd, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        gmax = fmaxf(gmax, ms[i]);
    }
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int i = 0; i < kSplits; ++i) {
        const float c = ms[i] == -INFINITY ? 0.0f : __expf(ms[i] - gmax);
        num += c * __hip_atomic_load(all + i * kPartial + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        den += c * __hip_atomic_load(all + i * kPartial + hd + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    out[h * hd + tid] = num / den;
}

// h[m, f] = silu(gu[m, f]) * gu[m, F + f]
__global__ __launch_bounds__(kBlock) void swiglu_kernel(const float *__restrict__ gu, int F,
                                                        float *__restrict__ hout) {
    const int m = blockIdx.y;
    const int f = blockIdx.x * kBlock + threadIdx.x;
    if (f < F) {
        const float g = gu[(size_t)m * 2 * F + f], u = gu[(size_t)m * 2 * F + F + f];
        hout[(size_t)m * F + f] = (g / (1.0f + __expf(-g))) * u;
    }
}

// Index of the largest of n values (the lowest index among equals); one workgroup.
// With `advance` the position counter hist_pos[0] is incremented first (the history slot is
// the new position); the history holds hist_cap entries; with `table` the row of the chosen index is copied to x_out (the next
// step's embedding): the tail of a greedy decode step in one launch.
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ v, int n,
                                                      int32_t *__restrict__ out,
                                                      int32_t *__restrict__ hist,
                                                      int32_t *__restrict__ hist_pos, int hist_cap,
                                                      unsigned *__restrict__ dev_flags, int advance,
                                                      const float *__restrict__ table, int H,
                                                      float *__restrict__ x_out) {
    __shared__ float s_v[16];
    __shared__ int s_i[16];
    __shared__ int s_pick;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    auto take = [&](float x, int i) {
        if (x > best || (x == best && i < bi)) {
            best = x;
            bi = i;
        }
    };
    // batches of 32 values per thread (eight 16-byte loads, all issued before the first
    // comparison: one memory round trip per batch instead of one per value)
    int base = 0;
    if ((reinterpret_cast<uintptr_t>(v) & 15u) == 0) {
        const int n4 = n & ~3;
        for (; base < n4; base += 32 * 1024) {
            float4 x[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int i = base + 4 * ((int)threadIdx.x + 1024 * j);
                x[j] = *reinterpret_cast<const float4 *>(v + min(i, n4 - 4));
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int i = base + 4 * ((int)threadIdx.x + 1024 * j);
                if (i < n4) take(x[j].x, i), take(x[j].y, i + 1), take(x[j].z, i + 2), take(x[j].w, i + 3);
            }
        }
        base = n4;
    }
    for (int i = base + threadIdx.x; i < n; i += 1024) take(v[i], i);
    for (int off = 32; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off);
        const int oi = __shfl_xor(bi, off);
        if (ob > best || (ob == best && oi < bi)) {
            best = ob;
            bi = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        s_v[threadIdx.x >> 6] = best;
        s_i[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (s_v[w] > best || (s_v[w] == best && s_i[w] < bi)) {
                best = s_v[w];
                bi = s_i[w];
            }
        bi = bi == 0x7fffffff ? 0 : bi;
        out[0] = bi;
        if (hist) {
            // a slot outside the history is neither written nor made the new position; the
            // host learns of it through the context's flag word
            const int p = hist_pos[0] + (advance ? 1 : 0);
            if (p >= 0 && p < hist_cap) {
                if (advance) hist_pos[0] = p;
                hist[p] = bi;
            } else {
                atomicOr(dev_flags, (unsigned)RBN_FLAG_HISTORY_OVERFLOW);
            }
        }
        s_pick = bi;
    }
    if (table == nullptr) return;
    __syncthreads();
    const float *row = table + (size_t)s_pick * H;
    for (int i = threadIdx.x; i < H; i += 1024) x_out[i] = row[i];
}

__global__ void add_i32_kernel(int32_t *p, int delta) { p[0] += delta; }

// out[i] = sigma * z_i, z_i standard normal from a counter-based generator (splitmix64 of
// (seed, i / 2), Box-Muller in f32).  For random-initialised weights that never leave the
// device; NOT the host generator of rbn_synth_normal_f32.
__global__ __launch_bounds__(kBlock) void synth_normal_device_kernel(uint64_t seed, float sigma,
                                                                     float *__restrict__ out,
                                                                     uint64_t n) {
    const uint64_t pair = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (2 * pair >= n) return;
    uint64_t z = seed * 0x9E3779B97F4A7C15ull + (pair + 1) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const float u1 = ((float)(uint32_t)(z >> 40) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
    const float u2 = (float)(uint32_t)((z >> 16) & 0xFFFFFF) * (1.0f / 16777216.0f);
    const float r = sqrtf(-2.0f * __logf(u1)) * sigma;
    float sn, cs;
    sincosf(6.283185307179586f * u2, &sn, &cs);
    out[2 * pair] = r * cs;
    if (2 * pair + 1 < n) out[2 * pair + 1] = r * sn;
}

}  // namespace

extern "C" {

int rbn_embed_f32(rbn_ctx *ctx, const float *d_table, const int32_t *d_tokens, uint64_t M,
                  uint64_t H, uint64_t vocab, float *d_x) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_table && d_tokens && d_x, "null pointer in rbn_embed_f32");
    RBN_REQUIRE(M > 0 && M < (1u << 20) && H > 0 && H < (1u << 24) && vocab > 0 && vocab < (1u << 30),
                "bad sizes in rbn_embed_f32");
    embed_kernel<<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(d_table, d_tokens, (int)H,
                                                                     (int)vocab, d_x);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_rmsnorm_quant_i8(rbn_ctx *ctx, float *d_x, const float *d_delta, const float *d_gate_up,
                         const float *d_gamma, float eps, uint64_t M, uint64_t H, int8_t *d_q,
                         float *d_act_scale, int32_t *d_rowsum) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_gamma && d_q && d_act_scale && d_rowsum, "null pointer in rbn_rmsnorm_quant_i8");
    RBN_REQUIRE((d_x != nullptr) != (d_gate_up != nullptr),
                "rbn_rmsnorm_quant_i8 takes either d_x (with optional d_delta) or d_gate_up");
    RBN_REQUIRE(d_gate_up == nullptr || d_delta == nullptr, "d_delta goes with d_x only");
    RBN_REQUIRE(M > 0 && M < (1u << 20), "bad M in rbn_rmsnorm_quant_i8");
    const uint64_t pitch = rbn_kpad(H);
    RBN_REQUIRE(H > 0 && pitch <= (uint64_t)kNormThreads * kPer, "rbn_rmsnorm_quant_i8 takes H <= %d",
                kNormThreads * kPer);
    rmsnorm_quant_kernel<<<dim3((unsigned)M), dim3(kNormThreads), 0, ctx->stream>>>(
        d_x, d_delta, d_gate_up, d_gamma, eps, (int)H, (int)pitch, d_q, d_act_scale, d_rowsum);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_rope_kv_store_f16(rbn_ctx *ctx, float *d_qkv, const int32_t *d_pos0, uint64_t M,
                          uint64_t heads, uint64_t head_dim, float theta, void *d_kcache,
                          void *d_vcache, uint64_t max_seq) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_qkv && d_pos0 && d_kcache && d_vcache, "null pointer in rbn_rope_kv_store_f16");
    RBN_REQUIRE(M > 0 && M < (1u << 20) && heads > 0 && heads < 4096 && head_dim >= 2 &&
                    head_dim <= 1024 && (head_dim & 1) == 0 && max_seq > 0 && max_seq < (1u << 24),
                "bad sizes in rbn_rope_kv_store_f16");
    rope_kv_store_kernel<<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
        d_qkv, d_pos0, (int)heads, (int)head_dim, theta, (__half *)d_kcache, (__half *)d_vcache,
        (int)max_seq);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_attention_f16kv(rbn_ctx *ctx, const float *d_qkv, const int32_t *d_pos0, uint64_t M,
                        uint64_t heads, uint64_t head_dim, const void *d_kcache,
                        const void *d_vcache, uint64_t max_seq, float *d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_qkv && d_pos0 && d_kcache && d_vcache && d_out, "null pointer in rbn_attention_f16kv");
    RBN_REQUIRE(head_dim == 128, "rbn_attention_f16kv takes head_dim == 128 (got %llu)",
                (unsigned long long)head_dim);
    RBN_REQUIRE(M > 0 && heads > 0 && M * heads < (1ull << 31) && max_seq > 0 && max_seq < (1u << 24),
                "bad sizes in rbn_attention_f16kv");
    // a single token (decode) gets more waves per head: only `heads` workgroups run;
    // prompts of at least 32 tokens go to the matrix cores
    if (M >= 32) {
        const uint64_t blocks = (M + 31) / 32 * heads;
        attention_mfma_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(
            d_qkv, d_pos0, (int)M, (int)heads, (const __half *)d_kcache, (const __half *)d_vcache,
            (int)max_seq, d_out);
    } else if (M == 1)
        attention_kernel<8><<<dim3((unsigned)(M * heads)), dim3(8 * 64), 0, ctx->stream>>>(
            d_qkv, d_pos0, (int)heads, (const __half *)d_kcache, (const __half *)d_vcache, (int)max_seq, d_out);
    else
        attention_kernel<4><<<dim3((unsigned)(M * heads)), dim3(4 * 64), 0, ctx->stream>>>(
            d_qkv, d_pos0, (int)heads, (const __half *)d_kcache, (const __half *)d_vcache, (int)max_seq, d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_attention_decode_f16kv(rbn_ctx *ctx, const float *d_qkv, const int32_t *d_pos, uint64_t heads,
                               uint64_t head_dim, float theta, void *d_kcache, void *d_vcache,
                               uint64_t max_seq, float *d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_qkv && d_pos && d_kcache && d_vcache && d_out, "null pointer in rbn_attention_decode_f16kv");
    RBN_REQUIRE(head_dim == 128, "rbn_attention_decode_f16kv takes head_dim == 128 (got %llu)",
                (unsigned long long)head_dim);
    // partial results and tickets live in the context's split workspace
    RBN_REQUIRE(heads > 0 && heads <= RBN_SPLITK_GROUPS && max_seq > 0 && max_seq < (1u << 24),
                "bad sizes in rbn_attention_decode_f16kv (heads <= %d)", RBN_SPLITK_GROUPS);
    static_assert((size_t)RBN_SPLITK_GROUPS * kSplits * kPartial * 4 <= (size_t)RBN_SPLITK_TILES * 4096,
                  "the attention partials must fit the split workspace");
    attention_decode_kernel<<<dim3((unsigned)(heads * kSplits)), dim3(256), 0, ctx->stream>>>(
        d_qkv, d_pos, (int)heads, theta, (__half *)d_kcache, (__half *)d_vcache, (int)max_seq,
        (float *)ctx->splitk_partials, ctx->splitk_tickets, d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_swiglu_f32(rbn_ctx *ctx, const float *d_gate_up, uint64_t M, uint64_t F, float *d_h) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_gate_up && d_h, "null pointer in rbn_swiglu_f32");
    RBN_REQUIRE(M > 0 && M < 65536 && F > 0 && F < (1u << 24), "bad sizes in rbn_swiglu_f32");
    swiglu_kernel<<<dim3((unsigned)((F + kBlock - 1) / kBlock), (unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
        d_gate_up, (int)F, d_h);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_argmax_f32(rbn_ctx *ctx, const float *d_values, uint64_t n, int32_t *d_index,
                   int32_t *d_history, const int32_t *d_history_pos, uint64_t history_capacity) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_values && d_index, "null pointer in rbn_argmax_f32");
    RBN_REQUIRE(n > 0 && n < (1u << 30), "bad n in rbn_argmax_f32");
    RBN_REQUIRE((d_history == nullptr) == (d_history_pos == nullptr),
                "d_history and d_history_pos go together");
    RBN_REQUIRE(d_history == nullptr || (history_capacity > 0 && history_capacity < (1ull << 31)),
                "history_capacity must be in [1, 2^31) when d_history is given");
    argmax_kernel<<<dim3(1), dim3(1024), 0, ctx->stream>>>(d_values, (int)n, d_index, d_history,
                                                          const_cast<int32_t *>(d_history_pos),
                                                          (int)history_capacity, ctx->dev_flags, 0, nullptr,
                                                          0, nullptr);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_greedy_next_f32(rbn_ctx *ctx, const float *d_logits, uint64_t vocab, int32_t *d_token,
                        int32_t *d_history, int32_t *d_pos, uint64_t history_capacity,
                        const float *d_table, uint64_t H, float *d_x) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_logits && d_token && d_history && d_pos && d_table && d_x && vocab > 0 && H > 0 &&
                    vocab < (1ull << 31) && H < (1ull << 31),
                "bad arguments in rbn_greedy_next_f32");
    RBN_REQUIRE(history_capacity > 0 && history_capacity < (1ull << 31),
                "history_capacity must be in [1, 2^31)");
    argmax_kernel<<<dim3(1), dim3(1024), 0, ctx->stream>>>(d_logits, (int)vocab, d_token, d_history, d_pos,
                                                          (int)history_capacity, ctx->dev_flags, 1, d_table,
                                                          (int)H, d_x);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_add_i32(rbn_ctx *ctx, int32_t *d_value, int32_t delta) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_value != nullptr, "null pointer in rbn_add_i32");
    add_i32_kernel<<<dim3(1), dim3(1), 0, ctx->stream>>>(d_value, delta);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_synth_normal_device_f32(rbn_ctx *ctx, uint64_t seed, float sigma, float *d_out, uint64_t n) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_out != nullptr && n > 0, "bad arguments in rbn_synth_normal_device_f32");
    const uint64_t pairs = (n + 1) / 2, blocks = (pairs + kBlock - 1) / kBlock;
    RBN_REQUIRE(blocks < (1ull << 31), "n too large");
    synth_normal_device_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, ctx->stream>>>(seed, sigma, d_out, n);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

}  // extern "C"

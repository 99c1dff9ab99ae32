// Activation quantisation.
//
// (a) Per-token absmax int8: build-defined, no counterpart in the reference (which
//     ternarises activations with quantize_ternary, bitnet/kernels.rs:277).
// (b) Reference-mode activations: quantize_ternary over the whole [M,K] tensor
//     (bitnet/quantization.rs:67-109) expanded to int8 {-1,0,+1} via get_value
//     (:275-291).
#include "common.hpp"

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ float wave_max(float v) {
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}

__device__ __forceinline__ int wave_sum(int v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__device__ __forceinline__ int quant1(float x, float inv) {
    float r = rintf(x * inv);  // round half to even
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

// One workgroup per token.  Pass 1: wavefront max-reduction of |x| over the row.
// Pass 2 (row is L2/L1 resident by then): scale, round, clamp, pack four int8 per
// store, and reduce the int32 row sum.
__global__ __launch_bounds__(kBlock) void act_quant_i8_kernel(
    const float *__restrict__ x, uint64_t K, uint64_t pitch, int8_t *__restrict__ q,
    float *__restrict__ act_scale, int32_t *__restrict__ rowsum) {
    __shared__ float s_max[kBlock / 64];
    __shared__ int s_sum[kBlock / 64];
    const uint64_t m = blockIdx.x;
    const float *row = x + m * K;
    const bool vec_ok = ((K & 3) == 0) && ((((uintptr_t)row) & 15u) == 0);
    const uint64_t quads = (K + 3) / 4;

    float amax = 0.0f;
    for (uint64_t qd = threadIdx.x; qd < quads; qd += kBlock) {
        if (vec_ok) {
            float4 v = reinterpret_cast<const float4 *>(row)[qd];
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        } else {
            for (int i = 0; i < 4; ++i) {
                uint64_t k = qd * 4 + i;
                if (k < K) amax = fmaxf(amax, fabsf(row[k]));
            }
        }
    }
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = s_max[0];
    for (int w = 1; w < kBlock / 64; ++w) amax = fmaxf(amax, s_max[w]);

    const float g = fmaxf(amax, 1e-5f);
    const float inv = 127.0f / g;
    int sum = 0;
    const uint64_t out_quads = pitch / 4;  // pitch is a multiple of 64
    uint32_t *qrow = reinterpret_cast<uint32_t *>(q + m * pitch);
    for (uint64_t qd = threadIdx.x; qd < out_quads; qd += kBlock) {
        int v[4] = {0, 0, 0, 0};
        if (qd < quads) {
            if (vec_ok) {
                float4 f = reinterpret_cast<const float4 *>(row)[qd];
                v[0] = quant1(f.x, inv);
                v[1] = quant1(f.y, inv);
                v[2] = quant1(f.z, inv);
                v[3] = quant1(f.w, inv);
            } else {
                for (int i = 0; i < 4; ++i) {
                    uint64_t k = qd * 4 + i;
                    if (k < K) v[i] = quant1(row[k], inv);
                }
            }
        }
        sum += v[0] + v[1] + v[2] + v[3];
        qrow[qd] = (uint32_t)(v[0] & 0xff) | ((uint32_t)(v[1] & 0xff) << 8) |
                   ((uint32_t)(v[2] & 0xff) << 16) | ((uint32_t)(v[3] & 0xff) << 24);
    }
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0) s_sum[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int w = 0; w < kBlock / 64; ++w) t += s_sum[w];
        rowsum[m] = t;
        act_scale[m] = g / 127.0f;
    }
}

// The same with the row kept in registers between the two passes (NQ 16-byte pieces per
// thread, K <= 1024 * NQ, K % 4 == 0, 16-byte aligned rows): the row is read from memory once,
// with all its loads in flight before the first comparison.
template <int NQ>
__global__ __launch_bounds__(kBlock) void act_quant_i8_regs_kernel(
    const float *__restrict__ x, uint64_t K, uint64_t pitch, int8_t *__restrict__ q,
    float *__restrict__ act_scale, int32_t *__restrict__ rowsum) {
    __shared__ float s_max[kBlock / 64];
    __shared__ int s_sum[kBlock / 64];
    const uint64_t m = blockIdx.x;
    const float4 *row = reinterpret_cast<const float4 *>(x + m * K);
    const uint32_t quads = (uint32_t)(K / 4), out_quads = (uint32_t)(pitch / 4);
    float4 v[NQ];
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
        const uint32_t qd = threadIdx.x + j * kBlock;
        v[j] = row[qd < quads ? qd : quads - 1];
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
        const uint32_t qd = threadIdx.x + j * kBlock;
        if (qd >= quads) v[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);  // the zero padding
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[j].x), fabsf(v[j].y)), fmaxf(fabsf(v[j].z), fabsf(v[j].w))));
    }
    amax = wave_max(amax);
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = s_max[0];
    for (int w = 1; w < kBlock / 64; ++w) amax = fmaxf(amax, s_max[w]);
    const float g = fmaxf(amax, 1e-5f);
    const float inv = 127.0f / g;
    int sum = 0;
    uint32_t *qrow = reinterpret_cast<uint32_t *>(q + m * pitch);
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
        const uint32_t qd = threadIdx.x + j * kBlock;
        const int a = quant1(v[j].x, inv), b = quant1(v[j].y, inv), c = quant1(v[j].z, inv),
                  d = quant1(v[j].w, inv);
        sum += a + b + c + d;
        if (qd < out_quads)
            qrow[qd] = (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
                       ((uint32_t)(d & 0xff) << 24);
    }
    sum = wave_sum(sum);
    if ((threadIdx.x & 63) == 0) s_sum[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int w = 0; w < kBlock / 64; ++w) t += s_sum[w];
        rowsum[m] = t;
        act_scale[m] = g / 127.0f;
    }
}

__global__ void fill_f32_kernel(float *dst, float value, uint64_t n) {
    uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = value;
}

}  // namespace

extern "C" {

int rbn_act_quant_i8(rbn_ctx *ctx, const float *d_x, uint64_t M, uint64_t K, int8_t *d_q,
                     float *d_act_scale, int32_t *d_rowsum) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(M > 0 && K > 0, "M and K must be positive");
    RBN_REQUIRE(d_x && d_q && d_act_scale && d_rowsum, "null pointer in rbn_act_quant_i8");
    RBN_REQUIRE(((uintptr_t)d_x & 3u) == 0 && ((uintptr_t)d_q & 15u) == 0,
                "d_x must be 4-byte and d_q 16-byte aligned");
    RBN_REQUIRE(M <= 0x7fffffffull, "too many rows");
    const uint64_t pitch = rbn_kpad(K);
    const bool in_regs = (K & 3) == 0 && ((uintptr_t)d_x & 15u) == 0 && pitch <= 16ull * 4 * kBlock;
    if (in_regs && pitch <= 4ull * 4 * kBlock)
        act_quant_i8_regs_kernel<4><<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
            d_x, K, pitch, d_q, d_act_scale, d_rowsum);
    else if (in_regs && pitch <= 8ull * 4 * kBlock)
        act_quant_i8_regs_kernel<8><<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
            d_x, K, pitch, d_q, d_act_scale, d_rowsum);
    else if (in_regs)
        act_quant_i8_regs_kernel<16><<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
            d_x, K, pitch, d_q, d_act_scale, d_rowsum);
    else
        act_quant_i8_kernel<<<dim3((unsigned)M), dim3(kBlock), 0, ctx->stream>>>(
            d_x, K, pitch, d_q, d_act_scale, d_rowsum);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

int rbn_act_quant_ternary(rbn_ctx *ctx, const float *d_x, uint64_t M, uint64_t K, int mode,
                          int8_t *d_q, float *d_act_scale, int32_t *d_rowsum, float *h_scale,
                          float *h_threshold) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(M > 0 && K > 0, "M and K must be positive");
    RBN_REQUIRE(d_x && d_q && d_act_scale && d_rowsum, "null pointer in rbn_act_quant_ternary");
    RBN_REQUIRE(M <= 0x7fffffffull, "too many rows");
    RBN_CHECK(rbn_refuse_while_capturing(ctx, "rbn_act_quant_ternary"));
    const uint64_t n = M * K;
    // "Packed" image of the activation tensor, in a buffer the context keeps (it only grows).
    void *d_tmp = nullptr;
    RBN_CHECK(rbn_workspace2(ctx, rbn_packed_capacity(n), &d_tmp));
    float scale = 1.0f, thr = 0.0f;
    int rc = rbn_quantize_ternary(ctx, d_x, n, mode, (uint8_t *)d_tmp, &scale, &thr, nullptr);
    if (rc == RBN_OK)
        rc = rbn_unpack_ternary_i8(ctx, (const uint8_t *)d_tmp, M, K, rbn_kpad(K), d_q, d_rowsum);
    if (rc == RBN_OK) {
        fill_f32_kernel<<<dim3((unsigned)((M + 255) / 256)), dim3(256), 0, ctx->stream>>>(
            d_act_scale, scale, M);
        if (hipGetLastError() != hipSuccess) rc = rbn_fail(RBN_ERR_HIP, "fill kernel launch failed");
    }
    if (rc != RBN_OK) return rc;
    if (h_scale) *h_scale = scale;
    if (h_threshold) *h_threshold = thr;
    return RBN_OK;
}

}  // extern "C"

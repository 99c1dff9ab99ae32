// Calibration probes: what the machine itself delivers, measured next to the kernels that
// are priced against it.  No reference counterpart.
//
// rbn_probe_mfma_i8 runs nothing but v_mfma_i32_32x32x32_i8 (eight independent
// accumulators per wave, two waves per SIMD, operands held in registers) and reports the
// rate.  The operand VALUES matter: the clock this chip sustains depends on how many bits
// toggle in the multiplier array, so the rate with real int8 activations and ternary
// codes is lower than with constant operands.
#include "common.hpp"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256, 2) void mfma_i8_probe_kernel(const v4i *__restrict__ ops,
                                                               int iters, int *__restrict__ sink) {
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    v4i a[4], b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        a[j] = ops[j * 256 + threadIdx.x];
        b[j] = ops[1024 + j * 256 + threadIdx.x];
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[(i + (i >> 2)) & 3], b[i & 3], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (s == 0x7fffffff) sink[0] = s;  // keeps the loop alive; practically never true
}

// What a launch that only READS costs: workgroups of four waves, a lane loads four 16-byte
// units 1 KiB apart (a wave reads 4 KiB of consecutive memory, a workgroup 16 KiB: the
// GEMV's access pattern without its arithmetic, staging, reduction and stores).
template <bool NT>
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4 *__restrict__ src, uint64_t units,
                                                          uint32_t *__restrict__ sink) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const uint64_t base = ((uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 256 + (threadIdx.x & 63);
    uint4 v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint64_t at = base + 64 * i;
        const uint4 *p = src + (at < units ? at : units - 1);
        if (NT) {
            const v4u t = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(p));
            v[i] = make_uint4(t.x, t.y, t.z, t.w);
        } else {
            v[i] = *p;
        }
    }
    uint32_t x = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) x |= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    if (x == 0x9E3779B9u) sink[0] = x;  // keeps the loads alive; practically never true
}

__global__ void empty_kernel() {}

}  // namespace

extern "C" int rbn_probe_empty_launch(rbn_ctx *ctx) {
    RBN_ENTER(ctx);
    empty_kernel<<<dim3(1), dim3(64), 0, ctx->stream>>>();
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

extern "C" int rbn_probe_stream_read(rbn_ctx *ctx, const void *d_src, uint64_t bytes, int nontemporal) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(d_src != nullptr && bytes >= 16 && ((uintptr_t)d_src & 15u) == 0,
                "rbn_probe_stream_read needs a 16-byte aligned buffer of at least 16 bytes");
    const uint64_t units = bytes / 16, blocks = (units + 1023) / 1024;
    RBN_REQUIRE(blocks < (1ull << 31), "buffer too large");
    uint32_t *ws = ctx->dev_flags + 16;  // a word nobody reads (never written in practice)
    if (nontemporal)
        stream_read_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((const uint4 *)d_src, units,
                                                                                      ws);
    else
        stream_read_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((const uint4 *)d_src, units,
                                                                                       ws);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

extern "C" int rbn_probe_mfma_i8(rbn_ctx *ctx, int operand_kind, double *h_tops) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(h_tops != nullptr, "h_tops is NULL");
    RBN_REQUIRE(operand_kind >= 0 && operand_kind <= 2, "operand_kind must be 0, 1 or 2");
    // 2048 operand registers of 16 bytes: A fragments first, B fragments second
    static uint8_t host[2048 * 16];
    uint64_t x = 88172645463325252ull;
    for (size_t i = 0; i < sizeof(host); ++i) {
        x ^= x << 13;
        x ^= x >> 7;
        x ^= x << 17;
        const bool is_b = i >= 1024 * 16;
        if (operand_kind == RBN_PROBE_CONSTANT)
            host[i] = 1;
        else if (is_b)
            host[i] = operand_kind == RBN_PROBE_I8_TERNARY ? (uint8_t)(x % 3) : (uint8_t)x;
        else
            host[i] = (uint8_t)(int8_t)((int)(x % 255) - 127);
    }
    void *ws = nullptr;
    RBN_CHECK(rbn_workspace(ctx, sizeof(host) + 256, &ws));
    RBN_HIP(hipMemcpyAsync(ws, host, sizeof(host), hipMemcpyHostToDevice, ctx->stream));
    int *sink = (int *)((char *)ws + sizeof(host));
    const int blocks = 2 * ctx->props.multiProcessorCount, iters = 8192, reps = 5;
    mfma_i8_probe_kernel<<<blocks, 256, 0, ctx->stream>>>((const v4i *)ws, iters, sink);  // warm-up
    RBN_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
    for (int r = 0; r < reps; ++r)
        mfma_i8_probe_kernel<<<blocks, 256, 0, ctx->stream>>>((const v4i *)ws, iters, sink);
    RBN_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
    RBN_HIP(hipEventSynchronize(ctx->ev_stop));
    float ms = 0;
    RBN_HIP(hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_stop));
    const double ops = (double)blocks * 4 * iters * 8 * 65536.0 * reps;
    *h_tops = ops / (ms * 1e-3) / 1e12;
    return RBN_OK;
}

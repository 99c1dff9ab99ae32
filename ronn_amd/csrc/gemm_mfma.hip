// Prefill-regime ternary GEMM on the int8 matrix cores:
// out[m,n] = ((float)acc * act_scale[m]) * w_scale, acc = sum_k q[m,k] * w[k,n] (int32).
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (epilogue order :168).
//
// Workgroup tile 128 (M) x 128 (N), four waves as 2 x 2, each wave 64 x 64 as 2 x 2
// v_mfma_i32_32x32x32_i8 tiles.  Activations go through LDS (double-buffered, rows
// padded to 80 B so that the 128-bit fragment reads are free of bank conflicts).
// The ternary weights never pass through LDS as bytes: a lane's B fragment for one
// MFMA (sixteen consecutive k of one column) is exactly ONE u32 of the tiled layout,
// loaded straight from global memory and expanded in registers with seven VALU
// operations ((w >> 2s) & 0x03030303).  Weights are stored as code = value + 1, so the
// per-token sum of q is subtracted in the epilogue (integer-exact).
#include "common.hpp"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kRowStride = 80;  // bytes per activation row in LDS (64 + 16 padding)

__device__ __forceinline__ v4i decode_b(uint32_t w) {
    v4i b;
    b.x = (int)(w & 0x03030303u);
    b.y = (int)((w >> 2) & 0x03030303u);
    b.z = (int)((w >> 4) & 0x03030303u);
    b.w = (int)((w >> 6) & 0x03030303u);
    return b;
}

__global__ __launch_bounds__(kThreads) void gemm_t2_i8_mfma_kernel(
    const int8_t *__restrict__ q,         // [M][Kpad]
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint32_t *__restrict__ wt,      // tiled: word ((n/4) * Kpad/16 + kb) * 4 + n%4
    float w_scale, int M, int Kpad, int N, int Npad, int32_t *__restrict__ acc_out,
    float *__restrict__ out) {
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][BM * kRowStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int n_tiles = (N + BN - 1) / BN;
    const int bm = blockIdx.x / n_tiles, bn = blockIdx.x % n_tiles;
    const int m0 = bm * BM, n0 = bn * BN;

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // global -> LDS staging of the activation tile: 128 rows x 64 B = 512 x 16 B
    const int st_row0 = tid >> 2, st_seg = tid & 3;  // rows st_row0 and st_row0 + 64
    auto load_a = [&](int k0, uint4 &r0, uint4 &r1) {
        int ra = m0 + st_row0, rb = m0 + st_row0 + 64;
        r0 = ra < M ? *reinterpret_cast<const uint4 *>(q + (size_t)ra * Kpad + k0 + st_seg * 16)
                    : make_uint4(0u, 0u, 0u, 0u);
        r1 = rb < M ? *reinterpret_cast<const uint4 *>(q + (size_t)rb * Kpad + k0 + st_seg * 16)
                    : make_uint4(0u, 0u, 0u, 0u);
    };
    auto store_a = [&](int buf, const uint4 &r0, const uint4 &r1) {
        *reinterpret_cast<uint4 *>(&s_a[buf][st_row0 * kRowStride + st_seg * 16]) = r0;
        *reinterpret_cast<uint4 *>(&s_a[buf][(st_row0 + 64) * kRowStride + st_seg * 16]) = r1;
    };
    // B words of one k step of 64: [nt][ks]
    const int b_col = n0 + wn * 64 + (lane & 31);
    const int b_kgrp = lane >> 5;
    const int kblocks = Kpad >> 4;
    auto load_b = [&](int k0, uint32_t (&w)[2][2]) {
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                int col = b_col + nt * 32;
                int kb = (k0 >> 4) + ks * 2 + b_kgrp;
                w[nt][ks] = col < Npad ? wt[((size_t)(col >> 2) * kblocks + kb) * 4 + (col & 3)]
                                       : 0x55555555u;
            }
    };

    uint4 ra0, ra1;
    uint32_t wb[2][2];
    load_a(0, ra0, ra1);
    load_b(0, wb);
    store_a(0, ra0, ra1);
    __syncthreads();

    const int iters = Kpad / BK;
    for (int it = 0; it < iters; ++it) {
        const int cur = it & 1;
        uint32_t wb_next[2][2];
        const bool more = it + 1 < iters;
        if (more) {
            load_a((it + 1) * BK, ra0, ra1);
            load_b((it + 1) * BK, wb_next);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v4i bf[2];
            bf[0] = decode_b(wb[0][ks]);
            bf[1] = decode_b(wb[1][ks]);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
                const int row = wm * 64 + mt * 32 + (lane & 31);
                const v4i af = *reinterpret_cast<const v4i *>(
                    &s_a[cur][row * kRowStride + ks * 32 + (lane >> 5) * 16]);
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    acc[mt][nt] =
                        __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[nt], acc[mt][nt], 0, 0, 0);
            }
        }
        if (more) {
            store_a(cur ^ 1, ra0, ra1);
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) wb[nt][ks] = wb_next[nt][ks];
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane & 31), rows 8*(r/4) + 4*(lane/32) + r%4 of each tile
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = m0 + wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            if (row >= M) continue;
            const int rs = rowsum[row];
            const float as = act_scale[row];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                const int col = n0 + wn * 64 + nt * 32 + (lane & 31);
                if (col < N) {
                    int total = acc[mt][nt][r] - rs;
                    if (acc_out) acc_out[(size_t)row * N + col] = total;
                    float v = (float)total * as;  // kernels.rs:168, left to right
                    v = v * w_scale;
                    out[(size_t)row * N + col] = v;
                }
            }
        }
    }
}

}  // namespace

extern "C" int rbn_gemm_t2_i8_mfma(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                   const int32_t *d_rowsum, const uint32_t *d_tiled,
                                   float w_scale, uint64_t M, uint64_t K, uint64_t N,
                                   int32_t *d_acc, float *d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(M > 0 && K > 0 && N > 0, "M, K and N must be positive");
    RBN_REQUIRE(d_q && d_act_scale && d_rowsum && d_tiled && d_out,
                "null pointer in rbn_gemm_t2_i8_mfma");
    RBN_REQUIRE((((uintptr_t)d_q | (uintptr_t)d_tiled) & 15u) == 0,
                "d_q and d_tiled must be 16-byte aligned");
    RBN_REQUIRE(M <= (1ull << 24) && K <= (1ull << 24) && N <= (1ull << 24), "dimension too large");
    const int Kpad = (int)rbn_kpad(K), Npad = (int)rbn_npad(N);
    const uint64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    RBN_REQUIRE(tiles <= 0x7fffffffull, "too many tiles");
    gemm_t2_i8_mfma_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, ctx->stream>>>(
        d_q, d_act_scale, d_rowsum, d_tiled, w_scale, (int)M, Kpad, (int)N, Npad, d_acc, d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

extern "C" int rbn_matmul_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                                uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc,
                                float *d_out) {
    if (M <= RBN_GEMV_MAX_M)
        return rbn_gemv_t2_i8(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc,
                              d_out);
    return rbn_gemm_t2_i8_mfma(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc,
                               d_out);
}

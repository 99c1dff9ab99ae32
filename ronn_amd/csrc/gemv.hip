// Decode-regime ternary GEMV: out[m,n] = ((float)acc * act_scale[m]) * w_scale with
// acc = sum_k q[m,k] * w[k,n] in int32, for M <= 16 tokens.
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (inner loop :161-165,
// epilogue :168).
//
// The kernel is bound by HBM: it streams the tiled 2-bit weights exactly once with
// 128-bit loads (four columns x sixteen k per lane and load), expands each word to
// int8-ready bytes in registers ((w >> 2s) & 0x03030303) and accumulates with the
// int8 dot instruction.  The weights are stored as code = value + 1, so
//     sum_k q*w = sum_k q*code - sum_k q
// and the per-token sum of q (rowsum) is subtracted once in the epilogue; this is
// integer-exact.  One workgroup owns 32 columns for the whole of K: its 256 lanes
// are 8 (columns/4) x 32 (k slices); partial sums meet through DPP/LDS, never
// through global memory, and the epilogue is fused.
#include "common.hpp"

namespace {

constexpr int kThreads = 256;
constexpr int kTN = 8;                   // lanes along n; each covers 4 columns
constexpr int kTK = kThreads / kTN;      // 32 k-slices
constexpr int kColsPerBlock = kTN * 4;   // 32
// kIters weight loads are in flight per lane and chunk; a chunk spans kTK * kIters
// k-blocks (8 -> 4096 k).  Sixteen tokens use 4 so that the activation chunk stays
// within the 64 KiB of static LDS.

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

template <int MT, int kIters>
__global__ __launch_bounds__(kThreads) void gemv_t2_i8_kernel(
    const uint4 *__restrict__ q4,         // [M][KB] 16 int8 each
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint4 *__restrict__ w4,         // [KB][Npad/4]
    float w_scale, int M, int KB, int N, int npad4, int32_t *__restrict__ acc_out,
    float *__restrict__ out) {
    constexpr int kChunkKb = kTK * kIters;
    __shared__ uint4 s_a[MT * kChunkKb];             // activation chunk, MT x 4 KiB
    __shared__ int s_red[kThreads / 64][MT][kColsPerBlock];

    const int tid = threadIdx.x;
    const int tn = tid & (kTN - 1);
    const int tk = tid >> 3;
    const int col4 = blockIdx.x * kTN + tn;  // < npad4 by construction of the grid

    int acc[MT][4];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[m][c] = 0;

    for (int kc0 = 0; kc0 < KB; kc0 += kChunkKb) {
        // 1. put this chunk's weight loads in flight
        uint4 w[kIters];
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            int kb = kc0 + it * kTK + tk;
            w[it] = kb < KB ? w4[(size_t)kb * npad4 + col4]
                            : make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);
        }
        // 2. stage the activations of the chunk in LDS
        if (kc0 != 0) __syncthreads();
        if (tid < kChunkKb) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                int kb = kc0 + tid;
                uint4 a = make_uint4(0u, 0u, 0u, 0u);
                if (m < M && kb < KB) a = q4[(size_t)m * KB + kb];
                s_a[m * kChunkKb + tid] = a;
            }
        }
        __syncthreads();
        // 3. decode and accumulate
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const uint32_t ww[4] = {w[it].x, w[it].y, w[it].z, w[it].w};
            uint32_t b[4][4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                b[c][0] = ww[c] & 0x03030303u;
                b[c][1] = (ww[c] >> 2) & 0x03030303u;
                b[c][2] = (ww[c] >> 4) & 0x03030303u;
                b[c][3] = (ww[c] >> 6) & 0x03030303u;
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const uint4 a = s_a[m * kChunkKb + it * kTK + tk];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    int v = acc[m][c];
                    v = dot4(a.x, b[c][0], v);
                    v = dot4(a.y, b[c][1], v);
                    v = dot4(a.z, b[c][2], v);
                    v = dot4(a.w, b[c][3], v);
                    acc[m][c] = v;
                }
            }
        }
    }

    // 4. reduce over the 32 k-slices: 8 inside the wave (lane bits 3..5), then 4 waves.
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int v = acc[m][c];
            v += __shfl_xor(v, 8);
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            acc[m][c] = v;
        }
    const int lane = tid & 63, wave = tid >> 6;
    if (lane < kTN) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int c = 0; c < 4; ++c) s_red[wave][m][lane * 4 + c] = acc[m][c];
    }
    __syncthreads();
    // 5. fused epilogue: one thread per (m, column)
    for (int idx = tid; idx < MT * kColsPerBlock; idx += kThreads) {
        int m = idx / kColsPerBlock, c = idx % kColsPerBlock;
        int n = blockIdx.x * kColsPerBlock + c;
        if (m < M && n < N) {
            int total = s_red[0][m][c] + s_red[1][m][c] + s_red[2][m][c] + s_red[3][m][c];
            total -= rowsum[m];
            if (acc_out) acc_out[(size_t)m * N + n] = total;
            float r = (float)total * act_scale[m];  // kernels.rs:168, left to right
            r = r * w_scale;
            out[(size_t)m * N + n] = r;
        }
    }
}

template <int MT>
void launch(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale, const int32_t *d_rowsum,
            const uint32_t *d_tiled, float w_scale, int M, int KB, int N, int npad4,
            int32_t *d_acc, float *d_out) {
    dim3 grid((unsigned)(npad4 / kTN));
    gemv_t2_i8_kernel<MT, (MT >= 16 ? 4 : 8)><<<grid, dim3(kThreads), 0, ctx->stream>>>(
        (const uint4 *)d_q, d_act_scale, d_rowsum, (const uint4 *)d_tiled, w_scale, M, KB, N,
        npad4, d_acc, d_out);
}

}  // namespace

extern "C" int rbn_gemv_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                              const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                              uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc, float *d_out) {
    RBN_ENTER(ctx);
    RBN_REQUIRE(M > 0 && K > 0 && N > 0, "M, K and N must be positive");
    RBN_REQUIRE(M <= RBN_GEMV_MAX_M, "rbn_gemv_t2_i8 takes M <= %d (got %llu)", RBN_GEMV_MAX_M,
                (unsigned long long)M);
    RBN_REQUIRE(d_q && d_act_scale && d_rowsum && d_tiled && d_out, "null pointer in rbn_gemv_t2_i8");
    RBN_REQUIRE((((uintptr_t)d_q | (uintptr_t)d_tiled) & 15u) == 0,
                "d_q and d_tiled must be 16-byte aligned");
    RBN_REQUIRE(K <= (1ull << 30) && N <= (1ull << 30), "dimension too large");
    const int KB = (int)(rbn_kpad(K) / 16);
    const int npad4 = (int)(rbn_npad(N) / 4);
    const int m = (int)M, n = (int)N;
    if (m == 1)
        launch<1>(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, m, KB, n, npad4, d_acc, d_out);
    else if (m == 2)
        launch<2>(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, m, KB, n, npad4, d_acc, d_out);
    else if (m <= 4)
        launch<4>(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, m, KB, n, npad4, d_acc, d_out);
    else if (m <= 8)
        launch<8>(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, m, KB, n, npad4, d_acc, d_out);
    else
        launch<16>(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, m, KB, n, npad4, d_acc,
                   d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

// Prefill-regime ternary GEMM on the int8 matrix cores:
// out[m,n] = ((float)acc * act_scale[m]) * w_scale, acc = sum_k q[m,k] * w[k,n] (int32).
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (epilogue order :168).
//
// Shape of the kernel (v_mfma_i32_32x32x32_i8, 64-wide waves):
//  * Workgroup tile 128 (M) x 256 (N), K step 128 per barrier; four waves as 2 x 2, each
//    wave 64 x 128 = 2 x 4 MFMA tiles (128 accumulator registers), two workgroups per CU.
//  * Weights stay 2-bit until they are in registers.  The tiled layout keeps the four
//    columns of a quad in one 16-byte unit per 16 k, and a lane's B fragment for one MFMA
//    (sixteen consecutive k of one column) is one u32 of it.  Lane l therefore reads ONE
//    16-byte unit (quad l%32, k-half l/32) per K step of 32 and expands it with 28 VALU
//    operations into the B fragments of FOUR MFMA tiles: tile j covers the columns
//    4*quad + j.  The same mapping lets the epilogue store four adjacent columns per lane
//    as one 128-bit store.
//  * Both operands go through LDS, double-buffered: activations as int8 rows padded to
//    144 B, weights still packed (2 KiB per 32 k) in [k-block][quad] order with an XOR
//    swizzle so that the transposing store and the fragment loads are conflict-free.
//    Global loads are whole 128-byte lines for both operands.
//  * Workgroups are numbered so that the eight XCDs each own a band of rows: a band's
//    activations (128 rows x K) stay in that XCD's L2 while the weights stream through.
//  * Weights are stored as code = value + 1, so the per-token sum of q is subtracted in
//    the epilogue (integer-exact).
#include "common.hpp"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BM = 128, BN = 256, BK = 128;
constexpr int kARow = BK + 16;        // bytes per activation row in LDS
constexpr int kQuads = BN / 4;        // 64 column quads per workgroup tile
constexpr int kKb = BK / 16;          // 8 k-blocks per K step
constexpr int kABytes = BM * kARow;   // 18432

__device__ __forceinline__ v4i decode_b(uint32_t w) {
    v4i b;
    b.x = (int)(w & 0x03030303u);
    b.y = (int)((w >> 2) & 0x03030303u);
    b.z = (int)((w >> 4) & 0x03030303u);
    b.w = (int)((w >> 6) & 0x03030303u);
    return b;
}

// 16-byte slot of (k-block kb, quad q) inside the packed weight tile in LDS
__device__ __forceinline__ int b_slot(int kb, int q) { return kb * kQuads + (q ^ ((kb & 7) << 1)); }

__global__ __launch_bounds__(kThreads, 2) void gemm_t2_i8_mfma_kernel(
    const int8_t *__restrict__ q,         // [M][Kpad]
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint4 *__restrict__ wt,         // tiled: uint4 index quad * KB + kb
    float w_scale, int M, int Kpad, int N, int nquads, int m_tiles, int n_tiles,
    int32_t *__restrict__ acc_out, float *__restrict__ out) {
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][kABytes];
    __shared__ __attribute__((aligned(16))) uint4 s_b[2][kKb * kQuads];
    __shared__ float s_scale[BM];
    __shared__ int s_rowsum[BM];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int KB = Kpad >> 4;

    // XCD-aware numbering: consecutive workgroups land on consecutive XCDs; give each XCD
    // a band of m tiles and let it walk the n tiles.
    int bm, bn;
    if ((m_tiles & 7) == 0) {
        const int per = m_tiles >> 3;
        const int xcd = blockIdx.x & 7, i = blockIdx.x >> 3;
        bm = xcd * per + i % per;
        bn = i / per;
    } else {
        bm = blockIdx.x % m_tiles;
        bn = blockIdx.x / m_tiles;
    }
    const int m0 = bm * BM, n0 = bn * BN;
    const int q0 = n0 >> 2;

    if (tid < BM) {
        const int row = m0 + tid;
        s_scale[tid] = row < M ? act_scale[row] : 0.0f;
        s_rowsum[tid] = row < M ? rowsum[row] : 0;
    }

    v16i acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // staging assignments: A tile 128 rows x 128 B = 1024 units of 16 B (4 per thread);
    // B tile 64 quads x 8 k-blocks = 512 units (2 per thread)
    const int a_seg = tid & 7, a_row0 = tid >> 3;      // rows a_row0 + 32*j
    const int b_kb = tid & 7, b_q0 = tid >> 3;         // quads b_q0 + 32*j
    uint4 ra[4], rb[2];
    // Loads are unconditional (clamped addresses) and their results are not touched until
    // store_tiles(), after the MFMA section: anything that consumes a loaded register
    // earlier would make the compiler wait for the load in front of the matrix work.
    auto load_tiles = [&](int k0) {
        const int kb0 = k0 >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + a_row0 + 32 * j;
            const int k = k0 + a_seg * 16;
            ra[j] = *reinterpret_cast<const uint4 *>(q + (size_t)min(row, M - 1) * Kpad +
                                                     min(k, Kpad - 16));
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int quad = q0 + b_q0 + 32 * j;
            const int kb = kb0 + b_kb;
            rb[j] = wt[(size_t)min(quad, nquads - 1) * KB + min(kb, KB - 1)];
        }
    };
    // Out-of-range rows / k contribute zero activations; out-of-range columns / k get the
    // zero-weight code.
    auto store_tiles = [&](int buf, int k0) {
        const int kb0 = k0 >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + a_row0 + 32 * j;
            const int k = k0 + a_seg * 16;
            const uint32_t keep = (row < M && k < Kpad) ? 0xffffffffu : 0u;
            *reinterpret_cast<uint4 *>(&s_a[buf][(a_row0 + 32 * j) * kARow + a_seg * 16]) =
                make_uint4(ra[j].x & keep, ra[j].y & keep, ra[j].z & keep, ra[j].w & keep);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int quad = q0 + b_q0 + 32 * j;
            const bool ok = quad < nquads && kb0 + b_kb < KB;
            s_b[buf][b_slot(b_kb, b_q0 + 32 * j)] =
                make_uint4(ok ? rb[j].x : 0x55555555u, ok ? rb[j].y : 0x55555555u,
                           ok ? rb[j].z : 0x55555555u, ok ? rb[j].w : 0x55555555u);
        }
    };

    load_tiles(0);
    store_tiles(0, 0);
    __syncthreads();

    const int iters = (Kpad + BK - 1) / BK;
    const int a_lane_off = (lane & 31) * kARow + (lane >> 5) * 16;
    for (int it = 0; it < iters; ++it) {
        const int cur = it & 1;
        const bool more = it + 1 < iters;
        if (more) load_tiles((it + 1) * BK);
        __builtin_amdgcn_sched_barrier(0);
        // Fragments of K step ks+1 are fetched from LDS while the MFMAs of step ks run.
        uint4 bw = s_b[cur][b_slot(lane >> 5, wn * 32 + (lane & 31))];
        v4i af0 = *reinterpret_cast<const v4i *>(&s_a[cur][(wm * 64) * kARow + a_lane_off]);
        v4i af1 = *reinterpret_cast<const v4i *>(&s_a[cur][(wm * 64 + 32) * kARow + a_lane_off]);
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            uint4 bw_n = bw;
            v4i af0_n = af0, af1_n = af1;
            if (ks + 1 < BK / 32) {
                bw_n = s_b[cur][b_slot((ks + 1) * 2 + (lane >> 5), wn * 32 + (lane & 31))];
                af0_n = *reinterpret_cast<const v4i *>(
                    &s_a[cur][(wm * 64) * kARow + a_lane_off + (ks + 1) * 32]);
                af1_n = *reinterpret_cast<const v4i *>(
                    &s_a[cur][(wm * 64 + 32) * kARow + a_lane_off + (ks + 1) * 32]);
            }
            // B: one 16-byte unit per lane -> fragments of the four column tiles
            v4i bf[4];
            bf[0] = decode_b(bw.x);
            bf[1] = decode_b(bw.y);
            bf[2] = decode_b(bw.z);
            bf[3] = decode_b(bw.w);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf[j], acc[0][j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[1][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af1, bf[j], acc[1][j], 0, 0, 0);
            bw = bw_n;
            af0 = af0_n;
            af1 = af1_n;
        }
        __builtin_amdgcn_sched_barrier(0);
        if (more) store_tiles(cur ^ 1, (it + 1) * BK);
        __syncthreads();
    }

    // epilogue: lane owns columns 4*quad .. 4*quad+3 (tile j -> column 4*quad + j) and rows
    // 8*(r/4) + 4*(lane/32) + r%4 of each 32-row tile
    const int col0 = n0 + (wn * 32 + (lane & 31)) * 4;
    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int lrow = wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            const int row = m0 + lrow;
            if (row >= M || col0 >= N) continue;
            const int rs = s_rowsum[lrow];
            const float as = s_scale[lrow];
            int t[4];
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                t[j] = acc[mt][j][r] - rs;
                float f = (float)t[j] * as;  // kernels.rs:168, left to right
                v[j] = f * w_scale;
            }
            const size_t o = (size_t)row * N + col0;
            if (vec_ok) {
                *reinterpret_cast<float4 *>(out + o) = make_float4(v[0], v[1], v[2], v[3]);
                if (acc_out) *reinterpret_cast<int4 *>(acc_out + o) = make_int4(t[0], t[1], t[2], t[3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (col0 + j < N) {
                        out[o + j] = v[j];
                        if (acc_out) acc_out[o + j] = t[j];
                    }
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
    RBN_REQUIRE((((uintptr_t)d_out | (uintptr_t)d_acc) & 15u) == 0,
                "d_out and d_acc must be 16-byte aligned");
    RBN_REQUIRE(M <= (1ull << 24) && K <= (1ull << 24) && N <= (1ull << 24), "dimension too large");
    const int Kpad = (int)rbn_kpad(K);
    const int nquads = (int)(rbn_npad(N) / 4);
    const int m_tiles = (int)((M + BM - 1) / BM), n_tiles = (int)((N + BN - 1) / BN);
    const uint64_t tiles = (uint64_t)m_tiles * n_tiles;
    RBN_REQUIRE(tiles <= 0x7fffffffull, "too many tiles");
    gemm_t2_i8_mfma_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, ctx->stream>>>(
        d_q, d_act_scale, d_rowsum, (const uint4 *)d_tiled, w_scale, (int)M, Kpad, (int)N, nquads,
        m_tiles, n_tiles, d_acc, d_out);
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

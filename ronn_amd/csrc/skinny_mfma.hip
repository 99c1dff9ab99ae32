// Small-batch ternary matmul (2 <= M <= 64 tokens) on the int8 matrix cores:
// out[m,n] = ((float)acc * act_scale[m]) * w_scale, acc = sum_k q[m,k] * w[k,n] (int32).
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (epilogue order :168).
//
// With a handful of tokens the weights are still read once and dominate the traffic, so
// the kernel is shaped like a streaming read (bound: HBM), but the dot products of 16
// tokens x 64 columns x 64 k run as four v_mfma_i32_16x16x64_i8 instead of 1024 lane-wise
// dot instructions per wave.
//  * A workgroup owns 64 adjacent columns (16 column quads) and one slice of k; its waves
//    split the slice into contiguous ranges of 64-k steps and meet once, through LDS, at
//    the end.  Nothing is shared between waves before that: no barrier in the loop.
//  * Matrices with few columns are also split along k ACROSS workgroups, so that every CU
//    streams.  Each workgroup of a column group writes its int32 partial tile to a
//    workspace owned by the context, then takes a ticket from the group's counter; the
//    one that draws the last ticket adds the partials up (integer addition: any order
//    gives the same bits), runs the epilogue and resets the counter.  Nobody waits for
//    anybody, so the scheme cannot hang whatever order the workgroups run in.  The tiles
//    travel as device-scope atomic stores and loads (they go to the level of the memory
//    system that all eight XCDs share), ordered against the ticket by the stores' own
//    completion: a device-scope FENCE instead would write back and invalidate a whole L2
//    per wave, which costs ten times the rest of the kernel.
//  * Per step a lane loads ONE 16-byte unit of the tiled weights (quad lane%16, k-block
//    lane/16: a wave reads 16 x 64 B, each quad's bytes contiguous along k) and expands it
//    with 28 VALU operations into the B operands of four MFMAs; tile j covers the columns
//    4*quad + j, so that after the reduction four adjacent columns sit in one lane and
//    leave as one 128-bit store.
//  * The activations of a step (16 tokens x 64 k per row tile) come straight from global
//    memory, 16 bytes per lane; every workgroup re-reads the whole [M, K] block, which
//    lives in L2.  Spare token rows repeat the last row and are never stored.
//  * Loads run D steps ahead of the MFMAs in a register ring; all loads are unconditional
//    (indices clamped) so the compiler counts them statically and waits with
//    vmcnt(in flight), never vmcnt(0).
//  * Weights are code = value + 1; the per-token sum of q is subtracted in the epilogue.
#include "common.hpp"
#include <type_traits>

// Optional cycle stamps (built only with -DRBN_SK_TRACE, e.g. `make -B EXTRA=-DRBN_SK_TRACE`): every wave of
// the first 64 workgroups of skinny_dma_kernel records the shader clock at five points - kernel start,
// transfers issued, last MFMA done, past the join barrier, stores acknowledged - and
// rbn_debug_sk_trace copies the stamps to the host.  `python3 bench.py --kernel skinny_trace` prints them.
#ifdef RBN_SK_TRACE
__device__ long long g_sk_trace[64 * 16 * 8];
#define SK_STAMP(i)                                                                                      \
    do {                                                                                                 \
        if ((threadIdx.x & 63) == 0 && blockIdx.x < 64)                                                  \
            g_sk_trace[(blockIdx.x * 16 + (threadIdx.x >> 6)) * 8 + (i)] = (long long)__builtin_readcyclecounter(); \
    } while (0)
extern "C" int rbn_debug_sk_trace(long long *h_out, int count) {
    if (!h_out || count < 0 || count > 64 * 16 * 8) return RBN_ERR_INVALID;
    return hipMemcpyFromSymbol(h_out, HIP_SYMBOL(g_sk_trace), sizeof(long long) * (size_t)count) == hipSuccess
               ? RBN_OK
               : RBN_ERR_HIP;
}
#else
#define SK_STAMP(i)
#endif

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v4i decode_b(uint32_t w) {
    v4i b;
    b.x = (int)(w & 0x03030303u);
    b.y = (int)((w >> 2) & 0x03030303u);
    b.z = (int)((w >> 4) & 0x03030303u);
    b.w = (int)((w >> 6) & 0x03030303u);
    return b;
}

// 16 bytes to / from memory at device scope, as two relaxed 64-bit atomics.
__device__ __forceinline__ void store_device_scope(int4 *p, int4 v) {
    unsigned long long *q = reinterpret_cast<unsigned long long *>(p);
    __hip_atomic_store(q, (unsigned long long)(uint32_t)v.x | ((unsigned long long)(uint32_t)v.y << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + 1, (unsigned long long)(uint32_t)v.z | ((unsigned long long)(uint32_t)v.w << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int4 load_device_scope(const int4 *p) {
    unsigned long long *q = reinterpret_cast<unsigned long long *>(const_cast<int4 *>(p));
    const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_int4((int)(uint32_t)lo, (int)(uint32_t)(lo >> 32), (int)(uint32_t)hi, (int)(uint32_t)(hi >> 32));
}

__device__ __forceinline__ v4i as_v4i(uint4 a) {
    v4i r = {(int)a.x, (int)a.y, (int)a.z, (int)a.w};
    return r;
}

// MT row tiles of 16 tokens, NG groups of 64 columns per wave (the activation fragments are
// loaded once and used for all of them: with four row tiles the activations, not the
// weights, are most of the traffic), D steps of loads in flight, REFILL: some wave's range
// is longer than D steps, MAXW: most waves per workgroup (sets the register budget).
template <int MT, int NG, int D, bool REFILL, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void skinny_t2_i8_kernel(
    const int8_t *__restrict__ q,         // [M][Kpad], Kpad % 128 == 0
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint4 *__restrict__ wt,         // tiled: uint4 index quad * KB + kb
    float w_scale, int M, int Kpad, int N, int groups, int splits,
    int4 *__restrict__ partials,      // [groups][splits][MT * 16 rows][NG * 16 quads], splits > 1
    unsigned *__restrict__ tickets,   // [groups], zero between launches
    int32_t *__restrict__ acc_out, float *__restrict__ out) {
    extern __shared__ int4 red[];  // [waves][MT * 16 rows][NG * 16 quads]
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;
    const int ql = lane & 15, g = lane >> 4;
    const int KB = Kpad >> 4;
    const int steps = Kpad >> 6;
    // consecutive workgroups: same k slice, adjacent column groups
    const int group = blockIdx.x % groups, split = blockIdx.x / groups;
    // this wave's share of the steps (the host keeps splits * nw <= steps)
    const int gw = split * nw + wave, gn = splits * nw;
    const int s0 = gw * steps / gn, s1 = (gw + 1) * steps / gn;

    // a step advances both operands by four 16-byte units
    const int cgroups = (int)(((size_t)N + 63) >> 6);  // groups of 64 columns that exist
    const uint4 *wp[NG];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
        wp[ng] = wt + (size_t)(min(group * NG + ng, cgroups - 1) * 16 + ql) * KB + g;
    const uint4 *ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        ap[mt] = reinterpret_cast<const uint4 *>(q + (size_t)min(mt * 16 + ql, M - 1) * Kpad) + g;

    v4i acc[NG][MT][4];
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[ng][mt][j] = v4i{0, 0, 0, 0};

    uint4 wr[D][NG], ar[D][MT];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const int s = max(min(s0 + d, s1 - 1), 0);  // never below step 0, whatever the launch shape
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ar[d][mt] = ap[mt][4 * s];
#pragma unroll
        for (int ng = 0; ng < NG; ++ng) wr[d][ng] = wp[ng][4 * s];
        // same issue order as the reloads in the loop, so that one wait count fits both
        __builtin_amdgcn_sched_barrier(0);
    }

    auto consume = [&](const uint4 (&w)[NG], const uint4 (&a)[MT]) {
#pragma unroll
        for (int ng = 0; ng < NG; ++ng) {
            const v4i b0 = decode_b(w[ng].x), b1 = decode_b(w[ng].y), b2 = decode_b(w[ng].z),
                      b3 = decode_b(w[ng].w);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const v4i af = as_v4i(a[mt]);
                acc[ng][mt][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, b0, acc[ng][mt][0], 0, 0, 0);
                acc[ng][mt][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, b1, acc[ng][mt][1], 0, 0, 0);
                acc[ng][mt][2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, b2, acc[ng][mt][2], 0, 0, 0);
                acc[ng][mt][3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, b3, acc[ng][mt][3], 0, 0, 0);
            }
        }
    };

    // Groups of D steps.  Slot d is multiplied, then reloaded in place with step s + D
    // (taking a copy of the slot in order to reload it earlier costs register moves that
    // wait for the whole ring).  Every wave runs whole groups: steps past its range are
    // clamped re-reads of its last step (cache hits) multiplied with zeroed activations.
    // That keeps the loop free of branches; with a branch around a step the compiler sinks
    // that step's loads into it, behind all the others, and the first wait becomes a wait
    // for everything.  Without REFILL the ring already holds the whole range.
    // sched_barrier keeps the steps apart: hoisting every expansion above the first MFMA
    // would multiply the live registers.
    int base = s0;
    do {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const uint32_t keep = base + d < s1 ? 0xffffffffu : 0u;
            uint4 a[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                a[mt] = make_uint4(ar[d][mt].x & keep, ar[d][mt].y & keep, ar[d][mt].z & keep,
                                   ar[d][mt].w & keep);
            consume(wr[d], a);
            if (REFILL) {
                const int sn = max(min(base + d + D, s1 - 1), 0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) ar[d][mt] = ap[mt][4 * sn];
#pragma unroll
                for (int ng = 0; ng < NG; ++ng) wr[d][ng] = wp[ng][4 * sn];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        base += D;
    } while (REFILL && base < s1);

    // Meet through LDS.  acc[ng][mt][j][i] is row mt*16 + 4*g + i, column 4*ql + j of the
    // ng-th group of 64 columns: one int4 per (row, quad).
    constexpr int rows = MT * 16, quads = NG * 16;
#pragma unroll
    for (int ng = 0; ng < NG; ++ng)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[(wave * rows + mt * 16 + 4 * g + i) * quads + ng * 16 + ql] = make_int4(
                    acc[ng][mt][0][i], acc[ng][mt][1][i], acc[ng][mt][2][i], acc[ng][mt][3][i]);
    __syncthreads();

    const bool vec_ok = (N & 3) == 0;
    auto finish = [&](int idx, int4 t) {
        const int row = idx / quads, qd = idx - row * quads;
        const int col0 = (group * quads + qd) * 4;
        if (row >= M || col0 >= N) return;
        const int rs = rowsum[row];
        const float as = act_scale[row];
        const int ti[4] = {t.x - rs, t.y - rs, t.z - rs, t.w - rs};
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float f = (float)ti[j] * as;  // kernels.rs:168, left to right
            v[j] = f * w_scale;
        }
        const size_t o = (size_t)row * N + col0;
        if (vec_ok) {
            *reinterpret_cast<float4 *>(out + o) = make_float4(v[0], v[1], v[2], v[3]);
            if (acc_out) *reinterpret_cast<int4 *>(acc_out + o) = make_int4(ti[0], ti[1], ti[2], ti[3]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (col0 + j < N) {
                    out[o + j] = v[j];
                    if (acc_out) acc_out[o + j] = ti[j];
                }
            }
        }
    };

    constexpr int tile = rows * quads;  // int4 entries of one partial tile
    int4 *mine = partials + ((size_t)group * splits + split) * tile;
    for (int idx = tid; idx < tile; idx += blockDim.x) {
        int4 t = red[idx];
        for (int w = 1; w < nw; ++w) {
            const int4 p = red[w * tile + idx];
            t.x += p.x;
            t.y += p.y;
            t.z += p.z;
            t.w += p.w;
        }
        if (splits == 1)
            finish(idx, t);
        else
            store_device_scope(mine + idx, t);
    }
    if (splits == 1) return;

    // The tile is published once its stores have completed: vmcnt(0) waits for this
    // wave's (a store leaves the counter when the memory system has acknowledged it), the
    // barrier for everybody's; then one thread draws.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(&tickets[group], 1u);
        const int last = ticket == (unsigned)splits - 1;
        if (last) atomicExch(&tickets[group], 0u);  // ready for the next launch
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    // every other workgroup of the group drew before this one, so its tile is complete
    const int4 *all = partials + (size_t)group * splits * tile;
    for (int idx = tid; idx < tile; idx += blockDim.x) {
        int4 t;
        if (splits == 2) {
            const int4 a = load_device_scope(all + idx), b = load_device_scope(all + tile + idx);
            t = make_int4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
        } else {
            // four tiles per round with their loads in flight together (clamped: the spare
            // ones re-read the last tile and add 0); one load after the other cost 0.7-1.1 us
            // with three and four parts
            t = make_int4(0, 0, 0, 0);
            for (int sp0 = 0; sp0 < splits; sp0 += 4) {
                int4 p[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    p[i] = load_device_scope(all + (size_t)min(sp0 + i, splits - 1) * tile + idx);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int keep = sp0 + i < splits ? -1 : 0;
                    t.x += p[i].x & keep;
                    t.y += p[i].y & keep;
                    t.z += p[i].z & keep;
                    t.w += p[i].w & keep;
                }
            }
        }
        finish(idx, t);
    }
}

struct Args {
    const int8_t *q;
    const float *act_scale;
    const int32_t *rowsum;
    const uint4 *wt;
    float w_scale;
    int M, Kpad, N, groups, splits, waves;
    int4 *partials;
    unsigned *tickets;
    int32_t *acc;
    float *out;
};

// Most waves per workgroup: bounded by registers (launch bounds) and by the reduction
// buffer, waves * MT * NG * 4 KiB of LDS (at most 128 KiB).
template <int MT, int NG>
constexpr int max_waves() { return MT * NG >= 8 ? 4 : (MT * NG >= 4 ? 8 : 16); }

template <int MT, int NG, int D, bool REFILL>
int launch(hipStream_t stream, const Args &a) {
    const size_t lds = (size_t)a.waves * MT * NG * 16 * 16 * sizeof(int4);
    skinny_t2_i8_kernel<MT, NG, D, REFILL, max_waves<MT, NG>()>
        <<<dim3((unsigned)(a.groups * a.splits)), dim3((unsigned)a.waves * 64), lds, stream>>>(
            a.q, a.act_scale, a.rowsum, a.wt, a.w_scale, a.M, a.Kpad, a.N, a.groups, a.splits,
            a.partials, a.tickets, a.acc, a.out);
    return RBN_OK;
}

// More than the default 64 KiB of dynamic LDS has to be asked for per kernel function.
template <int MT, int NG, int D, bool REFILL>
hipError_t allow_large_lds() {
    return hipFuncSetAttribute(
        reinterpret_cast<const void *>(skinny_t2_i8_kernel<MT, NG, D, REFILL, max_waves<MT, NG>()>),
        hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
}

// D: the smallest ring that holds a wave's whole range, else the deepest with reloads.
template <int MT, int NG>
int launch_d(hipStream_t stream, const Args &a) {
    const int steps = a.Kpad / 64, gn = a.splits * a.waves;
    const int longest = (steps + gn - 1) / gn;  // a wave gets floor or ceil of steps / gn
    if (longest <= 2) return launch<MT, NG, 2, false>(stream, a);
    if constexpr (MT * NG >= 8) {
        return launch<MT, NG, 2, true>(stream, a);
    } else {
        if (longest <= 4) return launch<MT, NG, 4, false>(stream, a);
        if constexpr (MT == 1) {
            if (longest <= 8) return launch<MT, NG, 8, false>(stream, a);
            return launch<MT, NG, 8, true>(stream, a);
        } else {
            return launch<MT, NG, 4, true>(stream, a);
        }
    }
}


// ---- up to 16 tokens: operands through LDS ------------------------------------------------
// The MFMA operand layout wants lane l to hold (quad l%16, k-block l/16) of the weights and
// (token l%16, k-block l/16) of the activations: sixty-four lanes, sixty-four different cache
// lines.  Loaded straight into registers that way, the texture addresser takes the lanes of a
// load one by one - measured with cycle counters, each SIMD of a CU got its next wave's
// eight loads issued ~2200 cycles after the previous wave's, so the sixteenth wave of a
// workgroup had its data ~8800 cycles after the first and everybody waited for it at the
// barrier.  Here the loads are global -> LDS transfers (global_load_lds_dwordx4) whose eight
// consecutive lanes fetch one 128-byte line - a quad's eight k-blocks, a token's 128 k - into a
// ring that each wave owns; the fragments are then read from LDS in operand order.  The LDS
// image is the prefill kernel's: unit row*8 + (slot ^ ((row>>1)&7)), which makes the 128-bit
// reads of sixteen consecutive lanes conflict-free.
// A stage is 128 k: two loads of weights (quads 0-7, 8-15) and two of activations (tokens
// 0-7, 8-15), 4 KiB of LDS.  Waves split k as before and never share a stage: no barrier in
// the loop.  The transfers are issued from inline assembly, so they are counted by hand:
// before stage d is read, s_waitcnt vmcnt leaves only the stages issued after it in flight.

typedef void __attribute__((address_space(3))) * lds_ptr;

__device__ __forceinline__ void dma16(const void *base, uint32_t lane_offset, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_wave_base), "v"(lane_offset), "s"(base)
                 : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vm() {
    static_assert(N >= 0 && N < 64, "vmcnt is six bits");
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

constexpr int kStageUnits = 256;  // 16-byte units of one stage: weights 0-127, activations 128-255

// HALF: at most eight tokens - the transfer of tokens 8-15 is left out (their rows of the stage
// keep whatever LDS held; the MFMA rows they feed are never stored).  WHALF: the workgroup owns at
// most eight column quads - the transfer of quads 8-15 is left out likewise (their columns are never
// stored).
// A workgroup owns the quads [group * nquads / groups, (group + 1) * nquads / groups): sixteen when
// there are at least as many groups of sixteen as the launch wants workgroups, fewer when the host
// spreads a narrower matrix over more workgroups so that every CU streams a share of the weights
// (what one CU can keep in flight is a quarter of a megabyte per microsecond or so; 4096 x 11008 on
// 172 workgroups of sixteen quads gave each CU 64 KiB to pull, on 256 workgroups 43 KiB).
template <int D, bool REFILL, bool HALF, bool WHALF>
__global__ __launch_bounds__(1024) void skinny_dma_kernel(
    const int8_t *__restrict__ q,         // [M][Kpad], Kpad % 128 == 0, M <= 16
    const float *__restrict__ act_scale, const int32_t *__restrict__ rowsum,
    const uint4 *__restrict__ wt,         // tiled: uint4 index quad * KB + kb
    float w_scale, int M, int Kpad, int N, int nquads /* of the tiled buffer: a multiple of 16 */, int groups,
    int splits, int4 *__restrict__ partials, unsigned *__restrict__ tickets,
    int32_t *__restrict__ acc_out, float *__restrict__ out) {
    extern __shared__ uint4 ring[];  // [waves][D][kStageUnits]; reused as [waves][256] int4 for the join
    __shared__ int s_last;

    SK_STAMP(0);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;
    const int ql = lane & 15, g = lane >> 4;
    const int KB = Kpad >> 4;
    const int stages = Kpad >> 7;  // of 128 k
    const int group = blockIdx.x % groups, split = blockIdx.x / groups;
    const int gw = split * nw + wave, gn = splits * nw;
    const int s0 = gw * stages / gn, s1 = (gw + 1) * stages / gn;  // >= 1 stage (the host sees to it)
    // this workgroup's quads: 1 to 16 of them (the host keeps nquads / groups within that)
    const int q_lo = (int)(((long long)group * nquads) / groups);
    const int nq = min(max((int)(((long long)(group + 1) * nquads) / groups) - q_lo, 1), 16);

    // transfer h of a stage: row (quad or token) 8h + lane/8, slot lane%8 holding k-block
    // slot ^ ((row>>1)&7) of the stage's eight; rows past the workgroup's quads or the tokens that
    // exist repeat the last one (fetched again, never stored)
    const int sub = lane >> 3, slot = lane & 7;
    uint32_t w_off[2], a_off[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = 8 * h + sub;
        const int kb = slot ^ ((row >> 1) & 7);
        w_off[h] = ((uint32_t)min(row, nq - 1) * (uint32_t)KB + (uint32_t)kb) * 16u;
        a_off[h] = (uint32_t)min(row, M - 1) * (uint32_t)Kpad + (uint32_t)kb * 16u;
    }
    const uint4 *w_base = wt + (size_t)min(q_lo, nquads - 1) * KB;
    // The epilogue's per-token scalars, asked for before the transfers (the memory counter retires in
    // order, and the hand-counted waits below count transfers only): a thread finishes the elements
    // tid, tid + blockDim.x, ... of the 16 x 16 tile, element e belonging to token e / 16.  Fetched at the
    // end they were a dependent round trip after the join barrier.
    int rs_pre[4] = {0, 0, 0, 0};
    float as_pre[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // a workgroup of one wave finishes four elements per thread, of four or more one
        const int idx = tid + j * (int)blockDim.x;
        if (idx < 256) {
            const int row = min(idx >> 4, M - 1);
            rs_pre[j] = rowsum[row];
            as_pre[j] = act_scale[row];
        }
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)ring + (uint32_t)wave * (D * kStageUnits * 16);
    auto issue = [&](int s, int d) {
        // past the range: a re-read of the last stage, multiplied by zero (and never below stage 0,
        // whatever the launch shape: the address must stay inside the matrix)
        const int sc = max(min(s, s1 - 1), 0);
        const uint4 *wb = w_base + (size_t)sc * 8;
        const int8_t *ab = q + (size_t)sc * 128;
        const uint32_t at = lds0 + (uint32_t)d * (kStageUnits * 16);
        dma16(wb, w_off[0], at);
        if (!WHALF) dma16(wb, w_off[1], at + 1024);
        dma16(ab, a_off[0], at + 2048);
        if (!HALF) dma16(ab, a_off[1], at + 3072);
    };
    constexpr int LPS = 4 - (HALF ? 1 : 0) - (WHALF ? 1 : 0);  // transfers per stage
#pragma unroll
    for (int d = 0; d < D; ++d) issue(s0 + d, d);
    SK_STAMP(1);

    // fragment positions inside a stage: row ql (quad for the weights, token for the
    // activations), k-block 4t + g for the two halves t of the stage
    int f_off[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) f_off[t] = ql * 8 + ((4 * t + g) ^ ((ql >> 1) & 7));

    v4i acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = v4i{0, 0, 0, 0};
    const uint4 *mine = ring + (size_t)wave * (D * kStageUnits);

    auto consume = [&](int d, uint32_t keep) {
        const uint4 *st = mine + d * kStageUnits;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint4 w = st[f_off[t]];
            const uint4 a = st[128 + f_off[t]];
            const v4i af = {(int)(a.x & keep), (int)(a.y & keep), (int)(a.z & keep), (int)(a.w & keep)};
            acc[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, decode_b(w.x), acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, decode_b(w.y), acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, decode_b(w.z), acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, decode_b(w.w), acc[3], 0, 0, 0);
        }
    };

    if (!REFILL) {
        // the ring holds the whole range: stage d has landed when only the 4 (D-1-d) later
        // transfers are outstanding
        auto step = [&](auto dt) {
            constexpr int d = decltype(dt)::value;
            wait_vm<LPS * (D - 1 - d)>();
            consume(d, s0 + d < s1 ? 0xffffffffu : 0u);
        };
        step(std::integral_constant<int, 0>{});
        if constexpr (D > 1) step(std::integral_constant<int, 1>{});
        if constexpr (D > 2) step(std::integral_constant<int, 2>{});
        if constexpr (D > 3) step(std::integral_constant<int, 3>{});
    } else {
        // rounds of D stages; stage d is refilled with stage s + D as soon as its fragments are in
        // registers (lgkmcnt(0): the reads have returned before the transfer may overwrite them)
        int base = s0;
        do {
            auto step = [&](auto dt) {
                constexpr int d = decltype(dt)::value;
                wait_vm<LPS * (D - 1)>();
                consume(d, base + d < s1 ? 0xffffffffu : 0u);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                issue(base + d + D, d);
            };
            step(std::integral_constant<int, 0>{});
            if constexpr (D > 1) step(std::integral_constant<int, 1>{});
            if constexpr (D > 2) step(std::integral_constant<int, 2>{});
            if constexpr (D > 3) step(std::integral_constant<int, 3>{});
            base += D;
        } while (base < s1);
        wait_vm<0>();  // the last refills (re-reads) must not land on the join below
    }

    SK_STAMP(2);
    // Join through LDS, each wave writing into its own ring space.  acc[j][i] is token 4*g + i,
    // column 4*ql + j: one int4 per (token, quad).
    constexpr int quads = 16, tile = 16 * quads;
    int4 *red = reinterpret_cast<int4 *>(ring);
    constexpr int wstride = D * kStageUnits;  // int4 units between two waves' spaces
#pragma unroll
    for (int i = 0; i < 4; ++i)
        red[wave * wstride + (4 * g + i) * quads + ql] = make_int4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
    __syncthreads();
    SK_STAMP(3);

    const bool vec_ok = (N & 3) == 0;
    auto finish = [&](int idx, int j, int4 t) {  // idx = tid + j * blockDim.x
        const int row = idx / quads, qd = idx - row * quads;
        const int col0 = (q_lo + qd) * 4;
        if (row >= M || qd >= nq || col0 >= N) return;
        const int rs = rs_pre[j];
        const float as = as_pre[j];
        const int ti[4] = {t.x - rs, t.y - rs, t.z - rs, t.w - rs};
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float f = (float)ti[j] * as;  // kernels.rs:168, left to right
            v[j] = f * w_scale;
        }
        const size_t o = (size_t)row * N + col0;
        if (vec_ok) {
            *reinterpret_cast<float4 *>(out + o) = make_float4(v[0], v[1], v[2], v[3]);
            if (acc_out) *reinterpret_cast<int4 *>(acc_out + o) = make_int4(ti[0], ti[1], ti[2], ti[3]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (col0 + j < N) {
                    out[o + j] = v[j];
                    if (acc_out) acc_out[o + j] = ti[j];
                }
            }
        }
    };

    int4 *my_part = partials + ((size_t)group * splits + split) * tile;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int idx = tid + j * (int)blockDim.x;
        if (idx >= tile) break;
        int4 t = red[idx];
        for (int w = 1; w < nw; ++w) {
            const int4 p = red[w * wstride + idx];
            t.x += p.x;
            t.y += p.y;
            t.z += p.z;
            t.w += p.w;
        }
        if (splits == 1)
            finish(idx, j, t);
        else
            store_device_scope(my_part + idx, t);
    }
    if (splits == 1) {
#ifdef RBN_SK_TRACE
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        SK_STAMP(4);
#endif
        return;
    }

    // same publication and ticket scheme as skinny_t2_i8_kernel
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = atomicAdd(&tickets[group], 1u);
        const int last = ticket == (unsigned)splits - 1;
        if (last) atomicExch(&tickets[group], 0u);
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    const int4 *all = partials + (size_t)group * splits * tile;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int idx = tid + j * (int)blockDim.x;
        if (idx >= tile) break;
        int4 t = make_int4(0, 0, 0, 0);
        for (int sp0 = 0; sp0 < splits; sp0 += 4) {
            int4 p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = load_device_scope(all + (size_t)min(sp0 + i, splits - 1) * tile + idx);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int keep = sp0 + i < splits ? -1 : 0;
                t.x += p[i].x & keep;
                t.y += p[i].y & keep;
                t.z += p[i].z & keep;
                t.w += p[i].w & keep;
            }
        }
        finish(idx, j, t);
    }
}

template <int D, bool REFILL>
int launch_dma(hipStream_t stream, const Args &a) {
    const size_t lds = (size_t)a.waves * D * kStageUnits * 16;
    const dim3 grid((unsigned)(a.groups * a.splits)), block((unsigned)a.waves * 64);
    const int nquads = (int)(rbn_npad((uint64_t)a.N) / 4);
    const bool half = a.M <= 8;                                   // no token beyond the eighth
    const bool whalf = (nquads + a.groups - 1) / a.groups <= 8;   // no workgroup with more than eight quads
    auto go = [&](auto kernel) {
        kernel<<<grid, block, lds, stream>>>(a.q, a.act_scale, a.rowsum, a.wt, a.w_scale, a.M, a.Kpad, a.N, nquads,
                                             a.groups, a.splits, a.partials, a.tickets, a.acc, a.out);
    };
    if (half && whalf)
        go(skinny_dma_kernel<D, REFILL, true, true>);
    else if (half)
        go(skinny_dma_kernel<D, REFILL, true, false>);
    else if (whalf)
        go(skinny_dma_kernel<D, REFILL, false, true>);
    else
        go(skinny_dma_kernel<D, REFILL, false, false>);
    return RBN_OK;
}

template <int D, bool REFILL>
hipError_t allow_large_lds_dma() {
    const void *fns[] = {reinterpret_cast<const void *>(skinny_dma_kernel<D, REFILL, true, true>),
                         reinterpret_cast<const void *>(skinny_dma_kernel<D, REFILL, true, false>),
                         reinterpret_cast<const void *>(skinny_dma_kernel<D, REFILL, false, true>),
                         reinterpret_cast<const void *>(skinny_dma_kernel<D, REFILL, false, false>)};
    for (const void *f : fns) {
        const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace

// Scratch of the entry point that allocates nothing (rbn_gemm_t2_i8_skinny_static): partial
// tiles first, then the ticket counters.  One copy per GPU, held until the process ends.
constexpr int kStaticTiles = 1024;   // partial tiles of 16 x 64 int32 (4 KiB each): 4 MiB
constexpr int kStaticGroups = 128;   // ticket counters (a split launch has fewer than 128 column groups)
constexpr size_t kStaticBytes = (size_t)kStaticTiles * 4096 + (size_t)kStaticGroups * sizeof(unsigned);
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_lock;
static void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, 0 until prepared
// The context that uses a GPU's static scratch: the first one to call the entry point, until it
// is destroyed.  Calls from two contexts would run on two streams and corrupt each other's
// partial tiles and counters, so a second context is refused instead.
static const rbn_ctx *g_scratch_owner[kMaxDevices];

void rbn_skinny_release(const rbn_ctx *ctx) {
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    for (int d = 0; d < kMaxDevices; ++d)
        if (g_scratch_owner[d] == ctx) g_scratch_owner[d] = nullptr;
}

__global__ void clear_tickets_kernel(unsigned *tickets, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) tickets[i] = 0u;
}

// Called once per context, with the context's device current and outside any stream capture:
// raises the dynamic-LDS limit of every instantiation that launch_d can pick and looks up this
// device's copy of the static scratch array.
int rbn_skinny_prepare(int device) {
    const hipError_t results[] = {
        allow_large_lds<1, 1, 2, false>(), allow_large_lds<1, 1, 4, false>(),
        allow_large_lds<1, 1, 8, false>(), allow_large_lds<1, 1, 8, true>(),
        allow_large_lds<2, 1, 2, false>(), allow_large_lds<2, 1, 4, false>(),
        allow_large_lds<2, 1, 4, true>(),  allow_large_lds<4, 1, 2, false>(),
        allow_large_lds<4, 1, 4, false>(), allow_large_lds<4, 1, 4, true>(),
        allow_large_lds<4, 2, 2, false>(), allow_large_lds<4, 2, 2, true>(),
    };
    const hipError_t results_dma[] = {allow_large_lds_dma<1, false>(), allow_large_lds_dma<2, false>(),
                                      allow_large_lds_dma<2, true>()};
    for (hipError_t e : results_dma)
        if (e != hipSuccess)
            return rbn_fail(RBN_ERR_HIP, "hipFuncSetAttribute(max dynamic LDS) failed: %s", hipGetErrorString(e));
    for (hipError_t e : results)
        if (e != hipSuccess)
            return rbn_fail(RBN_ERR_HIP, "hipFuncSetAttribute(max dynamic LDS) failed: %s",
                            hipGetErrorString(e));
    if (device < 0 || device >= kMaxDevices)
        return rbn_fail(RBN_ERR_UNSUPPORTED, "device index %d beyond the %d this library keeps scratch for",
                        device, kMaxDevices);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (g_scratch_ptr[device] == nullptr) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr)
            return rbn_fail(RBN_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", device,
                            hipGetErrorString(e));
        g_scratch_ptr[device] = ptr;
    }
    return RBN_OK;
}

// The launch shape of a small-batch product: which kernel, how many column groups, how k is split
// across workgroups and waves.  Pure arithmetic (no device), so the rules can be swept on the CPU.
struct SkinnyPlan {
    int mt, ng;       // row tiles of 16 tokens, groups of 64 columns per wave
    int groups;       // workgroups along N
    int splits;       // workgroups sharing a column group along k
    int waves;        // per workgroup
    int step_k;       // k of one step of a wave's range: 64 (register ring) or 128 (LDS ring)
    int steps;        // steps in all = Kpad / step_k
    int longest;      // most steps any wave gets
    int lds_ring;     // 1: skinny_dma_kernel (up to 16 tokens), 0: skinny_t2_i8_kernel
    int64_t tiles;    // partial tiles of 16 x 64 int32 the exchange needs (0 without a split)
    size_t lds_bytes;
};

// Returns false when `strict` and the exchange does not fit max_tiles / max_groups (the plan then
// holds what would have been needed); otherwise the split is reduced until it fits.
static bool plan_skinny(uint64_t M, uint64_t K, uint64_t N, int max_tiles, int max_groups, bool strict,
                        SkinnyPlan *p) {
    const int Kpad = (int)rbn_kpad(K);
    const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    // four row tiles and a wide matrix: a wave takes two groups of 64 columns, which halves
    // the activation traffic (8192 x 28672, M = 64: 55 -> 43 us); narrower matrices need
    // the workgroups more than the saving (4096 x 11008: 18 us with one group, 28 with two)
    const int cgroups = (int)(rbn_npad(N) / 64);
    const int ng = (mt == 4 && cgroups >= 256) ? 2 : 1;
    int groups = (cgroups + ng - 1) / ng;
    // Shape of the launch (measured on the decode shapes; 64-k steps per wave in brackets).
    // With enough column groups, one workgroup per group: 4096 x 11008 runs 16 waves [4],
    // 8192 x 28672 16 waves [8].  Narrower matrices are also split along k across
    // workgroups, towards ~256 of them; the round trip of the partial tiles through
    // memory costs 1-2 us, which is why wide matrices are not split.  A wave should get 4
    // steps (a ring of 4 with nothing masked), or 8 and more when the workgroup is full.
    const int steps = Kpad / 64;
    const int max_w = mt == 4 ? (ng == 2 ? max_waves<4, 2>() : max_waves<4, 1>())
                              : (mt == 2 ? max_waves<2, 1>() : max_waves<1, 1>());
    int splits = 1;
    if (groups < 128 || groups * max_w < 1024) splits = (256 + groups - 1) / groups;
    if (splits > steps / 4) splits = steps / 4 > 0 ? steps / 4 : 1;
    // ... and a split should keep 32 steps or more (48 up to 8 tokens): below that the round
    // trip of the partial tiles costs more than the extra workgroups bring (2560 x 2560,
    // M = 4: 8.5 us with 7 splits, 4.5 with one; 4096 x 256: 19 -> 5 us)
    {
        const int per = M <= 8 ? 48 : 32;
        const int want = (steps + per - 1) / per;
        if (want < splits) splits = want;
    }
    // Up to 16 tokens with a short k (the activation block is at most 64 KiB): where the rule above
    // would split along k, the matrix is cut along N instead, into up to 256 workgroups of four to
    // sixteen quads (the kernel gives workgroup g the quads [g * nquads / groups, (g + 1) * nquads /
    // groups)).  Every workgroup then reads the whole activation block, but nothing is exchanged
    // through memory: 4096 x 4096 5.6-5.9 -> 5.2-5.5 us, 2560 x 7680 and 2560 x 2560 at 16 tokens
    // 5.7 -> 5.0 and 5.2 -> 4.5 us.  With a longer k the activation traffic of that many workgroups
    // outweighs the exchange (11008 x 4096: 7.1 -> 8.3-9.5 us), and a matrix that needs no split gains
    // nothing from more workgroups (4096 x 11008 on 256 instead of 172: 5.9 -> 6.2 us).
    if (mt == 1 && splits > 1 && Kpad <= 4096) {
        const int nquads = cgroups * 16;
        int wide = nquads / 4 < 256 ? nquads / 4 : 256;
        if (wide > groups) {
            groups = wide;
            splits = 1;
        }
    }
    // the exchange area holds max_tiles tiles of 16 x 64 int32 and one ticket per group
    bool fits = true;
    if (strict) {
        fits = !(splits > 1 && ((int64_t)groups * splits * mt * ng > max_tiles || groups > max_groups));
    } else {
        while (splits > 1 && ((int64_t)groups * splits * mt * ng > max_tiles || groups > max_groups)) --splits;
    }
    const int steps_per_split = (steps + splits - 1) / splits;
    int waves = (steps_per_split + 3) / 4;
    if (waves > max_w) waves = max_w;
    if (waves > steps / splits) waves = steps / splits;  // every wave needs a step
    if (waves < 1) waves = 1;
    p->mt = mt;
    p->ng = ng;
    p->groups = groups;
    p->lds_ring = mt == 1;
    p->step_k = 64;
    p->steps = steps;
    if (p->lds_ring) {
        // stages of 128 k; a wave takes about two, every wave at least one
        const int stages = Kpad / 128;
        if (splits > stages) splits = stages;
        const int per_split = (stages + splits - 1) / splits;
        int w2 = (per_split + 1) / 2;
        if (w2 > 16) w2 = 16;
        // more workgroups than CUs: four waves (32 KiB of ring) let up to four workgroups share a CU,
        // so that all of them are resident at once instead of running in rounds (8192 x 28672, M = 8:
        // 18.5 us with sixteen waves, 14.9 with eight, 13.7 with four)
        if (groups * splits > 256 && w2 > 4) w2 = 4;
        if (w2 > stages / splits) w2 = stages / splits;
        if (w2 < 1) w2 = 1;
        waves = w2;
        p->step_k = 128;
        p->steps = stages;
    }
    p->splits = splits;
    p->waves = waves;
    const int gn = splits * waves;
    p->longest = (p->steps + gn - 1) / gn;
    p->tiles = splits > 1 ? (int64_t)groups * splits * mt * ng : 0;
    p->lds_bytes = p->lds_ring ? (size_t)waves * (p->longest <= 1 ? 1 : 2) * kStageUnits * 16
                               : (size_t)waves * mt * ng * 16 * 16 * sizeof(int4);
    return fits;
}

// What the kernels assume of a launch shape and cannot check themselves.
static bool plan_is_launchable(const SkinnyPlan &p) {
    return p.groups >= 1 && p.splits >= 1 && p.waves >= 1 && p.waves <= 16 &&
           (int64_t)p.splits * p.waves <= p.steps &&  // every wave owns at least one step
           p.lds_bytes <= 128 * 1024 && (int64_t)p.groups * p.splits < (1ll << 31);
}

extern "C" int rbn_skinny_launch_shape(uint64_t M, uint64_t K, uint64_t N, int32_t shape[8]) {
    if (!shape || M == 0 || M > RBN_SKINNY_MAX_M || K == 0 || N == 0 || K > (1ull << 24) || N > (1ull << 24))
        return RBN_ERR_INVALID;
    SkinnyPlan p;
    plan_skinny(M, K, N, RBN_SPLITK_TILES, RBN_SPLITK_GROUPS, false, &p);
    shape[0] = p.lds_ring;
    shape[1] = p.groups;
    shape[2] = p.splits;
    shape[3] = p.waves;
    shape[4] = p.step_k;
    shape[5] = p.steps;
    shape[6] = p.longest;
    shape[7] = (int32_t)p.lds_bytes;
    return plan_is_launchable(p) ? RBN_OK : RBN_ERR_UNSUPPORTED;
}

// partials / tickets: the split-k exchange area and what it holds (tiles of 4 KiB, counters).
// With `strict` a launch shape that does not fit is an error; otherwise the split is reduced
// until it fits (any split gives the same bits).
static int skinny_impl(rbn_ctx *ctx, const char *name, const int8_t *d_q, const float *d_act_scale,
                       const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale, uint64_t M,
                       uint64_t K, uint64_t N, int32_t *d_acc, float *d_out, void *partials,
                       unsigned *tickets, int max_tiles, int max_groups, bool strict) {
    RBN_REQUIRE(M > 0 && K > 0 && N > 0, "M, K and N must be positive");
    RBN_REQUIRE(M <= RBN_SKINNY_MAX_M, "%s takes M <= %d (got %llu)", name, RBN_SKINNY_MAX_M,
                (unsigned long long)M);
    RBN_REQUIRE(d_q && d_act_scale && d_rowsum && d_tiled && d_out, "null pointer in %s", name);
    RBN_REQUIRE((((uintptr_t)d_q | (uintptr_t)d_tiled) & 15u) == 0,
                "d_q and d_tiled must be 16-byte aligned");
    RBN_REQUIRE((((uintptr_t)d_out | (uintptr_t)d_acc) & 15u) == 0,
                "d_out and d_acc must be 16-byte aligned");
    RBN_REQUIRE(K <= (1ull << 24) && N <= (1ull << 24), "dimension too large");
    SkinnyPlan p;
    if (!plan_skinny(M, K, N, max_tiles, max_groups, strict, &p))
        return rbn_fail(RBN_ERR_UNSUPPORTED,
                        "%s: M=%llu K=%llu N=%llu needs %lld partial tiles and %d counters; the static "
                        "scratch holds %d tiles (%zu bytes) and %d counters - use rbn_gemm_t2_i8_skinny",
                        name, (unsigned long long)M, (unsigned long long)K, (unsigned long long)N,
                        (long long)p.groups * p.splits * p.mt * p.ng, p.groups, max_tiles, (size_t)max_tiles * 4096,
                        max_groups);
    // never launch a shape the kernels do not cover: an index outside a wave's range would be an
    // address outside the matrix
    if (!plan_is_launchable(p))
        return rbn_fail(RBN_ERR_UNSUPPORTED, "%s: no launch shape for M=%llu K=%llu N=%llu (splits %d, waves %d, steps %d)",
                        name, (unsigned long long)M, (unsigned long long)K, (unsigned long long)N, p.splits, p.waves,
                        p.steps);
    Args a;
    a.q = d_q;
    a.act_scale = d_act_scale;
    a.rowsum = d_rowsum;
    a.wt = (const uint4 *)d_tiled;
    a.w_scale = w_scale;
    a.M = (int)M;
    a.Kpad = (int)rbn_kpad(K);
    a.N = (int)N;
    a.partials = (int4 *)partials;
    a.tickets = tickets;
    a.acc = d_acc;
    a.out = d_out;
    a.groups = p.groups;
    a.splits = p.splits;
    a.waves = p.waves;
    if (strict && a.splits > 1) {
        // the array keeps the last call's contents: the counters this launch draws from start at zero
        clear_tickets_kernel<<<dim3(1), dim3(kStaticGroups), 0, ctx->stream>>>(tickets, kStaticGroups);
    }
    int rc;
    switch (p.mt) {
        case 1:
            rc = p.longest <= 1 ? launch_dma<1, false>(ctx->stream, a)
                                : p.longest <= 2 ? launch_dma<2, false>(ctx->stream, a)
                                                 : launch_dma<2, true>(ctx->stream, a);
            break;
        case 2: rc = launch_d<2, 1>(ctx->stream, a); break;
        default: rc = p.ng == 2 ? launch_d<4, 2>(ctx->stream, a) : launch_d<4, 1>(ctx->stream, a); break;
    }
    RBN_CHECK(rc);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

extern "C" int rbn_gemm_t2_i8_skinny(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                     const int32_t *d_rowsum, const uint32_t *d_tiled,
                                     float w_scale, uint64_t M, uint64_t K, uint64_t N,
                                     int32_t *d_acc, float *d_out) {
    RBN_ENTER(ctx);
    return skinny_impl(ctx, "rbn_gemm_t2_i8_skinny", d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N,
                       d_acc, d_out, ctx->splitk_partials, ctx->splitk_tickets, RBN_SPLITK_TILES,
                       RBN_SPLITK_GROUPS, false);
}

// The same kernels with the split-k exchange area in this file's static device array instead of
// memory the context allocated: no allocation anywhere on this path.
extern "C" int rbn_gemm_t2_i8_skinny_static(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                            const int32_t *d_rowsum, const uint32_t *d_tiled,
                                            float w_scale, uint64_t M, uint64_t K, uint64_t N,
                                            int32_t *d_acc, float *d_out) {
    RBN_ENTER(ctx);
    void *base = nullptr;
    bool mine = true;
    if (ctx->device >= 0 && ctx->device < kMaxDevices) {
        std::lock_guard<std::mutex> hold(g_scratch_lock);
        base = g_scratch_ptr[ctx->device];
        if (g_scratch_owner[ctx->device] == nullptr) g_scratch_owner[ctx->device] = ctx;
        mine = g_scratch_owner[ctx->device] == ctx;
    }
    if (base == nullptr)
        return rbn_fail(RBN_ERR_HIP, "the static scratch of device %d was never looked up", ctx->device);
    if (!mine)
        return rbn_fail(RBN_ERR_INVALID,
                        "the static scratch of device %d is in use by another context: one context per GPU "
                        "may call rbn_gemm_t2_i8_skinny_static (it is released when that context is destroyed)",
                        ctx->device);
    unsigned *tickets = reinterpret_cast<unsigned *>(static_cast<unsigned char *>(base) +
                                                     (size_t)kStaticTiles * 4096);
    return skinny_impl(ctx, "rbn_gemm_t2_i8_skinny_static", d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M,
                       K, N, d_acc, d_out, base, tickets, kStaticTiles, kStaticGroups, true);
}

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
        const int s = min(s0 + d, s1 - 1);
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
                const int sn = min(base + d + D, s1 - 1);
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
    const int mt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    // four row tiles and a wide matrix: a wave takes two groups of 64 columns, which halves
    // the activation traffic (8192 x 28672, M = 64: 55 -> 43 us); narrower matrices need
    // the workgroups more than the saving (4096 x 11008: 18 us with one group, 28 with two)
    const int cgroups = (int)(rbn_npad(N) / 64);
    const int ng = (mt == 4 && cgroups >= 256) ? 2 : 1;
    a.groups = (cgroups + ng - 1) / ng;
    // Shape of the launch (measured on the decode shapes; 64-k steps per wave in brackets).
    // With enough column groups, one workgroup per group: 4096 x 11008 runs 16 waves [4],
    // 8192 x 28672 16 waves [8].  Narrower matrices are also split along k across
    // workgroups, towards ~256 of them; the round trip of the partial tiles through
    // memory costs 1-2 us, which is why wide matrices are not split.  A wave should get 4
    // steps (a ring of 4 with nothing masked), or 8 and more when the workgroup is full.
    const int steps = a.Kpad / 64;
    const int max_w = mt == 4 ? (ng == 2 ? max_waves<4, 2>() : max_waves<4, 1>())
                              : (mt == 2 ? max_waves<2, 1>() : max_waves<1, 1>());
    int splits = 1;
    if (a.groups < 128 || a.groups * max_w < 1024) splits = (256 + a.groups - 1) / a.groups;
    if (splits > steps / 4) splits = steps / 4 > 0 ? steps / 4 : 1;
    // ... and a split should keep 32 steps or more (48 up to 8 tokens): below that the round
    // trip of the partial tiles costs more than the extra workgroups bring (2560 x 2560,
    // M = 4: 8.5 us with 7 splits, 4.5 with one; 4096 x 256: 19 -> 5 us)
    {
        const int per = M <= 8 ? 48 : 32;
        const int want = (steps + per - 1) / per;
        if (want < splits) splits = want;
    }
    // the exchange area holds max_tiles tiles of 16 x 64 int32 and one ticket per group
    if (strict) {
        if (splits > 1 && ((int64_t)a.groups * splits * mt * ng > max_tiles || a.groups > max_groups))
            return rbn_fail(RBN_ERR_UNSUPPORTED,
                            "%s: M=%llu K=%llu N=%llu needs %lld partial tiles and %d counters; the static "
                            "scratch holds %d tiles (%zu bytes) and %d counters - use rbn_gemm_t2_i8_skinny",
                            name, (unsigned long long)M, (unsigned long long)K, (unsigned long long)N,
                            (long long)a.groups * splits * mt * ng, a.groups, max_tiles,
                            (size_t)max_tiles * 4096, max_groups);
    } else {
        while (splits > 1 && ((int64_t)a.groups * splits * mt * ng > max_tiles || a.groups > max_groups))
            --splits;
    }
    const int steps_per_split = (steps + splits - 1) / splits;
    int waves = (steps_per_split + 3) / 4;
    if (waves > max_w) waves = max_w;
    if (waves > steps / splits) waves = steps / splits;  // every wave needs a step
    if (waves < 1) waves = 1;
    a.splits = splits;
    a.waves = waves;
    if (strict && splits > 1) {
        // the array keeps the last call's contents: the counters this launch draws from start at zero
        clear_tickets_kernel<<<dim3(1), dim3(kStaticGroups), 0, ctx->stream>>>(tickets, kStaticGroups);
    }
    int rc;
    switch (mt) {
        case 1: rc = launch_d<1, 1>(ctx->stream, a); break;
        case 2: rc = launch_d<2, 1>(ctx->stream, a); break;
        default: rc = ng == 2 ? launch_d<4, 2>(ctx->stream, a) : launch_d<4, 1>(ctx->stream, a); break;
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
    if (ctx->device >= 0 && ctx->device < kMaxDevices) {
        std::lock_guard<std::mutex> hold(g_scratch_lock);
        base = g_scratch_ptr[ctx->device];
    }
    if (base == nullptr)
        return rbn_fail(RBN_ERR_HIP, "the static scratch of device %d was never looked up", ctx->device);
    unsigned *tickets = reinterpret_cast<unsigned *>(static_cast<unsigned char *>(base) +
                                                     (size_t)kStaticTiles * 4096);
    return skinny_impl(ctx, "rbn_gemm_t2_i8_skinny_static", d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M,
                       K, N, d_acc, d_out, base, tickets, kStaticTiles, kStaticGroups, true);
}

// Prefill-regime ternary GEMM on the int8 matrix cores:
// out[m,n] = ((float)acc * act_scale[m]) * w_scale, acc = sum_k q[m,k] * w[k,n] (int32).
//
// Reference: BitNetKernel::execute_ternary_matmul,
// crates/ronn-providers/src/bitnet/kernels.rs:134-178 (epilogue order :168).
//
// Shape of the kernel (v_mfma_i32_32x32x32_i8, 64-wide waves):
//  * Workgroup tile 128 (M) x 256 (N), K step 128; four waves as 2 x 2, each wave
//    64 x 128 = 2 x 4 MFMA tiles (128 accumulator registers), two workgroups per CU.
//  * Both operands travel global memory -> LDS without touching registers
//    (global_load_lds_dwordx4), into a ring of three stages: the loads of K step it+2 are
//    issued while step it is multiplied, so HBM latency (each weight byte is used by only
//    two row tiles per XCD and therefore misses L2) is covered by two K steps.  The loads
//    are issued from inline assembly, so the compiler neither tracks nor waits for them;
//    the ring is synchronised by hand: an s_waitcnt vmcnt(n) that leaves exactly the newest
//    stage's loads in flight, then a bare s_barrier.  A wave issues such a load in about
//    33 cycles, in which it issues nothing else: the six loads of a stage are therefore
//    issued one at a time, each right behind an MFMA that keeps the matrix pipe busy for
//    32 cycles, and not as a block at the start of the K step (where they held the pipe
//    idle for 200 of a K step's 1,420 cycles).  The ring's three positions are
//    written out in the loop body, so LDS addresses are lane constants plus immediates.
//  * A lane of such a load picks its own global address (a workgroup-uniform base in scalar
//    registers plus a 32-bit lane offset) but lands at LDS base + 16 * lane,
//    so the LDS images are linear arrays of 16-byte units with an XOR swizzle chosen so
//    that (a) eight consecutive lanes fetch one 128-byte line of global memory and (b) the
//    128-bit fragment reads of eight consecutive lanes hit distinct banks:
//      activations  unit row*8 + (seg ^ ((row>>1) & 7))   holds q[row][16*seg .. 16*seg+15]
//      weights      unit quad*8 + (kb ^ ((quad>>1) & 7))  holds the four words of (quad, kb)
//    (LDS serves sixteen lanes of a 128-bit read per cycle from 64 banks: sixteen
//    consecutive rows must fall on sixteen different 16-byte bank groups, i.e. distinct
//    values of (row & 1) * 8 + slot, which the (row >> 1) swizzle gives)
//  * Weights stay 2-bit until they are in registers.  Lane l reads ONE 16-byte unit (quad
//    l%32, k-half l/32) per 32 k and expands it with 28 VALU operations into the B
//    fragments of FOUR MFMA tiles: tile j covers the columns 4*quad + j.  The same mapping
//    lets the epilogue store four adjacent columns per lane as one 128-bit store
//    (nontemporal: the output is written once and not read by this kernel).
//  * Workgroups are numbered so that the eight XCDs each own a band of rows: a band's
//    activations stay in that XCD's L2 while the weights stream through.
//  * Weights are stored as code = value + 1, so the per-token sum of q is subtracted in
//    the epilogue (integer-exact).  K is padded to 128 by the activation and weight
//    formats (zero activations, zero-weight codes), rows and columns past the edge are
//    clamped duplicates whose results are never stored.
#include "common.hpp"
#include <type_traits>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef void __attribute__((address_space(3))) * lds_ptr;
typedef const void __attribute__((address_space(1))) * global_ptr;

constexpr int kThreads = 256;
constexpr int BN = 256, BK = 128;
constexpr int kBUnits = (BN / 4) * 8;  // of one weight stage (8 KiB)

// s_waitcnt immediates (gfx9 encoding: vmcnt[3:0] | expcnt << 4 | lgkmcnt << 8 | vmcnt[5:4] << 14)
constexpr int kWaitVm0 = 0x0F70;       // vmcnt(0)

__device__ __forceinline__ v4i decode_b(uint32_t w) {
    v4i b;
    b.x = (int)(w & 0x03030303u);
    b.y = (int)((w >> 2) & 0x03030303u);
    b.z = (int)((w >> 4) & 0x03030303u);
    b.w = (int)((w >> 6) & 0x03030303u);
    return b;
}

// One wave-wide 16-byte-per-lane load from global memory straight into LDS: lane i's
// 16 bytes land at LDS byte address lds_wave_base + 16 * i (M0 carries the base).
__device__ __forceinline__ void dma16(const void *base, uint32_t lane_offset, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_wave_base), "v"(lane_offset), "s"(base)
                 : "memory", "m0");
}

// MT = 2: the regular tile of 128 rows (waves of 64 x 128).  MT = 1: tiles of 64 rows (waves
// of 32 x 128, half the accumulators, three workgroups per CU) for products whose 128-row
// tiling would leave most of the chip idle.
template <int MT>
__global__ __launch_bounds__(kThreads, MT == 2 ? 2 : 3) void gemm_t2_i8_mfma_kernel(
    const int8_t *__restrict__ q,         // [M][Kpad], Kpad % 128 == 0
    const float *__restrict__ act_scale,  // [M]
    const int32_t *__restrict__ rowsum,   // [M]
    const uint4 *__restrict__ wt,         // tiled: uint4 index quad * KB + kb
    float w_scale, int M, int Kpad, int N, int nquads, int m_tiles, int n_tiles, int splits,
    int32_t *partials, unsigned *tickets, int32_t *__restrict__ acc_out, float *__restrict__ out) {
    // Ring of three stages in one array (units of 16 bytes): weights of stage s at
    // s * kBUnits, activations at 3 * kBUnits + s * kAUnits.
    constexpr int TM = 64 * MT;                  // rows of the tile
    constexpr int kAUnits = TM * 8;              // 16-byte units of one activation stage
    constexpr int kLoads = 2 * MT + 2;           // LDS loads per wave and stage
    constexpr int kWaitStage = 0x0070 | kLoads;  // s_waitcnt vmcnt(kLoads) lgkmcnt(0)
    // at the hand-over inside a K step: the sixth load of a stage is issued behind it (MT = 2)
    constexpr int kWaitMid = 0x0070 | (MT == 2 ? 5 : 4);
    __shared__ __attribute__((aligned(16))) uint4 smem[3 * (kAUnits + kBUnits)];
    __shared__ __attribute__((aligned(16))) float s_scale[TM];
    __shared__ __attribute__((aligned(16))) int s_rowsum[TM];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int KB = Kpad >> 4;

    // XCD-aware numbering: consecutive workgroups land on consecutive XCDs; give each XCD
    // a band of m tiles and let it walk the n tiles.
    // With splits > 1 (few tiles, see the launch) `splits` consecutive workgroups share a
    // tile and take consecutive ranges of K steps.
    // every argument the set-up below needs, asked for in one go: left to the compiler, the scalar
    // loads of the arguments were fetched where first used, five dependent round trips before the
    // first transfer could be issued
    asm volatile("" : : "s"(M), "s"(Kpad), "s"(N), "s"(nquads), "s"(m_tiles), "s"(n_tiles), "s"(splits), "s"(q),
                 "s"(wt), "s"(act_scale), "s"(rowsum));
    int tile = blockIdx.x, split = 0;
    if (MT == 1 && splits > 1) {  // 128-row tiles are never split along K
        tile = blockIdx.x / splits;
        split = blockIdx.x - tile * splits;
    }
    int bm, bn;
    if ((m_tiles & 7) == 0 && (MT == 2 || splits == 1)) {
        const int per = m_tiles >> 3;
        const int xcd = tile & 7, i = tile >> 3;
        bm = xcd * per + i % per;
        bn = i / per;
    } else {
        bm = tile % m_tiles;
        bn = tile / m_tiles;
    }
    const int m0 = bm * TM, n0 = bn * BN;
    const int q0 = n0 >> 2;

    // The epilogue's per-row scalars are asked for here and written to LDS only after the first two
    // stages are on their way: staged at once, their round trip stood between the kernel's start and
    // its first transfer (2,700 cycles from start to the first transfer, 630 more to the first data).
    v16i acc[MT][4];  // zeroed below, behind the first transfers
    float pre_scale = 0.0f;
    int pre_rowsum = 0;
    if (tid < TM) {
        const int row = m0 + tid;
        pre_scale = row < M ? act_scale[row] : 0.0f;
        pre_rowsum = row < M ? rowsum[row] : 0;
    }

    // Per-lane source addresses of the stage loads.  Load j of wave w fills the units
    // (4j + w) * 64 + lane: row (or quad) (4j + w) * 8 + lane / 8, slot lane % 8, and the
    // slot holds segment (or k-block) slot ^ ((row >> 1) & 7) of that row.
    const int sub = lane >> 3;
    // a workgroup-uniform base (scalar registers) plus a 32-bit byte offset per lane
    const int8_t *a_base = q + (size_t)m0 * Kpad;  // advanced to this workgroup's first K step below
    uint32_t a_lane[2 * MT];
#pragma unroll
    for (int j = 0; j < 2 * MT; ++j) {
        const int lrow = (4 * j + wave) * 8 + sub;
        const int seg = (lane & 7) ^ ((lrow >> 1) & 7);
        a_lane[j] = (uint32_t)(min(m0 + lrow, M - 1) - m0) * (uint32_t)Kpad + seg * 16;
    }
    const uint4 *b_base = wt + (size_t)q0 * KB;
    uint32_t b_lane[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int lquad = (4 * j + wave) * 8 + sub;
        const int kb = (lane & 7) ^ ((lquad >> 1) & 7);
        b_lane[j] = ((uint32_t)(min(q0 + lquad, nquads - 1) - q0) * (uint32_t)KB + kb) * 16;
    }
    // this workgroup's K steps: [it_lo, it_lo + iters)
    const int iters_all = Kpad / BK;
    const int per_split = MT == 2 ? iters_all : (iters_all + splits - 1) / splits;
    const int it_lo = split * per_split;
    const int iters = min(per_split, iters_all - it_lo);  // >= 1 (the launch sees to it)
    a_base += (size_t)it_lo * BK;
    b_base += (size_t)it_lo * (BK / 16);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr)smem;
    auto issue = [&](int it, int stage) {
        const int kk = min(it, iters - 1);  // past the end: reload the last step, never read
        const uint32_t sb = lds0 + (uint32_t)(stage * kBUnits) * 16;
        const uint32_t sa = lds0 + (uint32_t)(3 * kBUnits + stage * kAUnits) * 16;
        const int8_t *ab = a_base + (size_t)kk * BK;
        const uint4 *bb = b_base + (size_t)kk * (BK / 16);
#pragma unroll
        for (int j = 0; j < 2 * MT; ++j) dma16(ab, a_lane[j], sa + (4 * j + wave) * 1024);
#pragma unroll
        for (int j = 0; j < 2; ++j) dma16(bb, b_lane[j], sb + (4 * j + wave) * 1024);
    };

    // load d of a stage on its own: d < 2 * MT is activation load d, the others are the weight loads
    auto issue_one = [&](int it, int stage, int d) {
        const int kk = min(it, iters - 1);
        if (d < 2 * MT) {
            const uint32_t sa = lds0 + (uint32_t)(3 * kBUnits + stage * kAUnits) * 16;
            dma16(a_base + (size_t)kk * BK, a_lane[d], sa + (4 * d + wave) * 1024);
        } else {
            const int j = d - 2 * MT;
            const uint32_t sb = lds0 + (uint32_t)(stage * kBUnits) * 16;
            dma16(b_base + (size_t)kk * (BK / 16), b_lane[j], sb + (4 * j + wave) * 1024);
        }
    };

    // fragment addresses (in 16-byte units, relative to a stage)
    const int frow0 = wm * (32 * MT) + (lane & 31), khalf = lane >> 5;
    const int fquad = wn * 32 + (lane & 31);
    auto a_unit = [&](int row, int seg) { return row * 8 + (seg ^ ((row >> 1) & 7)); };
    auto b_unit = [&](int kb) { return fquad * 8 + (kb ^ ((fquad >> 1) & 7)); };

    // Lane-constant fragment offsets (16-byte units inside a stage) of the four sub-steps.
    int a_off[4], b_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        a_off[ks] = a_unit(frow0, 2 * ks + khalf);
        b_off[ks] = b_unit(2 * ks + khalf);
    }

    // The K loop is a software pipeline that spans the stage boundary.  A K step has four
    // sub-steps of 32 k; sub-step ks multiplies with fragments that are already in
    // registers (weights decoded), while the VALU expands the weights of the next sub-step
    // and LDS delivers the raw fragments of the sub-step after that - across the boundary
    // the "next" sub-steps are sub-steps 0 and 1 of the following stage.  The stage
    // hand-over (wait for the DMA, barrier) therefore sits in the MIDDLE of a K step,
    // between sub-steps 1 and 2: by then every read of the current stage has been issued
    // (and is waited for), and the reads of the next stage start right after it, a full
    // sub-step (eight MFMAs, 256 cycles) before their first use.
    // A v_mfma_i32_32x32x32_i8 holds the matrix pipe for 32 cycles, in which the wave can
    // issue about seven other instructions; sched_group_barrier asks for that interleaving
    // (1 MFMA + 4 VALU, the first three groups also an LDS read), and sched_barrier(0)
    // keeps the compiler from moving anything between sub-steps (left alone it sinks every
    // LDS read down to its first use and waits for it there).
    uint4 rb[4], ra0[4], ra1[4];
    v4i bf[4], bf_n[4];
    auto lds_reads = [&](int stage, int ks) {
        const uint4 *sb = smem + stage * kBUnits;
        const uint4 *sa = smem + 3 * kBUnits + stage * kAUnits;
        rb[ks] = sb[b_off[ks]];
        ra0[ks] = sa[a_off[ks]];
        if constexpr (MT == 2) ra1[ks] = sa[a_off[ks] + 32 * 8];  // row + 32: same swizzle
    };
    auto decode_next = [&](int ks) {
        bf_n[0] = decode_b(rb[ks].x);
        bf_n[1] = decode_b(rb[ks].y);
        bf_n[2] = decode_b(rb[ks].z);
        bf_n[3] = decode_b(rb[ks].w);
    };
    // sub-step ks: read (read_stage, read_ks), decode dec_ks, multiply ks; `mid` runs between the
    // two halves of the sub-step (a transfer is issued there, behind an MFMA that keeps the pipe busy)
    auto substep = [&](int ks, int read_stage, int read_ks, int dec_ks, auto mid) {
        lds_reads(read_stage, read_ks);
        bf_n[0] = decode_b(rb[dec_ks].x);
        bf_n[1] = decode_b(rb[dec_ks].y);
        const v4i af0 = {(int)ra0[ks].x, (int)ra0[ks].y, (int)ra0[ks].z, (int)ra0[ks].w};
        const v4i af1 = {(int)ra1[ks].x, (int)ra1[ks].y, (int)ra1[ks].z, (int)ra1[ks].w};
        if constexpr (MT == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf[j], acc[0][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf[j], acc[0][j], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < 2 * MT; ++g) {
            if (g < MT + 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, 8 / MT, 0);             // VALU
        }
        __builtin_amdgcn_sched_barrier(0);
        mid();
        __builtin_amdgcn_sched_barrier(0);
        bf_n[2] = decode_b(rb[dec_ks].z);
        bf_n[3] = decode_b(rb[dec_ks].w);
        if constexpr (MT == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[1][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af1, bf[j], acc[1][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int j = 2; j < 4; ++j)
                acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af0, bf[j], acc[0][j], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < 2 * MT; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       // MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, 8 / MT, 0);  // VALU
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = bf_n[j];
        __builtin_amdgcn_sched_barrier(0);
    };

    // prologue: stages 0 and 1 in flight, wait for stage 0 (and for the LDS writes above),
    // then fill the pipeline: raw fragments of sub-steps 0 and 1, weights of 0 decoded
    issue(0, 0);
    issue(1, 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    if (tid < TM) {
        s_scale[tid] = pre_scale;
        s_rowsum[tid] = pre_rowsum;
    }
    __builtin_amdgcn_s_waitcnt(kWaitStage);
    __builtin_amdgcn_s_barrier();
    lds_reads(0, 0);
    lds_reads(0, 1);
    decode_next(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[j] = bf_n[j];
    __builtin_amdgcn_sched_barrier(0);

    // K step `it` on stage cur: the loads of step it+2 go into `fill` - the stage read
    // in step it-1, which every wave has left: all its reads were waited for before the
    // barrier inside step it-1.  They are issued one by one: before, in the middle of and
    // behind sub-steps 0 and 1, and (the sixth, MT = 2) in the middle of sub-step 2.  After
    // sub-step 1, wait until only the newest five (MT = 1: four) loads are outstanding - the
    // sixth load of stage nxt, issued in step it-1, is older than those, so stage nxt has
    // landed - and until this wave's reads of `cur` have returned, meet, and go on with the
    // reads of nxt.  In the last step nxt holds no new data; what is read from it is never used.
    // The loop body is written out for the three positions of the ring, so every LDS
    // address is a lane constant plus an immediate.
    auto kstep = [&](auto cur_tag, int it) {
        constexpr int cur = decltype(cur_tag)::value;
        constexpr int nxt = (cur + 1) % 3, fill = (cur + 2) % 3;
        auto none = [] {};
        issue_one(it + 2, fill, 0);
        __builtin_amdgcn_sched_barrier(0);
        substep(0, cur, 2, 1, [&] { issue_one(it + 2, fill, 1); });
        issue_one(it + 2, fill, 2);
        __builtin_amdgcn_sched_barrier(0);
        substep(1, cur, 3, 2, [&] { issue_one(it + 2, fill, 3); });
        if constexpr (MT == 2) issue_one(it + 2, fill, 4);
        __builtin_amdgcn_s_waitcnt(kWaitMid);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MT == 2) substep(2, nxt, 0, 3, [&] { issue_one(it + 2, fill, 5); });
        else substep(2, nxt, 0, 3, none);
        substep(3, nxt, 1, 0, none);
    };
    // The K loop runs at a higher wave priority than the epilogue: by default the older workgroup of a
    // CU wins the issue slots, also while it is in its epilogue (conversions, multiplies and stores),
    // where it held the younger one's loop at half its speed (2,090 cycles per K step against 1,450
    // with the CU to itself).
    __builtin_amdgcn_s_setprio(1);
    int it = 0;
    for (; it + 2 < iters; it += 3) {
        kstep(std::integral_constant<int, 0>{}, it);
        kstep(std::integral_constant<int, 1>{}, it + 1);
        kstep(std::integral_constant<int, 2>{}, it + 2);
    }
    if (it < iters) kstep(std::integral_constant<int, 0>{}, it);
    if (it + 1 < iters) kstep(std::integral_constant<int, 1>{}, it + 1);
    __builtin_amdgcn_s_waitcnt(kWaitVm0);  // no load may still be writing LDS at exit
    __builtin_amdgcn_s_setprio(0);

    if constexpr (MT == 1) {
        if (splits > 1) {
            // Partial tiles meet in the workspace: every workgroup publishes its accumulators
            // (register r of lane l of wave w at [(r * 4 + w) * 64 + l]) with device-scope
            // stores, waits for them, and draws a ticket; the last of a tile adds the others'
            // (integer sums: any order, same bits) and goes on to the epilogue.  Nobody waits
            // for anybody.  The pointer is walked in a register the compiler cannot see
            // through: folded into 64 constant offsets it costs 64 scalar register pairs.
            // Register pair i of lane l of wave w sits at 64-bit index (i * 4 + w) * 64 + l.
            // The lane offset is kept opaque to the compiler, which otherwise folds the 32
            // positions into as many scalar register pairs.
            constexpr size_t kPartialBytes = (size_t)64 * kThreads * 4;
            char *mine = reinterpret_cast<char *>(partials) + ((size_t)tile * splits + split) * kPartialBytes;
            uint32_t off = (uint32_t)(wave * 64 + lane) * 8;
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const unsigned long long pair = (unsigned)acc[0][j][r] |
                                                    ((unsigned long long)(unsigned)acc[0][j][r + 1] << 32);
                    __hip_atomic_store(reinterpret_cast<unsigned long long *>(mine + off), pair,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    off += kThreads * 8;
                    asm volatile("" : "+v"(off));
                }
            // the partial tile is published once its stores are acknowledged: the fence keeps the
            // compiler from moving them below the wait, the wait covers this wave's stores, the
            // barrier everybody's
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const unsigned ticket = atomicAdd(&tickets[tile], 1u);
                const int is_last = ticket == (unsigned)splits - 1;
                if (is_last) atomicExch(&tickets[tile], 0u);  // ready for the next launch
                s_last = is_last;
            }
            __syncthreads();
            if (!s_last) return;
            for (int s2 = 0; s2 < splits; ++s2) {
                if (s2 == split) continue;
                const char *theirs =
                    reinterpret_cast<const char *>(partials) + ((size_t)tile * splits + s2) * kPartialBytes;
                off = (uint32_t)(wave * 64 + lane) * 8;
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int r = 0; r < 16; r += 2) {
                        const unsigned long long pair =
                            __hip_atomic_load(reinterpret_cast<const unsigned long long *>(theirs + off),
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        acc[0][j][r] += (int)(unsigned)pair;
                        acc[0][j][r + 1] += (int)(unsigned)(pair >> 32);
                        off += kThreads * 8;
                        asm volatile("" : "+v"(off));
                    }
            }
        }
    }

    // epilogue: lane owns columns 4*quad .. 4*quad+3 (tile j -> column 4*quad + j) and rows
    // 8*(r/4) + 4*(lane/32) + r%4 of each 32-row tile
    const int col0 = n0 + fquad * 4;
    const bool vec_ok = (N & 3) == 0;
    // A tile that lies inside the matrix (all but the last row and column of tiles): the scalars of a
    // lane's rows come from LDS as vectors, all reads in flight together, and the 16 x MT stores per
    // lane follow each other without a branch or a wait in between.  (Row by row, with two dependent
    // LDS reads and three branches per row, this took 8,000-11,500 cycles per workgroup, most of it
    // latency; while a workgroup is in its epilogue its CU has one stream of MFMAs instead of two, and
    // the kernel's last epilogues are not overlapped with anything.)
    if (vec_ok && m0 + TM <= M && n0 + BN <= N) {
        v4f sc[MT][4];
        v4i rsv[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int lrow = wm * (32 * MT) + mt * 32 + 8 * g4 + 4 * (lane >> 5);  // rows lrow .. lrow + 3
                sc[mt][g4] = *reinterpret_cast<const v4f *>(&s_scale[lrow]);
                rsv[mt][g4] = *reinterpret_cast<const v4i *>(&s_rowsum[lrow]);
            }
        float *orow = out + (size_t)(m0 + wm * (32 * MT) + 4 * (lane >> 5)) * N + col0;
        int32_t *arow = acc_out ? acc_out + (size_t)(m0 + wm * (32 * MT) + 4 * (lane >> 5)) * N + col0 : nullptr;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int rs = rsv[mt][r >> 2][r & 3];
                const float as = sc[mt][r >> 2][r & 3];
                int t[4];
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    t[j] = acc[mt][j][r] - rs;
                    const float f = (float)t[j] * as;  // kernels.rs:168, left to right
                    v[j] = f * w_scale;
                }
                const size_t o = (size_t)(mt * 32 + 8 * (r >> 2) + (r & 3)) * N;
                __builtin_nontemporal_store(v4f{v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f *>(orow + o));
                if (arow) __builtin_nontemporal_store(v4i{t[0], t[1], t[2], t[3]}, reinterpret_cast<v4i *>(arow + o));
            }
        return;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int lrow = wm * (32 * MT) + mt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
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
                __builtin_nontemporal_store(v4f{v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f *>(out + o));
                if (acc_out) __builtin_nontemporal_store(v4i{t[0], t[1], t[2], t[3]}, reinterpret_cast<v4i *>(acc_out + o));
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
    static_assert(BK == 128, "the K padding of the formats must equal the K step");
    const int nquads = (int)(rbn_npad(N) / 4);
    // 128-row tiles, two workgroups per CU; when those would fill at most half of the slots,
    // 64-row tiles (twice as many workgroups, three per CU)
    const int n_tiles = (int)((N + BN - 1) / BN);
    const uint64_t slots = 2ull * (uint64_t)ctx->props.multiProcessorCount;
    const bool low = ((M + 127) / 128) * (uint64_t)n_tiles * 2 <= slots;
    const int m_tiles = (int)((M + (low ? 63 : 127)) / (low ? 64 : 128));
    const uint64_t tiles = (uint64_t)m_tiles * n_tiles;
    RBN_REQUIRE(tiles <= 0x7fffffffull, "too many tiles");
    // Very few tiles and a long K: split K over up to four workgroups per tile.  The parts
    // meet through memory (64 KiB per partial tile, device-scope accesses), which costs about
    // as much as ten K steps: measured, it pays up to ~96 tiles with at least sixteen K steps
    // per part (6912 x 2560, M = 512: 26 -> 20 us; 11008 x 4096, M = 64: 39 -> 20 us) and
    // loses beyond (4096 x 11008, M = 256: 18 -> 23 us).
    int splits = 1;
    if (low && tiles <= 96) {
        const int iters = Kpad / BK;
        const uint64_t room = 3ull * (uint64_t)ctx->props.multiProcessorCount;
        while (splits < 4 && tiles * (splits + 1) <= room && iters / (splits + 1) >= 16) ++splits;
        while (splits > 1 && (splits - 1) * ((iters + splits - 1) / splits) >= iters) --splits;
        if (tiles > (uint64_t)RBN_SPLITK_GROUPS || tiles * splits * 16 > (uint64_t)RBN_SPLITK_TILES)
            splits = 1;
    }
    const unsigned grid = (unsigned)(tiles * splits);
    if (low)
        gemm_t2_i8_mfma_kernel<1><<<dim3(grid), dim3(kThreads), 0, ctx->stream>>>(
            d_q, d_act_scale, d_rowsum, (const uint4 *)d_tiled, w_scale, (int)M, Kpad, (int)N,
            nquads, m_tiles, n_tiles, splits, (int32_t *)ctx->splitk_partials, ctx->splitk_tickets,
            d_acc, d_out);
    else
        gemm_t2_i8_mfma_kernel<2><<<dim3(grid), dim3(kThreads), 0, ctx->stream>>>(
            d_q, d_act_scale, d_rowsum, (const uint4 *)d_tiled, w_scale, (int)M, Kpad, (int)N,
            nquads, m_tiles, n_tiles, 1, nullptr, nullptr, d_acc, d_out);
    RBN_HIP(hipGetLastError());
    return RBN_OK;
}

extern "C" int rbn_matmul_kernel_choice(uint64_t M, uint64_t K, uint64_t N) {
    // measured crossovers: the dot-instruction GEMV wins for one and two tokens (its time
    // grows with M, so not for two tokens on a wide matrix with a short k) and up to four
    // tokens on small matrices; the streaming small-batch kernel up to 32 tokens (16 on very
    // large matrices) and, on small matrices, up to its limit of 64; the tiled kernel beyond
    const uint64_t kn = K * N;
    if (M == 1) return RBN_KERNEL_GEMV;
    if (M == 2 && !(K <= 3072 && kn >= (1ull << 25))) return RBN_KERNEL_GEMV;
    if (M >= 3 && M <= 4 && kn <= (1ull << 24)) return RBN_KERNEL_GEMV;
    if (M <= 16 || (M <= 32 && kn < (1ull << 27)) || (M <= RBN_SKINNY_MAX_M && kn < (1ull << 25)))
        return RBN_KERNEL_SKINNY;
    return RBN_KERNEL_MFMA;
}

extern "C" int rbn_matmul_t2_i8(rbn_ctx *ctx, const int8_t *d_q, const float *d_act_scale,
                                const int32_t *d_rowsum, const uint32_t *d_tiled, float w_scale,
                                uint64_t M, uint64_t K, uint64_t N, int32_t *d_acc,
                                float *d_out) {
    switch (rbn_matmul_kernel_choice(M, K, N)) {
        case RBN_KERNEL_GEMV:
            return rbn_gemv_t2_i8(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc, d_out);
        case RBN_KERNEL_SKINNY:
            return rbn_gemm_t2_i8_skinny(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc,
                                         d_out);
        default:
            return rbn_gemm_t2_i8_mfma(ctx, d_q, d_act_scale, d_rowsum, d_tiled, w_scale, M, K, N, d_acc,
                                       d_out);
    }
}

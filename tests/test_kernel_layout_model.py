"""A CPU model of the address arithmetic of the LDS-ring small-batch kernel (skinny_dma_kernel in
ronn_amd/csrc/skinny_mfma.hip): which 16 bytes every lane of every global->LDS transfer fetches,
where they land in the wave's stage, which unit every lane reads back as its MFMA fragment, and
what the four v_mfma_i32_16x16x64_i8 per half stage then compute.  It follows the kernel
statement by statement with the launch shape the library itself picks (rbn_skinny_launch_shape),
asserts that every global address stays inside its buffer and every LDS address inside the wave's
ring, and that the accumulators equal the exact integer product - so the layout (tiled weights,
swizzled LDS image, operand lanes) is pinned without a GPU, and a change to the kernel's indexing
can be tried here first.  What it cannot model is timing (the hand-counted s_waitcnt)."""
import ctypes as C
import os

import numpy as np
import pytest

from ronn_amd import _lib


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__ as g
        g.build()
    return _lib.load()


def tile_weights(vals):
    """int8 ternary values [K, N] -> the tiled buffer as bytes (include/ronn_bitnet_hip.h): the 16 bytes
    at uint4 index quad*KB + kb are four u32, word c = column 4*quad + c, weight k = 16*kb + 4*s + b
    at bit 8*b + 2*s as code = value + 1; padding is code 1."""
    K, N = vals.shape
    kpad, npad = (K + 127) // 128 * 128, (N + 63) // 64 * 64
    code = np.ones((kpad, npad), dtype=np.uint32)
    code[:K, :N] = vals.astype(np.int32) + 1
    KB = kpad // 16
    words = np.zeros((npad // 4, KB, 4), dtype=np.uint32)
    c4 = code.reshape(KB, 16, npad // 4, 4)            # [kb][k in block][quad][c]
    for s in range(4):
        for b in range(4):
            words |= c4[:, 4 * s + b].transpose(1, 0, 2) << np.uint32(8 * b + 2 * s)
    return words.reshape(-1).view(np.uint8), kpad, npad


def decode_b(word):
    """decode_b(): the four int8 operand registers of one u32 of codes, as 16 codes in k order."""
    return np.array([(word >> (8 * b + 2 * s)) & 3 for s in range(4) for b in range(4)], dtype=np.int64)


@pytest.mark.parametrize("M,K,N", [(16, 256, 64), (5, 384, 130), (16, 1100, 64), (3, 128, 37), (9, 4096, 64),
                                   (16, 256, 704), (8, 128, 1100), (12, 256, 2752)])
def test_lds_ring_kernel_model(lib, M, K, N):
    rng = np.random.default_rng(M * 1000 + K + N)
    vals = rng.integers(-1, 2, size=(K, N)).astype(np.int8)
    q_src = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    tiled, kpad, npad = tile_weights(vals)
    KB = kpad // 16
    q = np.zeros((M, kpad), dtype=np.int8)
    q[:, :K] = q_src
    qbytes = q.reshape(-1).view(np.uint8)

    shape = (C.c_int32 * 8)()
    assert lib.rbn_skinny_launch_shape(M, K, N, shape) == 0
    ring, groups, splits, nw, step_k, stages, longest, lds_bytes = list(shape)
    assert ring == 1 and step_k == 128 and stages == kpad // 128
    D = 1 if longest <= 1 else 2
    refill = longest > 2
    assert lds_bytes == nw * D * 4096

    acc_total = np.zeros((groups, 16, 64), dtype=np.int64)      # [group][token][column in group]
    nquads = npad // 4
    half = M <= 8                                    # the transfer of tokens 8-15 is left out
    whalf = (nquads + groups - 1) // groups <= 8     # ... and that of quads 8-15
    lanes = np.arange(64)
    sub, slot = lanes >> 3, lanes & 7
    ql, g = lanes & 15, lanes >> 4
    q_los, nqs = [], []
    for group in range(groups):
        # the workgroup's quads: [group * nquads / groups, (group + 1) * nquads / groups)
        q_lo = group * nquads // groups
        nq = min(max((group + 1) * nquads // groups - q_lo, 1), 16)
        assert (group + 1) * nquads // groups - q_lo == nq and q_lo + nq <= nquads
        assert nq <= 8 or not whalf
        q_los.append(q_lo)
        nqs.append(nq)
        for split in range(splits):
            for wave in range(nw):
                gw, gn = split * nw + wave, splits * nw
                s0, s1 = gw * stages // gn, (gw + 1) * stages // gn
                assert s1 > s0
                # this wave's ring; it starts with whatever the last kernel left there
                lds = rng.integers(0, 256, size=(D, 4096)).astype(np.uint8)
                acc = np.zeros((64, 4, 4), dtype=np.int64)      # [lane][tile j][register i]

                def issue(s, d):
                    sc = max(min(s, s1 - 1), 0)
                    for h in range(2):
                        row = 8 * h + sub
                        kb = slot ^ ((row >> 1) & 7)
                        w_off = (np.minimum(row, nq - 1) * KB + kb) * 16 + (q_lo * KB + sc * 8) * 16
                        a_off = np.minimum(row, M - 1) * kpad + kb * 16 + sc * 128
                        assert w_off.min() >= 0 and w_off.max() + 16 <= tiled.size
                        assert a_off.min() >= 0 and a_off.max() + 16 <= qbytes.size
                        for l in range(64):                      # lane l's 16 bytes land at base + 16 l
                            if not (h == 1 and whalf):
                                lds[d, h * 1024 + 16 * l:h * 1024 + 16 * l + 16] = tiled[w_off[l]:w_off[l] + 16]
                            if not (h == 1 and half):
                                lds[d, 2048 + h * 1024 + 16 * l:2048 + h * 1024 + 16 * l + 16] = qbytes[a_off[l]:a_off[l] + 16]

                def consume(d, keep):
                    for t in range(2):
                        unit = ql * 8 + ((4 * t + g) ^ ((ql >> 1) & 7))
                        assert unit.max() < 128
                        # B operands of the four MFMAs: lane (ql, g) gives column 4 ql + j, k-block 4 t + g
                        w = np.stack([lds[d, 16 * u:16 * u + 16].view(np.uint32) for u in unit])      # [lane][4 words]
                        a = np.stack([lds[d, 2048 + 16 * u:2048 + 16 * u + 16].view(np.int8) for u in unit]).astype(np.int64)
                        if not keep:
                            a[:] = 0
                        for j in range(4):
                            bj = np.stack([decode_b(int(w[l, j])) for l in range(64)])                  # [lane][16 k]
                            # D[i][c] += sum over g, k of A[(i, g)][k] * B[(c, g)][k]; the result register r of
                            # lane (c, gg) is row i = 4 gg + r
                            for gg in range(4):
                                A = a[16 * gg:16 * gg + 16]          # rows i = lane % 16
                                B = bj[16 * gg:16 * gg + 16]         # columns c = lane % 16
                                Dm = A @ B.T                          # [i][c]
                                for c in range(16):
                                    for g2 in range(4):
                                        acc[16 * g2 + c, j, :] += Dm[4 * g2:4 * g2 + 4, c]

                for d in range(D):
                    issue(s0 + d, d)
                if not refill:
                    for d in range(D):
                        consume(d, s0 + d < s1)
                else:
                    base = s0
                    while True:
                        for d in range(D):
                            consume(d, base + d < s1)
                            issue(base + d + D, d)
                        base += D
                        if base >= s1:
                            break
                # the join: acc[j][i] of lane (ql, g) is token 4 g + i, column 4 ql + j
                for l in range(64):
                    for j in range(4):
                        for i in range(4):
                            acc_total[group, 4 * g[l] + i, 4 * ql[l] + j] += acc[l, j, i]
    # finish(): quad qd of the tile is column quad q_lo + qd, stored when qd < nq (and the token exists)
    got = np.full((16, npad), np.iinfo(np.int64).min, dtype=np.int64)
    for group in range(groups):
        for qd in range(nqs[group]):
            c0 = (q_los[group] + qd) * 4
            assert (got[:, c0:c0 + 4] == np.iinfo(np.int64).min).all()      # no column is written twice
            got[:, c0:c0 + 4] = acc_total[group, :, 4 * qd:4 * qd + 4]
    got = got[:M, :N]
    # weights are codes = value + 1: the kernel subtracts the token's sum of q in the epilogue
    want = q_src.astype(np.int64) @ vals.astype(np.int64)
    rowsum = q.astype(np.int64).sum(axis=1, keepdims=True)
    assert (got - rowsum == want).all()


# ---- prefill kernel (gemm_t2_i8_mfma_kernel<2> in ronn_amd/csrc/gemm_mfma.hip), one workgroup ------------

def mfma_32x32x32_i8(a_lane, b_lane):
    """v_mfma_i32_32x32x32_i8: lane l gives A[row l%32][16 k of half l//32] and B[the same k][column l%32];
    result register r of lane l is D[8*(r//4) + 4*(l//32) + r%4][l%32]."""
    A = np.zeros((32, 32), dtype=np.int64)
    B = np.zeros((32, 32), dtype=np.int64)
    for l in range(64):
        A[l % 32, 16 * (l // 32):16 * (l // 32) + 16] = a_lane[l]
        B[16 * (l // 32):16 * (l // 32) + 16, l % 32] = b_lane[l]
    D = A @ B
    out = np.zeros((64, 16), dtype=np.int64)
    for l in range(64):
        for r in range(16):
            out[l, r] = D[8 * (r // 4) + 4 * (l // 32) + r % 4, l % 32]
    return out


@pytest.mark.parametrize("M,K,N,bm,bn", [(128, 256, 256, 0, 0), (200, 384, 300, 1, 1), (130, 128, 260, 1, 0)])
def test_prefill_tile_model(M, K, N, bm, bn):
    """One 128 x 256 tile (bm, bn): the stage transfers' source addresses and LDS units, the fragment
    units every lane reads, the 32 MFMAs per K step and the epilogue's row / column mapping."""
    rng = np.random.default_rng(M + K + N)
    vals = rng.integers(-1, 2, size=(K, N)).astype(np.int8)
    q_src = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    tiled, kpad, npad = tile_weights(vals)
    KB, nquads = kpad // 16, npad // 4
    q = np.zeros((M, kpad), dtype=np.int8)
    q[:, :K] = q_src
    qbytes = q.reshape(-1).view(np.uint8)
    TM, BN, BK = 128, 256, 128
    kA, kB = TM * 8, (BN // 4) * 8           # 16-byte units of an activation / a weight stage
    m0, n0 = bm * TM, bn * BN
    q0 = n0 >> 2
    iters = kpad // BK
    result = np.zeros((TM, BN), dtype=np.int64)
    for it in range(iters):
        # --- issue(): four waves, per wave 4 activation transfers and 2 weight transfers of 64 lanes
        sa = np.zeros(kA * 16, dtype=np.uint8)
        sb = np.zeros(kB * 16, dtype=np.uint8)
        for wave in range(4):
            for lane in range(64):
                sub = lane >> 3
                for j in range(4):
                    lrow = (4 * j + wave) * 8 + sub
                    seg = (lane & 7) ^ ((lrow >> 1) & 7)
                    src = (m0 * kpad + it * BK) + (min(m0 + lrow, M - 1) - m0) * kpad + seg * 16
                    assert 0 <= src and src + 16 <= qbytes.size
                    dst = (4 * j + wave) * 1024 + 16 * lane
                    sa[dst:dst + 16] = qbytes[src:src + 16]
                for j in range(2):
                    lquad = (4 * j + wave) * 8 + sub
                    kb = (lane & 7) ^ ((lquad >> 1) & 7)
                    src = (q0 * KB + it * (BK // 16)) * 16 + ((min(q0 + lquad, nquads - 1) - q0) * KB + kb) * 16
                    assert 0 <= src and src + 16 <= tiled.size
                    dst = (4 * j + wave) * 1024 + 16 * lane
                    sb[dst:dst + 16] = tiled[src:src + 16]
        # --- fragments and MFMAs: wave (wm, wn) owns rows wm*64 .. +63, quads wn*32 .. +31
        for wave in range(4):
            wm, wn = wave >> 1, wave & 1
            lanes = np.arange(64)
            frow0 = wm * 64 + (lanes & 31)
            khalf = lanes >> 5
            fquad = wn * 32 + (lanes & 31)
            acc = np.zeros((2, 4, 64, 16), dtype=np.int64)
            for ks in range(4):
                seg = 2 * ks + khalf
                a_unit = frow0 * 8 + (seg ^ ((frow0 >> 1) & 7))
                b_unit = fquad * 8 + (seg ^ ((fquad >> 1) & 7))
                assert a_unit.max() + 32 * 8 < kA and b_unit.max() < kB
                ra0 = np.stack([sa[16 * u:16 * u + 16].view(np.int8) for u in a_unit]).astype(np.int64)
                ra1 = np.stack([sa[16 * (u + 256):16 * (u + 256) + 16].view(np.int8) for u in a_unit]).astype(np.int64)
                rb = np.stack([sb[16 * u:16 * u + 16].view(np.uint32) for u in b_unit])
                for j in range(4):
                    bf = np.stack([decode_b(int(rb[l, j])) for l in range(64)])
                    acc[0, j] += mfma_32x32x32_i8(ra0, bf)
                    acc[1, j] += mfma_32x32x32_i8(ra1, bf)
            # --- epilogue mapping: lane owns columns 4*fquad + j, rows wm*64 + mt*32 + 8*(r//4) + 4*(lane//32) + r%4
            for mt in range(2):
                for j in range(4):
                    for l in range(64):
                        for r in range(16):
                            lrow = wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * (l >> 5) + (r & 3)
                            result[lrow, fquad[l] * 4 + j] += acc[mt, j, l, r]
    rows = min(TM, M - m0)
    cols = min(BN, N - n0)
    rowsum = q.astype(np.int64).sum(axis=1)[m0:m0 + rows, None]
    want = (q_src.astype(np.int64) @ vals.astype(np.int64))[m0:m0 + rows, n0:n0 + cols]
    assert (result[:rows, :cols] - rowsum == want).all()


def prefill_ring_schedule(mt, iters):
    """A wave's program of ring events for `iters` K steps, in program order, as gemm_t2_i8_mfma_kernel<mt>
    issues them: ("load", step, d) starts transfer d of K step `step` into buffer step % 3, ("read", step)
    reads fragments of that step's buffer, ("wait", n) is s_waitcnt vmcnt(n) lgkmcnt(0), ("barrier",)."""
    loads = 2 * mt + 2
    ev = [("load", 0, d) for d in range(loads)] + [("load", 1, d) for d in range(loads)]
    ev += [("wait", loads), ("barrier",), ("read", 0), ("read", 0)]
    for it in range(iters):
        ev += [("load", it + 2, 0), ("read", it), ("load", it + 2, 1)]           # sub-step 0 and its middle
        ev += [("load", it + 2, 2), ("read", it), ("load", it + 2, 3)]           # sub-step 1
        if mt == 2:
            ev += [("load", it + 2, 4)]
        ev += [("wait", 5 if mt == 2 else 4), ("barrier",)]
        ev += [("read", it + 1)]                                                   # sub-step 2
        if mt == 2:
            ev += [("load", it + 2, 5)]
        ev += [("read", it + 1)]                                                   # sub-step 3
    ev += [("wait", 0)]
    return ev, loads


@pytest.mark.parametrize("mt,iters", [(2, 1), (2, 2), (2, 7), (1, 1), (1, 5)])
def test_prefill_ring_schedule_never_reads_early_or_overwrites_late(mt, iters):
    """The hand-counted vmcnt of the prefill kernel's three-stage ring, replayed: loads retire in order,
    a wait for n leaves the newest n in flight, and every wave runs the same program between barriers.
    (a) Every read finds all loads of its K step landed in every wave: each wave waited for them before
    the last barrier.  (b) A load into a buffer is issued only behind a barrier that every wave reached
    after its last read of that buffer's previous content had returned."""
    ev, loads = prefill_ring_schedule(mt, iters)
    in_flight = []                 # (step, d), oldest first
    landed = set()                 # loads this wave knows to have landed
    published = set()              # landed before the last barrier: true of all four waves
    reads_returned = set()         # steps whose reads so far have returned (lgkmcnt(0)), as of the last wait
    reads_issued = []              # steps read since the last wait
    safe_to_overwrite = set()      # steps every wave has finished reading, as of the last barrier
    last_read_at = {}
    for i, e in enumerate(ev):
        if e[0] == "read":
            last_read_at[e[1]] = i
    for i, e in enumerate(ev):
        if e[0] == "load":
            step = e[1]
            if step >= 3:
                assert step - 3 in safe_to_overwrite, (i, e)
            in_flight.append((step, e[2]))
        elif e[0] == "wait":
            while len(in_flight) > e[1]:
                landed.add(in_flight.pop(0))
            reads_returned = set(reads_issued)
            pending_done = {s for s in reads_returned if last_read_at[s] < i}
            reads_done_before_wait = pending_done
        elif e[0] == "barrier":
            published = set(landed)
            safe_to_overwrite |= reads_done_before_wait
        elif e[0] == "read":
            step = e[1]
            if step < iters:       # past the last step the buffer holds nothing new and the result is unused
                assert all((step, d) in published for d in range(loads)), (i, e)
            reads_issued.append(step)
    assert not in_flight           # nothing still writes LDS when the epilogue reuses it


# ---- decode GEMV (gemv.hip): the 4-bit planes that feed v_dot8 ---------------------------------------------

def test_gemv_nibble_planes_reproduce_the_int8_dot_product():
    """to_nibble_planes() and the even / odd 2-bit fields of a tiled weight word: an int8 activation is
    16 * hi + lo (hi a signed, lo an unsigned nibble); (w & 0x33333333) and ((w >> 2) & 0x33333333) are
    the codes of k = (0,8,1,9,2,10,3,11) and (4,12,5,13,6,14,7,15) as nibbles, the order the planes are
    packed in, so that 16 * (sdot8 + sdot8) + (udot8 + udot8) is the dot product with the 16 codes."""
    rng = np.random.default_rng(5)
    for _ in range(200):
        a = rng.integers(-128, 128, size=16).astype(np.int8)
        code = rng.integers(0, 3, size=16).astype(np.uint32)
        w = np.uint32(0)
        for k in range(16):
            s, b = k // 4, k % 4
            w |= np.uint32(int(code[k]) << (8 * b + 2 * s))
        ax, ay, az, aw = (int(x) for x in a.view(np.uint32))
        px = ((ax >> 4) & 0x0F0F0F0F) | (az & 0xF0F0F0F0)
        py = (ax & 0x0F0F0F0F) | ((az & 0x0F0F0F0F) << 4)
        pz = ((ay >> 4) & 0x0F0F0F0F) | (aw & 0xF0F0F0F0)
        pw = (ay & 0x0F0F0F0F) | ((aw & 0x0F0F0F0F) << 4)
        ev, od = int(w) & 0x33333333, (int(w) >> 2) & 0x33333333

        def nibbles(x, signed):
            out = [(x >> (4 * i)) & 15 for i in range(8)]
            return [n - 16 if signed and n >= 8 else n for n in out]

        def dot8(x, y, signed):
            return sum(p * q for p, q in zip(nibbles(x, signed), nibbles(y, signed)))

        hi = dot8(px, ev, True) + dot8(pz, od, True)
        lo = dot8(py, ev, False) + dot8(pw, od, False)
        assert 16 * hi + lo == int((a.astype(np.int64) * code.astype(np.int64)).sum())

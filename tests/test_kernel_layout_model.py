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


@pytest.mark.parametrize("M,K,N", [(16, 256, 64), (5, 384, 130), (16, 1100, 64), (3, 128, 37), (9, 4096, 64)])
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
    lanes = np.arange(64)
    sub, slot = lanes >> 3, lanes & 7
    ql, g = lanes & 15, lanes >> 4
    for group in range(groups):
        for split in range(splits):
            for wave in range(nw):
                gw, gn = split * nw + wave, splits * nw
                s0, s1 = gw * stages // gn, (gw + 1) * stages // gn
                assert s1 > s0
                lds = np.zeros((D, 4096), dtype=np.uint8)       # this wave's ring
                acc = np.zeros((64, 4, 4), dtype=np.int64)      # [lane][tile j][register i]

                def issue(s, d):
                    sc = max(min(s, s1 - 1), 0)
                    for h in range(2):
                        row = 8 * h + sub
                        kb = slot ^ ((row >> 1) & 7)
                        w_off = (row * KB + kb) * 16 + (group * 16 * KB + sc * 8) * 16
                        a_off = np.minimum(row, M - 1) * kpad + kb * 16 + sc * 128
                        assert w_off.min() >= 0 and w_off.max() + 16 <= tiled.size
                        assert a_off.min() >= 0 and a_off.max() + 16 <= qbytes.size
                        for l in range(64):                      # lane l's 16 bytes land at base + 16 l
                            lds[d, h * 1024 + 16 * l:h * 1024 + 16 * l + 16] = tiled[w_off[l]:w_off[l] + 16]
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
    got = acc_total.transpose(1, 0, 2).reshape(16, groups * 64)[:M, :N]
    # weights are codes = value + 1: the kernel subtracts the token's sum of q in the epilogue
    want = q_src.astype(np.int64) @ vals.astype(np.int64)
    rowsum = q.astype(np.int64).sum(axis=1, keepdims=True)
    assert (got - rowsum == want).all()

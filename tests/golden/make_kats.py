"""Re-derives tests/golden/ternary_kats.json from the reference's literal test inputs.

The arithmetic below is written out by hand in numpy f32, step by step, from the text
of crates/ronn-providers/src/bitnet/quantization.rs:67-153 and kernels.rs:134-178; it
does not import the oracle, the device library or the reference.  Run it to print the
vectors; the committed JSON holds the same numbers.
"""
import json
import struct

import numpy as np


def bits(x):
    return "0x%08x" % struct.unpack("<I", struct.pack("<f", float(x)))[0]


def quantize(data):
    x = np.array(data, dtype=np.float32)
    s = np.float32(0)
    for v in x:                                  # sequential f32 fold (:79)
        s = np.float32(s + np.abs(v))
    thr = np.float32(np.float32(s / np.float32(x.size)) * np.float32(0.7))
    nz = [np.abs(v) for v in x if np.abs(v) > thr]  # survivors in order (:82-91)
    ss = np.float32(0)
    for v in nz:
        ss = np.float32(ss + v)
    scale = np.float32(1.0) if not nz else np.float32(ss / np.float32(len(nz)))
    codes = [1 if np.abs(v) <= thr else (2 if v > 0 else 0) for v in x]   # :138-144
    packed = bytearray((len(codes) + 3) // 4)
    for i, c in enumerate(codes):
        packed[i // 4] |= c << ((i % 4) * 2)     # :146-149
    values = [{0: -1, 1: 0, 2: 1, 3: 0}[c] for c in codes]                # :285-290
    return values, packed.hex(), thr, scale


def matmul(a, b, m, n, k):
    va, _, _, sa = quantize(a)
    vb, _, _, sb = quantize(b)
    acc, out = [], []
    for i in range(m):
        for j in range(n):
            d = sum(va[i * k + l] * vb[l * n + j] for l in range(k))
            acc.append(d)
            out.append(bits(np.float32(np.float32(np.float32(d) * sa) * sb)))  # :168
    return acc, out


if __name__ == "__main__":
    inputs = [[1.5, -2.0, 0.1, -0.05], [2.0, -1.5, 0.1, -0.05, 1.8, -2.1, 0.02, -0.01],
              [2.0, -1.5, 0.1, -0.05, 1.8, -2.1], [1.0, -2.0, 0.05, -1.5, 2.5, 0.1]]
    for d in inputs:
        v, p, t, s = quantize(d)
        print(json.dumps({"data": d, "values": v, "packed_hex": p, "threshold_bits": bits(t),
                          "scale_bits": bits(s)}))
    print(matmul(inputs[2], inputs[3], 2, 2, 3))

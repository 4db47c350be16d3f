"""Writes the committed known-answer fixtures for the BGEMM path.

The reference holds no golden vectors and none of it can be built or run here, so the
expected values below come from (a) bit patterns worked out by hand from the pack rule in
lowbit_kernel/csrc/utils/weight_prepacking.h:181-190 and (b) dense integer matmuls on
de-binarised operands written directly in numpy (no bit tricks, no oracle, no HIP code).
Both the C oracle and the HIP library are checked against these files.

Run:  python tests/golden/make_golden.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def pack_kat():
    """Hand-derived cases: list of (fp16 bit patterns of one row, expected words)."""
    P, Nn = 0x3C00, 0xBC00          # +1.0, -1.0
    cases = []

    def row(neg_positions, K=32, fill=P):
        r = [fill] * K
        for p in neg_positions:
            r[p] = Nn
        return r
    # element i negative -> bit 31-i (k<16: (x&0x8000)<<(16-k); k>=16: (x&0x8000)>>(k-16))
    cases.append({"halves": row([0]), "words": [0x80000000]})
    cases.append({"halves": row([15]), "words": [0x00010000]})
    cases.append({"halves": row([16]), "words": [0x00008000]})
    cases.append({"halves": row([31]), "words": [0x00000001]})
    cases.append({"halves": row([1, 2, 29]), "words": [0x60000004]})
    cases.append({"halves": row(range(32)), "words": [0xFFFFFFFF]})
    # special values: -0.0, +0.0, -inf, +inf, NaN with / without sign, +-subnormal
    specials = [0x8000, 0x0000, 0xFC00, 0x7C00, 0xFE00, 0x7E00, 0x8001, 0x0001]
    cases.append({"halves": specials + [P] * 24, "words": [0xAA000000]})
    # two words, second one ragged: K = 40 -> bits 31..24 of word 1, rest zero
    r = row([], K=40)
    r[32], r[39] = Nn, Nn
    cases.append({"halves": r, "words": [0x00000000, 0x81000000]})
    return cases


def ternary_kat():
    P, Nn = 0x3C00, 0xBC00
    # +-0 -> 0 ; subnormals are nonzero ; NaN counts as nonzero with its sign bit
    halves = [0x8000, 0x0000, Nn, P, 0x8001, 0x0001, 0xFE00, 0x7E00] + [0x0000] * 24
    return [{"halves": halves, "nz": [0x3F000000], "sg": [0x2A000000]}]


def dense_cases(seed=20240607):
    rng = np.random.default_rng(seed)
    out = {}
    shapes = [(8, 5, 32), (33, 7, 40), (32, 32, 128), (10, 3, 784), (64, 1, 256), (65, 17, 300)]
    for idx, (M, N, K) in enumerate(shapes):
        w = rng.standard_normal((M, K)).astype(np.float16)
        x = rng.standard_normal((N, K)).astype(np.float16)
        # sprinkle exact zeros of both signs
        zi = rng.integers(0, K, size=max(1, K // 16))
        x[:, zi] = np.float16(0.0)
        x[0, zi[: len(zi) // 2]] = np.float16(-0.0)
        w[0, zi[:2]] = np.float16(-0.0)
        a = (w.view(np.uint16) >> 15).astype(np.int64)      # 1 = sign bit set
        b = (x.view(np.uint16) >> 15).astype(np.int64)
        xs = x.view(np.uint16)
        t = np.where((xs & 0x7FFF) == 0, 0, np.where(xs >> 15, -1, 1)).astype(np.int64)
        out["w%d" % idx] = w.view(np.uint16)
        out["x%d" % idx] = x.view(np.uint16)
        out["and%d" % idx] = (b @ a.T).astype(np.int32)
        out["xor%d" % idx] = ((1 - 2 * b) @ (1 - 2 * a).T).astype(np.int32)
        out["attn%d" % idx] = ((1 - 2 * b) @ (1 - a).T).astype(np.int32)
        out["attnx%d" % idx] = ((1 - b) @ (1 - 2 * a).T).astype(np.int32)
        out["bwta%d" % idx] = (t @ (1 - 2 * a).T).astype(np.int32)
    out["n_cases"] = np.array(len(shapes))
    return out


def f16_rounding_kat():
    """Integers whose fp16 rounding exercises ties-to-even and overflow; expected bits via numpy."""
    vals = [0, 1, -1, 2047, 2048, 2049, 2050, 2051, 4097, 4098, 4099, 4101, 4102, 8196, 8188, 32784,
            32800, 65504, 65519, 65520, 65536, -2049, -2051, -65519, -65520, 16777215, -16777215, 1000001]
    exp = [int(np.float32(v).astype(np.float16).view(np.uint16)) for v in vals]
    return {"values": vals, "f16_bits": exp}


if __name__ == "__main__":
    with np.errstate(over="ignore"):
        rounding = f16_rounding_kat()
    with open(os.path.join(HERE, "pack_kat.json"), "w") as f:
        json.dump({"sign": pack_kat(), "ternary": ternary_kat(), "rounding": rounding}, f, indent=1)
    np.savez_compressed(os.path.join(HERE, "dense_kat.npz"), **dense_cases())
    print("wrote pack_kat.json, dense_kat.npz")

"""Writes tests/golden/half_golden.npz from the reference's own fp16 routines.

Run in the container where the reference tree is mounted, after
`make -C oracle` has built oracle/_ref/libhvdref.so from the reference's
common/half.h and common/half.cc (compiled in place; nothing is copied).
The fixture holds inputs and the reference's outputs only:

  h2f_out    uint32[65536]   HalfBits2Float bits for every half 0..65535
  f2h_in     uint32[N]       fp32 bit patterns: boundary cases + seeded random
  f2h_out    uint16[N]       Float2HalfBits of f2h_in
  sum_a/b    uint16[M]       seeded half pairs (incl. subnormals, inf, max)
  sum_out    uint16[M]       float16_sum(in=sum_a, inout=sum_b)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_util  # noqa: E402


def f2h_inputs():
    rng = np.random.default_rng(20240531)
    cases = [0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x7f800001, 0xff800001,
             0x7fffffff, 0x00000001, 0x80000001, 0x007fffff, 0x00800000]
    # every half value widened, plus its fp32 neighbours and the exact midpoints between halves
    h = np.arange(65536, dtype=np.uint16)
    w = h.view(np.float16).astype(np.float32).view(np.uint32)
    w = w[~np.isnan(w.view(np.float32))]
    # (strided with different phases to keep the fixture small)
    blocks = [np.array(cases, np.uint32), w[0::4], w[1::6] + np.uint32(1), w[2::6] - np.uint32(1),
              w[3::4] + np.uint32(0x1000), w[4::6] + np.uint32(0x0fff), w[5::6] + np.uint32(0x1001)]
    # magnitudes around the half subnormal range and the overflow threshold
    for e in range(127 - 30, 127 + 18):
        m = rng.integers(0, 1 << 23, 256, dtype=np.uint32)
        s = rng.integers(0, 2, 256, dtype=np.uint32) << np.uint32(31)
        blocks.append(s | np.uint32(e << 23) | m)
        blocks.append(s | np.uint32(e << 23) | (m & np.uint32(0x7fe000)) | np.uint32(0x1000))  # exact ties
    blocks.append(rng.integers(0, 1 << 32, 32768, dtype=np.uint64).astype(np.uint32))
    return np.concatenate(blocks)


def sum_inputs():
    rng = np.random.default_rng(77)
    a = rng.integers(0, 1 << 16, 1 << 15, dtype=np.uint32).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 1 << 15, dtype=np.uint32).astype(np.uint16)
    # a block of small magnitudes so that many sums are subnormal halves
    a[:8192] &= np.uint16(0x83ff)
    b[:8192] &= np.uint16(0x87ff)
    keep = ~(np.isnan(a.view(np.float16)) | np.isnan(b.view(np.float16)))
    return a[keep], b[keep]


def main():
    ref = oracle_util.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libhvdref.so is missing: run `make -C oracle` where the reference is mounted")
    h = np.arange(65536, dtype=np.uint16)
    h2f_out = ref.half2float(h).view(np.uint32)
    f2h_in = f2h_inputs()
    f2h_out = ref.float2half(f2h_in.view(np.float32))
    sa, sb = sum_inputs()
    sum_out = ref.float16_sum(sa, sb)
    out = os.path.join(HERE, "half_golden.npz")
    np.savez_compressed(out, h2f_out=h2f_out, f2h_in=f2h_in, f2h_out=f2h_out, sum_a=sa, sum_b=sb, sum_out=sum_out)
    print("wrote", out, os.path.getsize(out), "bytes;", f2h_in.size, "f2h cases,", sa.size, "sum cases")


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Writes tests/golden/refbuild_q80_vectors.npz: inputs and the Q8_0 activation codes / scales the reference's own x86
quantizer gives for them (quantize_oracle_q8_0 behind act_quant_q8_1, src/kernels/cpu/expert.cpp:92-130, 402-407).

Run in the build container, on a CPU with AVX-512 VNNI / VBMI (the options the reference compiles that file with):
`make -C oracle` builds oracle/_ref/libmaya_ref_q80.so from the reference's file where it lies; this script calls it.
The vectors let tests/test_oracle_pins.py hold the CPU checker's mo_quant_q80 to the reference on any machine.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def cases():
    """The input rows (each a multiple of 32 values, at most 2560): the reference test's five distributions
    (src/kernels/quantize_act_parity.cpp:236-270) and the boundary cases its quantizer's branches name."""
    rng = np.random.default_rng(20261126)
    n = 2560
    out = {}
    out["normal"] = rng.standard_normal(n).astype(np.float32)
    out["small_1e-6"] = (rng.standard_normal(n) * 1e-6).astype(np.float32)
    out["zeros"] = np.zeros(n, dtype=np.float32)
    half = ((np.arange(n) % 200) - 100 + 0.5).astype(np.float32)      # x / d on exact .5 boundaries: amax 127 a block
    half[0::32] = 127.0
    out["exact_halves"] = half
    ext = np.zeros(n, dtype=np.float32)
    ext[0::32] = 1000.0 + (np.arange(n // 32) % 7)
    out["one_extreme"] = ext
    both = rng.standard_normal(n).astype(np.float32)                   # +amax and -amax in one block, either order
    both[0::64], both[5::64] = 3.0, -3.0
    both[32::64], both[39::64] = -3.0, 3.0
    out["both_sign_maxima"] = both
    big = (rng.standard_normal(n) * 3e6).astype(np.float32)            # amax / 127 past 65504 in some blocks: the clamp
    big[0::96] = 1.2e7
    out["past_fp16_range"] = big
    sub = (rng.standard_normal(n) * 2e-7).astype(np.float32)           # FP16-subnormal block scales
    out["subnormal_scale"] = sub
    wide = (rng.standard_normal(n) * np.exp(rng.uniform(-8, 8, n))).astype(np.float32)
    out["wide_range"] = wide
    return out


def main():
    path = os.path.join(ROOT, "oracle", "_ref", "libmaya_ref_q80.so")
    if not os.path.exists(path):
        sys.exit("oracle/_ref/libmaya_ref_q80.so is missing: run `make -C oracle` where the reference tree is present")
    if "avx512_vnni" not in open("/proc/cpuinfo").read():
        sys.exit("this CPU lacks AVX-512 VNNI: the reference's expert.cpp cannot run here")
    R = C.CDLL(path)
    R.ref_q80_quant.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
    out = {}
    for name, x in cases().items():
        q = np.zeros(x.size, dtype=np.int8)
        d = np.zeros(x.size // 32, dtype=np.float32)
        assert R.ref_q80_quant(x.ctypes.data, x.size, q.ctypes.data, d.ctypes.data) == 0
        out[name + "_x"], out[name + "_q"], out[name + "_d"] = x, q, d
    dst = os.path.join(HERE, "refbuild_q80_vectors.npz")
    np.savez_compressed(dst, **out)
    print(dst, os.path.getsize(dst), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()

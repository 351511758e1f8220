#!/usr/bin/env python3
"""Writes tests/golden/refbuild_vectors.npz: inputs and the outputs the reference's own CPU expert sources give for them.

Run in the build container, where the reference tree is present: `make -C oracle` compiles those sources in place into
oracle/_ref/libmaya_ref.so (nothing of the reference is copied), and this script calls it on seeded constructed blocks.
The vectors (inputs + expected outputs, a few hundred KB) let tests/test_golden_vectors.py hold the CPU checker to the
reference on a machine that has neither the reference tree nor its build.
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [os.path.join(ROOT, "project-maya_amd"), os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")]

import oracle_py  # noqa: E402
import synth  # noqa: E402


def main():
    R = oracle_py.ref()
    if R is None:
        sys.exit("oracle/_ref/libmaya_ref.so is missing: run `make -C oracle` where the reference tree is present")
    out = {}
    rng = np.random.default_rng(20261125)

    # Q8_K activation blocks (strata::ds4::par::quant): codes and block scales
    k = 1536
    x = rng.standard_normal(k).astype(np.float32)
    x[256:512] = 0.0
    x[512:768] = np.float32(0.5)
    x[768], x[769] = -3.0, 3.0
    x[1024:1280] = (np.arange(256) - 128).astype(np.float32) / 254.0 * 3.0
    act = np.zeros(int(R.ref_par_act_bytes(k)), dtype=np.uint8)
    R.ref_par_quant(x.ctypes.data, k, act.ctypes.data)
    out["q8k_x"] = x
    out["q8k_codes"] = act[:k].view(np.int8).copy()
    out["q8k_scales"] = act[k:].view(np.float32).copy()

    # contract row dots and gate/up rows (strata::kernels::cpu::iq256_rows / iq256_gu_rows)
    for t in (22, 12, 29):
        kk, n = 768, 12
        w = synth.constructed_rows(t, n, kk, rng)
        xs = rng.standard_normal((2, kk)).astype(np.float32)
        xs[1] *= 21.0
        acts = [oracle_py.quant_q8k(v) for v in xs]     # inputs of the rows: stored, not trusted
        actp = (C.c_void_p * 2)(*[a.ctypes.data for a in acts])
        outs = [np.zeros(n, dtype=np.float32) for _ in range(2)]
        outp = (C.c_void_p * 2)(*[o.ctypes.data for o in outs])
        R.ref_iq256_rows(t, w.ctypes.data, oracle_py.row_bytes(t, kk), kk, actp, 2, outp, 0, n)
        out["rows%d_w" % t] = w
        out["rows%d_act" % t] = np.stack(acts)
        out["rows%d_y" % t] = np.stack(outs)
        blob = np.concatenate([synth.constructed_rows(t, n, kk, rng, d_scale=4.0), synth.constructed_rows(t, n, kk, rng)])
        rb = oracle_py.row_bytes(t, kk)
        gouts = [np.zeros(n, dtype=np.float32) for _ in range(2)]
        goutp = (C.c_void_p * 2)(*[o.ctypes.data for o in gouts])
        R.ref_iq256_gu_rows(t, blob.ctypes.data, rb, n * rb, kk, actp, 2, goutp, 0, n)
        out["gu%d_w" % t] = blob
        out["gu%d_h" % t] = np.stack(gouts)

    # IQ2_S rows in the device-arithmetic lane (strata::ds4::par::row_ref), 32 and 16 lanes a row
    kk, n = 2048, 6
    w = synth.constructed_rows(22, n, kk, rng)
    x = rng.standard_normal(kk).astype(np.float32)
    act = np.zeros(int(R.ref_par_act_bytes(kk)), dtype=np.uint8)
    R.ref_par_quant(x.ctypes.data, kk, act.ctypes.data)
    rb = oracle_py.row_bytes(22, kk)
    R.ref_par_row.restype = C.c_float
    out["lane_w"], out["lane_act"] = w, act
    out["lane_y"] = np.array([[R.ref_par_row(22, w.ctypes.data + r * rb, kk, act.ctypes.data, lpr) for r in range(n)]
                              for lpr in (32, 16)], dtype=np.float32)

    # exp_portable / swiglu_portable
    ys = np.concatenate([rng.uniform(-100, 100, 600), [0.0, -87.0, -87.5, 88.9, 89.0, 127.0]]).astype(np.float32)
    R.ref_exp_portable.restype = C.c_float
    R.ref_exp_portable.argtypes = [C.c_float]
    out["exp_x"] = ys
    out["exp_y"] = np.array([R.ref_exp_portable(float(y)) for y in ys], dtype=np.float32)

    # Q4_K / Q8_0 dequant (include/strata/artifact/dequant.hpp)
    b4 = synth.constructed_rows(12, 1, 256 * 6, rng)
    o4 = np.zeros(256 * 6, dtype=np.float32)
    for i in range(6):
        R.ref_dequant_q4_K(b4.ctypes.data + 144 * i, o4.ctypes.data + 1024 * i)
    out["dq4k_w"], out["dq4k_y"] = b4, o4
    b8 = synth.constructed_rows(8, 1, 32 * 20, rng)
    o8 = np.zeros(32 * 20, dtype=np.float32)
    for i in range(20):
        R.ref_dequant_q8_0(b8.ctypes.data + 34 * i, o8.ctypes.data + 128 * i)
    out["dq80_w"], out["dq80_y"] = b8, o8

    # EXL3 mat-vec (exl3_ref.cpp: exl3_inner_k2 + exl3_mv)
    kk, n, k2, cb = 256, 128, 6, 2
    tr = rng.integers(0, 2 ** 32, (kk // 16) * (n // 16) * 4 * k2, dtype=np.uint64).astype(np.uint32)
    wv = np.zeros((kk, n), dtype=np.float32)
    R.ref_exl3_inner(tr.ctypes.data, n // 16, kk, n, k2, cb, wv.ctypes.data)
    suh = (rng.integers(0, 2, kk) * 2 - 1).astype(np.float16).view(np.uint16)
    svh = ((rng.integers(0, 2, n) * 2 - 1) * rng.uniform(0.25, 2, n)).astype(np.float16).view(np.uint16)
    xv = rng.standard_normal(kk).astype(np.float32)
    yv = np.zeros(n, dtype=np.float32)
    R.ref_exl3_mv(wv.ctypes.data, suh.ctypes.data, svh.ctypes.data, kk, n, xv.ctypes.data, yv.ctypes.data)
    out.update(exl3_tr=tr, exl3_w=wv.astype(np.float16), exl3_suh=suh, exl3_svh=svh, exl3_x=xv, exl3_y=yv)

    path = os.path.join(HERE, "refbuild_vectors.npz")
    # IQ2_XXS rows (a generator of its own, so that the vectors above keep their values)
    rng16 = np.random.default_rng(20261216)
    for t in (16,):
        kk, n = 768, 12
        w = synth.constructed_rows(t, n, kk, rng16)
        xs = rng16.standard_normal((2, kk)).astype(np.float32)
        xs[1] *= 21.0
        acts = [oracle_py.quant_q8k(v) for v in xs]
        actp = (C.c_void_p * 2)(*[a.ctypes.data for a in acts])
        outs = [np.zeros(n, dtype=np.float32) for _ in range(2)]
        outp = (C.c_void_p * 2)(*[o.ctypes.data for o in outs])
        R.ref_iq256_rows(t, w.ctypes.data, oracle_py.row_bytes(t, kk), kk, actp, 2, outp, 0, n)
        out["rows%d_w" % t] = w
        out["rows%d_act" % t] = np.stack(acts)
        out["rows%d_y" % t] = np.stack(outs)
        blob = np.concatenate([synth.constructed_rows(t, n, kk, rng16, d_scale=4.0), synth.constructed_rows(t, n, kk, rng16)])
        rb = oracle_py.row_bytes(t, kk)
        gouts = [np.zeros(n, dtype=np.float32) for _ in range(2)]
        goutp = (C.c_void_p * 2)(*[o.ctypes.data for o in gouts])
        R.ref_iq256_gu_rows(t, blob.ctypes.data, rb, n * rb, kk, actp, 2, goutp, 0, n)
        out["gu%d_w" % t] = blob
        out["gu%d_h" % t] = np.stack(gouts)

    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()

"""The CPU checker against the reference build (oracle/_ref: the reference's own CPU expert sources compiled in place),
bit for bit, on seeded constructed blocks.  Skipped where the reference build does not exist; the committed vectors in
tests/golden/refbuild_vectors.npz (test_golden_vectors.py) carry the same checks to such a machine."""
import ctypes as C

import numpy as np
import pytest

import synth

TYPES_256 = (22, 12, 29, 16)


def _acts(oracle, k, nt, seed):
    rng = np.random.default_rng(seed)
    xs = rng.standard_normal((nt, k)).astype(np.float32)
    xs[0, :7] = 0.0
    if nt > 1:
        xs[1] *= 37.5
    return xs, [oracle.quant_q8k(x) for x in xs]


def test_q8k_quant_matches_reference_build(oracle, refbuild):
    rng = np.random.default_rng(1)
    k = 2048
    x = rng.standard_normal(k).astype(np.float32)
    x[256:512] = 0.0                     # an all-zero block
    x[512:768] = np.float32(0.5)         # ties everywhere: the first maximum wins, q = -127 * ... exact halves
    x[768] = -3.0
    x[769] = 3.0                         # equal magnitudes: the first (negative) one sets the sign of iscale
    x[1024:1280] = (np.arange(256) - 128).astype(np.float32) / 254.0 * 3.0   # exact .5 products
    blocks = oracle.quant_q8k(x)
    d, qs, bs = oracle.q8k_fields(blocks)
    act = np.zeros(int(refbuild.ref_par_act_bytes(k)), dtype=np.uint8)
    refbuild.ref_par_quant(x.ctypes.data, k, act.ctypes.data)
    rq = act[:k].view(np.int8)
    rd = act[k:].view(np.float32).reshape(-1, 8)
    assert np.array_equal(qs, rq)
    assert np.array_equal(d.view(np.uint32), rd[:, 0].view(np.uint32))
    assert np.array_equal(bs.sum(axis=1), qs.astype(np.int32).reshape(-1, 256).sum(axis=1))
    assert np.array_equal(bs, qs.astype(np.int32).reshape(-1, 16, 16).sum(axis=2))
    assert d[1] == 0 and not qs[256:512].any()


@pytest.mark.parametrize("t", TYPES_256)
def test_rows_bit_exact(oracle, refbuild, t):
    k, n, nt = 1024, 24, 3
    rng = np.random.default_rng(100 + t)
    w = synth.constructed_rows(t, n, k, rng)
    xs, acts = _acts(oracle, k, nt, 7)
    actp = (C.c_void_p * nt)(*[a.ctypes.data for a in acts])
    outs = [np.zeros(n, dtype=np.float32) for _ in range(nt)]
    outp = (C.c_void_p * nt)(*[o.ctypes.data for o in outs])
    assert refbuild.ref_iq256_supported(t)
    refbuild.ref_iq256_rows(t, w.ctypes.data, oracle.row_bytes(t, k), k, actp, nt, outp, 0, n)
    for i in range(nt):
        got = oracle.rows(t, w, k, n, acts[i])
        assert np.array_equal(got.view(np.uint32), outs[i].view(np.uint32)), (t, i, got[:4], outs[i][:4])
        # and both are the double dot of the dequantized operands to float rounding
        wf = oracle.dequant_rows(t, w, k, n).astype(np.float64)
        d, qs, _ = oracle.q8k_fields(acts[i])
        xf = qs.astype(np.float64).reshape(-1, 256) * d.astype(np.float64)[:, None]
        want = wf @ xf.reshape(-1)
        assert np.max(np.abs(got - want)) <= 2e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("t", TYPES_256)
def test_gu_rows_bit_exact(oracle, refbuild, t):
    k, n, nt = 512, 16, 2
    rng = np.random.default_rng(200 + t)
    blob = np.concatenate([synth.constructed_rows(t, n, k, rng, d_scale=4.0), synth.constructed_rows(t, n, k, rng)])
    xs, acts = _acts(oracle, k, nt, 9)
    rb = oracle.row_bytes(t, k)
    actp = (C.c_void_p * nt)(*[a.ctypes.data for a in acts])
    outs = [np.zeros(n, dtype=np.float32) for _ in range(nt)]
    outp = (C.c_void_p * nt)(*[o.ctypes.data for o in outs])
    refbuild.ref_iq256_gu_rows(t, blob.ctypes.data, rb, n * rb, k, actp, nt, outp, 0, n)
    L = oracle.lib()
    for i in range(nt):
        g = oracle.rows(t, blob[: n * rb], k, n, acts[i])
        u = oracle.rows(t, blob[n * rb:], k, n, acts[i])
        got = np.array([L.mo_swiglu(float(a), float(b), float("inf")) for a, b in zip(g, u)], dtype=np.float32)
        assert np.array_equal(got.view(np.uint32), outs[i].view(np.uint32))


def test_lane_order_rows_bit_exact(oracle, refbuild):
    """The device-arithmetic lane for IQ2_S (sub-blocks dealt to 32 / 16 lanes, fma(dx, d * isum, acc), lanes folded)."""
    k, n = 2048, 12
    rng = np.random.default_rng(31)
    w = synth.constructed_rows(22, n, k, rng)
    x = rng.standard_normal(k).astype(np.float32)
    act = np.zeros(int(refbuild.ref_par_act_bytes(k)), dtype=np.uint8)
    refbuild.ref_par_quant(x.ctypes.data, k, act.ctypes.data)
    q = act[:k].view(np.int8).copy()
    d32 = act[k:].view(np.float32).copy()
    rb = oracle.row_bytes(22, k)
    L = oracle.lib()
    for lpr in (32, 16):
        for r in range(n):
            want = refbuild.ref_par_row(22, w.ctypes.data + r * rb, k, act.ctypes.data, lpr)
            got = L.mo_row_lanes(22, w.ctypes.data + r * rb, k, q.ctypes.data, d32.ctypes.data, lpr)
            assert np.float32(got).view(np.uint32) == np.float32(want).view(np.uint32)


def test_exp_portable_bit_exact(oracle, refbuild):
    L = oracle.lib()
    rng = np.random.default_rng(4)
    ys = np.concatenate([rng.uniform(-100, 100, 4000), rng.standard_normal(2000) * 3, [0.0, -87.0, -87.5, 88.9, 89.0, 127.0]])
    for y in ys.astype(np.float32):
        a, b = np.float32(L.mo_exp_portable(float(y))), np.float32(refbuild.ref_exp_portable(float(y)))
        assert a.view(np.uint32) == b.view(np.uint32)
        if -80 < y < 80:
            assert abs(float(a) - np.exp(np.float64(y))) <= 1.2e-7 * np.exp(np.float64(y)) * 2
    for g, u, lim in ((1.5, -2.0, 0.0), (12.0, 9.0, 7.0), (-3.0, -11.0, 7.0)):
        a = np.float32(L.mo_swiglu_portable(g, u, lim))
        b = np.float32(refbuild.ref_swiglu_portable(g, u, lim))
        assert a.view(np.uint32) == b.view(np.uint32)


def test_f16_round_matches_reference_build(oracle, refbuild):
    L = oracle.lib()
    rng = np.random.default_rng(8)
    for v in np.concatenate([rng.standard_normal(3000) * 50, rng.standard_normal(1000) * 1e-6]).astype(np.float32):
        assert L.mo_f32_to_f16(float(v)) == refbuild.ref_f32_to_f16(float(v))

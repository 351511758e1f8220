"""The CPU checker against the committed vectors of the reference build (tests/golden/refbuild_vectors.npz, written by
tests/golden/make_refbuild_vectors.py from the reference's own CPU expert sources): bit for bit, with no reference tree
and no reference build on the machine."""
import ctypes as C
import os

import numpy as np
import pytest

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "refbuild_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    return np.load(PATH, allow_pickle=False)


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_q8k_blocks(oracle, vec):
    d, qs, bs = oracle.q8k_fields(oracle.quant_q8k(vec["q8k_x"]))
    assert np.array_equal(qs, vec["q8k_codes"])
    assert np.array_equal(bits(d), bits(vec["q8k_scales"].reshape(-1, 8)[:, 0]))
    assert np.array_equal(bs, qs.astype(np.int32).reshape(-1, 16, 16).sum(axis=2))


@pytest.mark.parametrize("t", (22, 12, 29, 16))
def test_contract_rows_and_gate_up(oracle, vec, t):
    k, n = 768, 12
    acts = vec["rows%d_act" % t]
    for i in range(2):
        got = oracle.rows(t, vec["rows%d_w" % t], k, n, acts[i])
        assert np.array_equal(bits(got), bits(vec["rows%d_y" % t][i]))
    blob = vec["gu%d_w" % t]
    rb = oracle.row_bytes(t, k)
    L = oracle.lib()
    for i in range(2):
        g = oracle.rows(t, blob[:n * rb], k, n, acts[i])
        u = oracle.rows(t, blob[n * rb:], k, n, acts[i])
        h = np.array([L.mo_swiglu(float(a), float(b), float("inf")) for a, b in zip(g, u)], dtype=np.float32)
        assert np.array_equal(bits(h), bits(vec["gu%d_h" % t][i]))


def test_lane_order_rows(oracle, vec):
    k, n = 2048, 6
    w, act = np.ascontiguousarray(vec["lane_w"]), np.ascontiguousarray(vec["lane_act"])
    q = act[:k].view(np.int8).copy()
    d32 = act[k:].view(np.float32).copy()
    rb = oracle.row_bytes(22, k)
    L = oracle.lib()
    for li, lpr in enumerate((32, 16)):
        got = np.array([L.mo_row_lanes(22, w.ctypes.data + r * rb, k, q.ctypes.data, d32.ctypes.data, lpr) for r in range(n)],
                       dtype=np.float32)
        assert np.array_equal(bits(got), bits(vec["lane_y"][li]))


def test_exp_portable(oracle, vec):
    L = oracle.lib()
    got = np.array([L.mo_exp_portable(float(y)) for y in vec["exp_x"]], dtype=np.float32)
    assert np.array_equal(bits(got), bits(vec["exp_y"]))


def test_q4k_q80_dequant(oracle, vec):
    assert np.array_equal(bits(oracle.dequant_rows(12, vec["dq4k_w"], 256 * 6, 1)[0]), bits(vec["dq4k_y"]))
    assert np.array_equal(bits(oracle.dequant_rows(8, vec["dq80_w"], 32 * 20, 1)[0]), bits(vec["dq80_y"]))


def test_exl3_inner_and_mv(oracle, vec):
    k, n = 256, 128
    w = oracle.exl3_inner(vec["exl3_tr"], k, n, 6, 2)
    assert np.array_equal(w.astype(np.float16).view(np.uint16), vec["exl3_w"].view(np.uint16))
    y = oracle.exl3_mv(w, vec["exl3_suh"], vec["exl3_svh"], vec["exl3_x"])
    assert np.array_equal(bits(y), bits(vec["exl3_y"]))

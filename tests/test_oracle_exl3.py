"""The CPU checker's EXL3 decoder against the reference's own golden vectors (made by exllamav3 itself) and, where it
exists, against the reference build of exl3_ref.cpp."""
import glob
import os
import struct

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "exl3-exllamav3")


def read_exh1(path):
    b = open(path, "rb").read()
    assert b[:4] == b"EXH1"
    k2, ki, nj, cb, words = struct.unpack_from("<iiiii", b, 4)
    assert words == 8 * k2
    o = 24
    n_tr = ki * nj * words * 2
    n_st = ki * nj * 256 * 2
    assert len(b) == o + n_tr + 2 * n_st
    tr = np.frombuffer(b, dtype="<i2", count=ki * nj * words, offset=o).reshape(ki, nj, words)
    st = np.frombuffer(b, dtype="<u2", count=ki * nj * 256, offset=o + n_tr).reshape(ki, nj, 256)
    wh = np.frombuffer(b, dtype="<u2", count=ki * nj * 256, offset=o + n_tr + n_st).reshape(ki * 16, nj * 16)
    return dict(k2=k2, ki=ki, nj=nj, cb=cb, trellis=tr, states=st, w_hat=wh)


FILES = sorted(glob.glob(os.path.join(GOLD, "exl3_k2_*_cb*.bin")))


def test_fixture_set_complete():
    assert len(FILES) == 13
    assert os.path.join(GOLD, "exl3_k2_6_cb2.bin") in FILES


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
def test_states_and_weights_match_exllamav3(oracle, path):
    f = read_exh1(path)
    L = oracle.lib()
    words = np.ascontiguousarray(f["trellis"]).view(np.uint32).reshape(f["ki"], f["nj"], 4 * f["k2"])
    st = np.zeros(256, dtype=np.uint16)
    for i in range(f["ki"]):
        for j in range(f["nj"]):
            tile = np.ascontiguousarray(words[i, j])
            L.mo_exl3_tile_states(tile.ctypes.data, f["k2"], st.ctypes.data)
            assert np.array_equal(st, f["states"][i, j]), (i, j)
    w = oracle.exl3_inner(words.reshape(-1), 16 * f["ki"], 16 * f["nj"], f["k2"], f["cb"])
    assert np.array_equal(w.astype(np.float16).view(np.uint16), f["w_hat"])
    assert np.array_equal(w.astype(np.float16).astype(np.float32), w)      # every value is an FP16 value


def test_mul1_state_zero(oracle):
    # state 0: bytesum 0 -> fp16(1024 * k_inv + k_bias) (tests/exl3_test.cu:143-144)
    k_inv = np.array([0x1EEE], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    k_bias = np.array([0xC931], dtype=np.uint16).view(np.float16).astype(np.float64)[0]
    want = np.float16(1024.0 * k_inv + k_bias)
    assert np.float32(oracle.lib().mo_exl3_decode(0, 2)) == np.float32(want)


def test_hadamard_involution_and_closed_form(oracle):
    rng = np.random.default_rng(5)
    v = rng.standard_normal(384).astype(np.float32)
    a = v.copy()
    oracle.lib().mo_exl3_had128(a.ctypes.data, a.size)
    # Sylvester closed form: H[i][j] = (-1)^popcount(i & j) / sqrt(128)
    i = np.arange(128)
    H = (1 - 2 * (np.array([[bin(x & y).count("1") & 1 for y in i] for x in i]))) / np.sqrt(128.0)
    want = (v.reshape(3, 128).astype(np.float64) @ H.T).reshape(-1)
    assert np.max(np.abs(a - want)) < 1e-5
    b = a.copy()
    oracle.lib().mo_exl3_had128(b.ctypes.data, b.size)
    assert np.max(np.abs(b - v)) < 1e-5


def test_against_reference_build(oracle, refbuild):
    rng = np.random.default_rng(12)
    L = oracle.lib()
    for cb in (0, 1, 2):
        for s in rng.integers(0, 65536, 3000):
            a, b = np.float32(L.mo_exl3_decode(int(s), cb)), np.float32(refbuild.ref_exl3_decode(int(s), cb))
            assert a.view(np.uint32) == b.view(np.uint32)
    k, n, k2 = 256, 128, 6
    tr = rng.integers(0, 2**32, size=(k // 16) * (n // 16) * 4 * k2, dtype=np.uint32)
    w = oracle.exl3_inner(tr, k, n, k2, 2)
    w2 = np.zeros_like(w)
    refbuild.ref_exl3_inner(tr.ctypes.data, n // 16, k, n, k2, 2, w2.ctypes.data)
    assert np.array_equal(w.view(np.uint32), w2.view(np.uint32))
    suh = (rng.uniform(0.25, 2, k) * rng.choice([-1, 1], k)).astype(np.float16).view(np.uint16)
    svh = (rng.uniform(0.25, 2, n) * rng.choice([-1, 1], n)).astype(np.float16).view(np.uint16)
    x = rng.standard_normal(k).astype(np.float32)
    y = oracle.exl3_mv(w, suh, svh, x)
    y2 = np.zeros(n, dtype=np.float32)
    refbuild.ref_exl3_mv(w.ctypes.data, suh.ctypes.data, svh.ctypes.data, k, n, x.ctypes.data, y2.ctypes.data)
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))

"""What holds the CPU checker's Q8_0 activation quantizer, its Q8_0 x Q8_0 row dot and its IQ1_S decode / row dot to the
reference without the device: the reference's own x86 quantizer (golden vectors made from it, and the live build where
it exists), independent numpy restatements written from the format definitions, and IQ1_M - whose row dot the reference
build pins bit for bit - as the carrier of every IQ1_S block (an IQ1_M block can say everything an IQ1_S block says)."""
import ctypes as C
import os

import numpy as np
import pytest

import synth

HERE = os.path.dirname(os.path.abspath(__file__))
Q8_0, IQ1_S, IQ1_M = 8, 19, 29


# ------------------------------------------------------------------------------------------------ Q8_0 activations

def q80_fields(blocks):
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, 34)
    return b[:, 0:2].copy().view(np.uint16).reshape(-1), b[:, 2:34].copy().view(np.int8).reshape(-1)


def q80_numpy(x):
    """The x86 contract written out independently (ggml-cpu's quantize_row_q8_0 as src/kernels/cpu/expert.cpp:92-130 restates
    it): every step in float32, nearest-even codes, the scale stored as FP16 and kept finite."""
    xb = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.max(np.abs(xb), axis=1)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        d = (amax / np.float32(127.0)).astype(np.float32)
        big = d > np.float32(65504.0)
        d = np.where(big, np.float32(65504.0), d)
        inv = np.where(amax == 0, np.float32(0), np.where(big, np.float32(1.0) / np.float32(65504.0),
                                                           np.float32(127.0) / amax)).astype(np.float32)
    prod = (xb * inv[:, None]).astype(np.float32)
    q = np.clip(np.rint(prod), -128, 127).astype(np.int8)     # np.rint: halves to even
    return d.astype(np.float16).view(np.uint16), q.reshape(-1)


def q80_roundf(x):
    """ggml's scalar quantize_row_q8_0_ref: roundf(x * (1 / d)), halves away from zero."""
    xb = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.max(np.abs(xb), axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    p = (xb * inv[:, None]).astype(np.float32)
    return (np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))).astype(np.int8).reshape(-1)


def q80_gpu_reference(x):
    """The reference's GPU quantize_q8_0 and its host twin (src/kernels/quantize_act_parity.cpp:47-70): rint of the double
    quotient x / d32."""
    xb = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.max(np.abs(xb), axis=1)
    d32 = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint(xb.astype(np.float64) / d32.astype(np.float64)[:, None])
    q = np.where(amax[:, None] == 0, 0.0, q)
    return np.clip(q, -128, 127).astype(np.int8).reshape(-1)


@pytest.fixture(scope="module")
def q80_golden():
    return np.load(os.path.join(HERE, "golden", "refbuild_q80_vectors.npz"))


def q80_names(g):
    return sorted(k[:-2] for k in g.files if k.endswith("_x"))


def test_q80_quantizer_equals_the_reference_x86_quantizer(oracle, q80_golden):
    g = q80_golden
    assert len(q80_names(g)) >= 9
    for name in q80_names(g):
        x = g[name + "_x"]
        dbits, q = q80_fields(oracle.quant_act(Q8_0, x))
        assert np.array_equal(q, g[name + "_q"]), name
        # the reference keeps the FP16 scale widened to F32
        assert np.array_equal(dbits.view(np.float16).astype(np.float32).view(np.uint32), g[name + "_d"].view(np.uint32)), name


def test_q80_quantizer_equals_the_live_reference_build(oracle):
    path = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libmaya_ref_q80.so")
    if not os.path.exists(path) or "avx512_vnni" not in open("/proc/cpuinfo").read():
        pytest.skip("the reference's x86 quantizer was not built here, or this CPU cannot run it")
    R = C.CDLL(path)
    R.ref_q80_quant.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
    rng = np.random.default_rng(5)
    for scale in (1.0, 1e-4, 37.0, 3e5):
        x = (rng.standard_normal(2560) * scale).astype(np.float32)
        x[rng.integers(0, 2560, 40)] = 0.0
        q = np.zeros(x.size, dtype=np.int8)
        d = np.zeros(x.size // 32, dtype=np.float32)
        assert R.ref_q80_quant(x.ctypes.data, x.size, q.ctypes.data, d.ctypes.data) == 0
        dbits, got = q80_fields(oracle.quant_act(Q8_0, x))
        assert np.array_equal(got, q)
        assert np.array_equal(dbits.view(np.float16).astype(np.float32), d)


def test_q80_quantizer_equals_an_independent_closed_form(oracle, q80_golden):
    rng = np.random.default_rng(6)
    xs = [q80_golden[n + "_x"] for n in q80_names(q80_golden)]
    xs.append(rng.standard_normal(32 * 4096).astype(np.float32))
    # products on exact halves of either sign: amax 127 makes 127 / amax = 1, so x = n + 0.5 stays a tie
    t = (rng.integers(-126, 126, 32 * 512) + 0.5).astype(np.float32)
    t[0::32] = -127.0
    xs.append(t)
    for x in xs:
        dbits, q = q80_fields(oracle.quant_act(Q8_0, x))
        wd, wq = q80_numpy(x)
        assert np.array_equal(q, wq)
        assert np.array_equal(dbits, wd)
    # the ties went to even: 0.5 -> 0, 1.5 -> 2, -2.5 -> -2, and a wrong rule (away from zero) would not
    _, q = q80_fields(oracle.quant_act(Q8_0, t))
    assert np.array_equal(q, np.rint(t).astype(np.int8))
    assert not np.array_equal(q, q80_roundf(t))
    # zero blocks: scale 0, codes 0
    dbits, q = q80_fields(oracle.quant_act(Q8_0, np.zeros(64, dtype=np.float32)))
    assert not dbits.any() and not q.any()


def test_q80_the_three_statements_differ_only_next_to_a_boundary(oracle):
    """ggml's scalar form and the reference's GPU form give the same scale; their codes leave the x86 contract's by one
    step on a small share of N(0, 1) values (the product x * (127 / amax) against x * (1 / d) or x / d), never by more."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal(32 * 20000).astype(np.float32)
    _, q = q80_fields(oracle.quant_act(Q8_0, x))
    for other in (q80_roundf(x), q80_gpu_reference(x)):
        diff = np.abs(q.astype(np.int32) - other.astype(np.int32))
        assert diff.max() <= 1
        assert np.count_nonzero(diff) < 2e-4 * x.size
    # the reference test's own constructed cases on which every statement agrees (src/kernels/quantize_act_parity.cpp:252-270)
    ext = np.zeros(32 * 64, dtype=np.float32)
    ext[0::32] = 1000.0 + (np.arange(64) % 7)
    half = ((np.arange(32 * 64) % 200) - 100 + 0.5).astype(np.float32)
    half[0::32] = 127.0
    for c in (ext, half, np.zeros(128, dtype=np.float32)):
        _, q = q80_fields(oracle.quant_act(Q8_0, c))
        assert np.array_equal(q, q80_gpu_reference(c))


# ------------------------------------------------------------------------------------------------ Q8_0 x Q8_0 rows

def test_q80_row_dot(oracle):
    rng = np.random.default_rng(8)
    k, n = 2048, 24
    w = synth.constructed_rows(Q8_0, n, k, rng)
    codes0 = w.reshape(-1, 34)[:, 2:]
    codes0[codes0 == 0x80] = 0x81            # (-128 has no negation in int8; the negation checks below need one)
    x = rng.standard_normal(k).astype(np.float32)
    act = oracle.quant_act(Q8_0, x)
    got = oracle.rows_of(Q8_0, w, k, n, act)
    # independent: both operands dequantized with numpy from the block layout (f16 d; 32 int8), the product in float64
    wb = w.reshape(n, k // 32, 34)
    wd = wb[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(n, k // 32)
    wq = wb[:, :, 2:].copy().view(np.int8).astype(np.float64)
    ad, aq = q80_fields(act)
    ad = ad.view(np.float16).astype(np.float64)
    aq = aq.reshape(k // 32, 32).astype(np.float64)
    terms = wd[:, :, None] * wq * (ad[None, :, None] * aq[None, :, :])
    want = terms.sum(axis=(1, 2))
    assert np.max(np.abs(got - want) / np.abs(terms).sum(axis=(1, 2))) < 1e-6
    # invariants: the same permutation of both operands' blocks only reorders the float sum; negating the codes of a
    # block in both operands changes nothing at all; negating every weight code negates the result exactly
    perm = rng.permutation(k // 32)
    wp = wb[:, perm, :].reshape(-1)
    ap = act.reshape(k // 32, 34)[perm].reshape(-1)
    gp = oracle.rows_of(Q8_0, wp, k, n, ap)
    assert np.max(np.abs(gp - got) / np.abs(terms).sum(axis=(1, 2))) < 1e-6
    wn = wb.copy()
    an = act.reshape(k // 32, 34).copy()
    blk = 5
    wn[:, blk, 2:] = (-wn[:, blk, 2:].view(np.int8)).view(np.uint8)
    an[blk, 2:] = (-an[blk, 2:].view(np.int8)).view(np.uint8)
    assert np.array_equal(oracle.rows_of(Q8_0, wn.reshape(-1), k, n, an.reshape(-1)), got)
    wneg = wb.copy()
    wneg[:, :, 2:] = (-wb[:, :, 2:].view(np.int8)).view(np.uint8)
    assert np.array_equal(oracle.rows_of(Q8_0, wneg.reshape(-1), k, n, act), -got)


# ------------------------------------------------------------------------------------------------ IQ1_S

def iq1s_all_cases():
    """IQ1_S blocks (ggml-common.h:425-430: f16 d; u8 qs[32]; u16 qh[8]) that together hold every grid index 0..2047 under
    every 3-bit scale and either delta sign: 1024 blocks."""
    nb = 1024
    blocks = np.zeros((nb, 50), dtype=np.uint8)
    rng = np.random.default_rng(10)
    d = rng.uniform(4e-3, 1.2e-2, nb).astype(np.float16)
    d[:8] = np.array([6e-8, 1e-7, 3e-6, 6.1e-5, 1.0, 37.5, 2048.0, 65504.0], dtype=np.float16)   # subnormal .. largest
    blocks[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    qs = np.zeros((nb, 32), dtype=np.uint8)
    qh = np.zeros((nb, 8), dtype=np.uint16)
    sub = 0
    for s in range(8):
        for neg in range(2):
            for base in range(0, 2048, 4):
                b, ib = divmod(sub, 8)
                word = (s << 12) | (neg << 15)
                for il in range(4):
                    idx = base + il
                    qs[b, 4 * ib + il] = idx & 255
                    word |= (idx >> 8) << (3 * il)
                qh[b, ib] = word
                sub += 1
    assert sub == nb * 8
    blocks[:, 2:34] = qs
    blocks[:, 34:50] = qh.view(np.uint8).reshape(nb, 16)
    return blocks


def iq1s_numpy(blocks, grid):
    """Decode written from the layout and dq_iq1_s's formula (src/kernels/cuda/iq_kernels.cu:825-837): grid index = qs |
    (3 bits of qh << 8), scale from qh bits 12-14, delta -1/8 when bit 15 is set else +1/8, w = (d * (2 s + 1)) * (g + delta),
    each product rounded to float32."""
    nb = blocks.shape[0]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(nb)
    qs = blocks[:, 2:34].astype(np.int64).reshape(nb, 8, 4)
    qh = blocks[:, 34:50].copy().view(np.uint16).astype(np.int64).reshape(nb, 8)
    hi = np.stack([(qh >> (3 * il)) & 7 for il in range(4)], axis=2)
    idx = qs | (hi << 8)
    s = (qh >> 12) & 7
    delta = np.where(qh >> 15 != 0, np.float32(-0.125), np.float32(0.125)).astype(np.float32)
    dl = (d[:, None] * (2 * s + 1).astype(np.float32)).astype(np.float32)
    g = grid[idx].astype(np.float32)                                      # [nb, 8, 4, 8] values -1, 0, +1
    return (dl[:, :, None, None] * (g + delta[:, :, None, None]).astype(np.float32)).astype(np.float32).reshape(nb, 256)


def iq1s_to_iq1m(blocks):
    """Every IQ1_S block as the IQ1_M block (ggml-common.h:433-438: u8 qs[32]; u8 qh[16]; u8 scales[8]) that decodes to the
    same values: the sub-block's 3-bit scale written for both of its halves, its delta bit for each of its four groups,
    the FP16 block scale spread over the top nibbles of the four scale words."""
    nb = blocks.shape[0]
    out = np.zeros((nb, 56), dtype=np.uint8)
    out[:, 0:32] = blocks[:, 2:34]
    qh = blocks[:, 34:50].copy().view(np.uint16).astype(np.int64).reshape(nb, 8)
    dbits = blocks[:, 0:2].copy().view(np.uint16).astype(np.int64).reshape(nb)
    qhm = np.zeros((nb, 16), dtype=np.int64)
    sc = np.zeros((nb, 4), dtype=np.int64)
    for ib in range(8):
        s, neg = (qh[:, ib] >> 12) & 7, qh[:, ib] >> 15
        for il in range(4):
            nib = ((qh[:, ib] >> (3 * il)) & 7) | (neg << 3)
            qhm[:, 2 * ib + il // 2] |= nib << (4 * (il % 2))
        for ib16 in (2 * ib, 2 * ib + 1):
            sc[:, ib16 // 4] |= s << (3 * (ib16 % 4))
    for j in range(4):
        sc[:, j] |= ((dbits >> (4 * j)) & 15) << 12
    out[:, 32:48] = qhm.astype(np.uint8)
    out[:, 48:56] = sc.astype(np.uint16).view(np.uint8).reshape(nb, 8)
    return out


@pytest.fixture(scope="module")
def iq1_grid(oracle):
    return np.ctypeslib.as_array(oracle.lib().mo_iq1s_grid(), shape=(2048,)).copy().view(np.int8).reshape(2048, 8)


def test_iq1s_dequant_every_index_scale_and_delta(oracle, iq1_grid):
    blocks = iq1s_all_cases()
    nb = blocks.shape[0]
    got = oracle.dequant_rows(IQ1_S, blocks.reshape(-1), 256 * nb, 1).reshape(nb, 256)
    want = iq1s_numpy(blocks, iq1_grid)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # a decode with a wrong field would not pass: the scale read from bits 11-13, the delta sign flipped, the high index
    # bits taken two at a time
    wrong = blocks.copy()
    q = wrong[:, 34:50].view(np.uint16)
    q ^= 0x8000
    assert not np.array_equal(iq1s_numpy(wrong, iq1_grid), want)
    # random blocks too
    rng = np.random.default_rng(11)
    rb = synth.constructed_rows(IQ1_S, 1, 256 * 300, rng).reshape(300, 50)
    got = oracle.dequant_rows(IQ1_S, rb.reshape(-1), 256 * 300, 1).reshape(300, 256)
    assert np.array_equal(got.view(np.uint32), iq1s_numpy(rb, iq1_grid).view(np.uint32))


def test_iq1s_equals_iq1m_carrying_the_same_block(oracle, iq1_grid):
    """IQ1_M's integer decode and row dot are held bit for bit to the reference build (iq256_rows(29, ...),
    tests/test_oracle_vs_ref.py, tests/test_golden_vectors.py); an IQ1_S block rewritten as IQ1_M must give the same values
    and - up to the order of the float sums - the same row dot."""
    rng = np.random.default_rng(12)
    k, n = 2048, 16
    w = np.concatenate([iq1s_all_cases()[:64], synth.constructed_rows(IQ1_S, n - 8, k, rng).reshape(-1, 50)])
    assert w.shape[0] == n * (k // 256)
    wm = iq1s_to_iq1m(w)
    a = oracle.dequant_rows(IQ1_S, w.reshape(-1), k, n)
    b = oracle.dequant_rows(IQ1_M, wm.reshape(-1), k, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    x = rng.standard_normal(k).astype(np.float32)
    act = oracle.quant_q8k(x)
    ys = oracle.rows_of(IQ1_S, w.reshape(-1), k, n, act)
    ym = oracle.rows_of(IQ1_M, wm.reshape(-1), k, n, act)
    d, q, _ = oracle.q8k_fields(act)
    xa = (np.repeat(d, 256).astype(np.float64) * q.astype(np.float64))
    mag = np.abs(a.astype(np.float64) * xa[None, :]).sum(axis=1)
    assert np.max(np.abs(ys - ym) / mag) < 1e-6
    # and against the float64 dot of the independently decoded weights with the dequantized activation
    want = (iq1s_numpy(w, iq1_grid).reshape(n, k).astype(np.float64) * xa[None, :]).sum(axis=1)
    assert np.max(np.abs(ys - want) / mag) < 1e-6
    # the reference build itself on the carrier blocks, where it exists
    ref = oracle.ref()
    if ref is not None:
        out = np.zeros(n, dtype=np.float32)
        actp = (C.c_void_p * 1)(act.ctypes.data)
        outp = (C.c_void_p * 1)(out.ctypes.data)
        wmc = np.ascontiguousarray(wm.reshape(-1))
        ref.ref_iq256_rows(IQ1_M, wmc.ctypes.data, oracle.row_bytes(IQ1_M, k), k, actp, 1, outp, 0, n)
        assert np.array_equal(out, ym)
        assert np.max(np.abs(ys - out) / mag) < 1e-6


def test_iq1s_row_dot_invariants(oracle, iq1_grid):
    rng = np.random.default_rng(13)
    k, n = 1536, 10
    w = synth.constructed_rows(IQ1_S, n, k, rng).reshape(n, k // 256, 50)
    x = rng.standard_normal(k).astype(np.float32)
    act = oracle.quant_q8k(x)
    got = oracle.rows_of(IQ1_S, w.reshape(-1), k, n, act)
    # the same permutation of the weights' and the activation's 256-value blocks: the float sum's order only
    perm = rng.permutation(k // 256)
    gp = oracle.rows_of(IQ1_S, w[:, perm].reshape(-1), k, n, act.reshape(k // 256, 292)[perm].reshape(-1))
    d, q, _ = oracle.q8k_fields(act)
    xa = np.repeat(d, 256).astype(np.float64) * q.astype(np.float64)
    mag = np.abs(iq1s_numpy(w.reshape(-1, 50), iq1_grid).reshape(n, k).astype(np.float64) * xa[None, :]).sum(axis=1)
    assert np.max(np.abs(gp - got) / mag) < 1e-6
    # a block scale doubled in one block changes the row by exactly that block's share
    w2 = w.copy()
    d16 = w2[:, 2, 0:2].copy().view(np.float16)
    w2[:, 2, 0:2] = (d16 * np.float16(2)).view(np.uint8).reshape(n, 2)
    g2 = oracle.rows_of(IQ1_S, w2.reshape(-1), k, n, act)
    blk = (iq1s_numpy(w[:, 2], iq1_grid).astype(np.float64) * xa[None, 512:768]).sum(axis=1)
    assert np.max(np.abs((g2 - got) - blk) / mag) < 1e-6


# ---------------------------------------------------------------------------------------------------------------- EXL3
# The reference's CPU lane for EXL3 experts (exl3_cpu.cpp, what ds4's CPU flow runs) against the checker's EXL3 mat-vec:
# two independent statements of the same matrix product - the lane keeps weights and rotated input unrounded, the
# checker (exl3_ref.cpp's form, the device's) rounds both to FP16 - so they agree to the roundings: about 3e-4, bar 1e-3.
def _exl3cpu_golden():
    return np.load(os.path.join(HERE, "golden", "refbuild_exl3cpu_vectors.npz"))


def _exl3cpu_case(exl3, row):
    import zlib
    n_embd, n_ff, kg, ku, kd, bseed, xseed = (int(v) for v in row)
    l, nbytes = exl3.make_layout(n_embd, n_ff, [kg, ku, kd], 2)
    blob = exl3.synth_blob(l, nbytes, bseed)
    x = np.random.default_rng(xseed).standard_normal(n_embd).astype(np.float32)
    return l, blob, x, zlib.crc32(x.tobytes(), zlib.crc32(blob.tobytes()))


def _swiglu32(g, u, limit):
    g, u = g.astype(np.float32), u.astype(np.float32)
    if limit > 0:
        g = np.minimum(g, np.float32(limit))
        u = np.clip(u, -np.float32(limit), np.float32(limit))
    return (g / (np.float32(1) + np.exp(-g)) * u).astype(np.float32)


def test_exl3_expert_agrees_with_the_reference_cpu_lane(oracle):
    exl3 = pytest.importorskip("maya_amd.exl3")
    g = _exl3cpu_golden()
    checked = 0
    for i, row in enumerate(g["cases"]):
        if row[0] > 2048:
            continue                      # (the full shape is the GPU test's: seconds of scalar checker here)
        l, blob, x, crc = _exl3cpu_case(exl3, row)
        if crc != int(g["crc_%d" % i]):
            continue                      # another numpy generator: the stored expectations are not for these bytes
        mats = []
        for r in range(3):
            k, n = exl3.matrix_of(l, r)
            tr, suh, svh = exl3.parts_of(l, blob, r)
            mats.append((oracle.exl3_inner(tr, k, n, l.k2[r], 2), suh, svh))
        h = _swiglu32(oracle.exl3_mv(*mats[0], x), oracle.exl3_mv(*mats[1], x), float(g["limits"][i]))
        out = oracle.exl3_mv(*mats[2], h)
        eh = np.linalg.norm(h - g["h_%d" % i]) / np.linalg.norm(g["h_%d" % i])
        eo = np.linalg.norm(out - g["out_%d" % i]) / np.linalg.norm(g["out_%d" % i])
        assert eh <= 1e-3 and eo <= 1e-3, (i, eh, eo)
        assert eh > 1e-6            # not the same arithmetic: the FP16 roundings are there
        checked += 1
    assert checked >= 3


def test_exl3_cpu_lane_live_where_it_was_built(oracle):
    """Where oracle/_ref holds the CPU lane (the build container): fresh random matrices at every bitrate it takes."""
    import ctypes as C
    path = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libmaya_ref_exl3cpu.so")
    if not os.path.exists(path):
        pytest.skip("no reference build of the CPU lane here")
    R = C.CDLL(path)
    R.ref_exl3_cpu_mv.argtypes = [C.c_void_p] * 3 + [C.c_int] * 3 + [C.c_void_p] * 2
    rng = np.random.default_rng(77)
    for k, n, k2 in ((256, 128, 2), (256, 256, 3), (384, 128, 4), (128, 256, 5), (256, 128, 6), (256, 128, 7), (128, 128, 8),
                     (256, 128, 10), (128, 256, 12), (256, 128, 14), (128, 128, 16)):
        words = rng.integers(0, 2 ** 32, (k // 16) * (n // 16) * 4 * k2, dtype=np.uint64).astype(np.uint32)
        suh = (rng.integers(0, 2, k) * 2 - 1).astype(np.float16).view(np.uint16)
        svh = ((rng.integers(0, 2, n) * 2 - 1) * rng.uniform(0.5, 1.5, n)).astype(np.float16).view(np.uint16)
        x = rng.standard_normal(k).astype(np.float32)
        want = np.zeros(n, dtype=np.float32)
        assert R.ref_exl3_cpu_mv(words.ctypes.data, suh.ctypes.data, svh.ctypes.data, k, n, k2, x.ctypes.data, want.ctypes.data) == 0
        got = oracle.exl3_mv(oracle.exl3_inner(words, k, n, k2, 2), suh, svh, x)
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-3, (k, n, k2)
        # a transposed operand, a dropped scale or a wrong rotation is not a rounding: far outside the bar
        assert np.linalg.norm(oracle.exl3_mv(oracle.exl3_inner(words, k, n, k2, 2), suh, svh, x[::-1].copy()) - want) / np.linalg.norm(want) > 0.1

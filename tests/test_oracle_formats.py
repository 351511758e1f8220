"""The CPU checker's format layer against what pins it without the device: exhaustive conversions, the reference build
(oracle/_ref, compiled from the reference's own sources) where it exists, brute force and structural invariants."""
import ctypes as C

import numpy as np
import pytest

import synth


def test_f16_to_f32_exhaustive(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.mo_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_round_trip_and_ties(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    back = np.array([L.mo_f32_to_f16(float(v)) for v in f[ok]], dtype=np.uint16)
    assert np.array_equal(back, bits[ok])
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 300.0, 7e4)])
    # exact ties between neighbouring halves, and one float ulp either side of them
    h = rng.integers(0, 0x7bff, size=4000).astype(np.uint16)
    lo, hi = h.view(np.float16).astype(np.float64), (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid])
    want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.mo_f32_to_f16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(5000) * 10).astype(np.float32)
    import torch
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.mo_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    back = np.array([L.mo_bf16_to_f32(int(b)) for b in got], dtype=np.float32)
    assert np.array_equal(back.view(np.uint32), got.astype(np.uint32) << 16)


def test_codebooks(oracle):
    L = oracle.lib()
    g2 = np.ctypeslib.as_array(L.mo_iq2s_grid(), shape=(1024,)).copy()
    g1 = np.ctypeslib.as_array(L.mo_iq1s_grid(), shape=(2048,)).copy()
    assert set(np.unique(g2.view(np.uint8))) == {8, 25, 43}
    assert set(np.unique(g1.view(np.int8))) == {-1, 0, 1}
    assert len(np.unique(g2)) == 1024 and len(np.unique(g1)) == 2048
    # the first / last entries as the format definition prints them (ggml-common.h:759, 1136)
    assert g2[0] == 0x0808080808080808 and g2[1] == 0x080808080808082B
    assert g1[0] == 0xFFFFFFFFFFFFFFFF and g1[1] == 0xFFFFFFFFFFFFFF01
    assert L.mo_crc32(g2.ctypes.data, g2.nbytes) == 0x25AE5BF1
    assert L.mo_crc32(g1.ctypes.data, g1.nbytes) == 0xB85E6CCF
    gx = np.ctypeslib.as_array(L.mo_iq2xxs_grid(), shape=(256,)).copy()
    assert set(np.unique(gx.view(np.uint8))) == {8, 25, 43} and len(np.unique(gx)) == 256
    assert gx[0] == 0x0808080808080808 and gx[1] == 0x080808080808082B   # (ggml-common.h:561)
    assert L.mo_crc32(gx.ctypes.data, gx.nbytes) == 0x9924FF02


def test_codebooks_against_reference_tree(oracle):
    import os
    import re
    path = "/root/reference/third_party/ggml/ggml-common.h"
    if not os.path.exists(path):
        pytest.skip("no reference tree here")
    src = open(path).read()
    L = oracle.lib()
    for decl, fn, n in (("GGML_TABLE_BEGIN(uint64_t, iq2s_grid, 1024)", L.mo_iq2s_grid, 1024),
                        ("GGML_TABLE_BEGIN(uint64_t, iq1s_grid, NGRID_IQ1S)", L.mo_iq1s_grid, 2048),
                        ("GGML_TABLE_BEGIN(uint64_t, iq2xxs_grid, 256)", L.mo_iq2xxs_grid, 256)):
        m = re.search(re.escape(decl) + r"(.*?)GGML_TABLE_END", src, re.S)
        want = np.array([int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", m.group(1))], dtype=np.uint64)
        got = np.ctypeslib.as_array(fn(), shape=(n,))
        assert np.array_equal(got, want)


def test_geometry(oracle):
    L = oracle.lib()
    for t, bb in synth.BLOCK_BYTES.items():
        assert L.mo_block_bytes(t) == bb and L.mo_block_values(t) == synth.BLOCK_VALUES[t]
    # the row sizes the configs name
    assert oracle.row_bytes(12, 7168) == 4032 and oracle.row_bytes(12, 2048) == 1152
    assert oracle.row_bytes(22, 7168) == 2296 and oracle.row_bytes(22, 2048) == 656
    assert oracle.row_bytes(8, 7168) == 7616 and oracle.row_bytes(8, 2048) == 2176
    assert synth.blob_offsets(22, 22, 7168, 2048)[2] == 14106624
    assert synth.blob_offsets(12, 12, 7168, 2048)[2] == 24772608
    assert synth.blob_offsets(22, 12, 7168, 2048)[2] == 17661952
    assert synth.blob_offsets(8, 8, 7168, 2048)[2] == 46792704


def test_q8_0_dequant_closed_form(oracle):
    rng = np.random.default_rng(11)
    w = synth.constructed_rows(8, 4, 256, rng)
    got = oracle.dequant_rows(8, w, 256, 4).reshape(-1, 32)
    b = w.reshape(-1, 34)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32)
    q = b[:, 2:].copy().view(np.int8).astype(np.float32)
    assert np.array_equal(got, q * d)


def test_q4_k_dequant_brute_force(oracle):
    """Every (6-bit scale, 6-bit min) pair in every sub-block position, every nibble value: w = (d*sc)*q - (dmin*m),
    each operation rounded once, decoded by an independent numpy restatement of the packing."""
    rng = np.random.default_rng(5)
    nb = 64 * 64 // 8
    blocks = np.zeros((nb, 144), dtype=np.uint8)
    pairs = [(s, m) for s in range(64) for m in range(64)]
    rng.shuffle(pairs)
    d = rng.uniform(1e-4, 1e-2, nb).astype(np.float16)
    dm = rng.uniform(1e-4, 1e-2, nb).astype(np.float16)
    blocks[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    blocks[:, 2:4] = dm.view(np.uint8).reshape(nb, 2)
    blocks[:, 16:] = rng.integers(0, 256, size=(nb, 128), dtype=np.uint8)
    sc = np.zeros((nb, 8), dtype=np.int64)
    mn = np.zeros((nb, 8), dtype=np.int64)
    for b in range(nb):
        for j in range(8):
            sc[b, j], mn[b, j] = pairs[b * 8 + j]
    s = np.zeros((nb, 12), dtype=np.int64)
    for j in range(4):
        s[:, j] |= sc[:, j]
        s[:, j + 4] |= mn[:, j]
    for j in range(4, 8):
        s[:, j + 4] |= (sc[:, j] & 15) | ((mn[:, j] & 15) << 4)
        s[:, j - 4] |= (sc[:, j] >> 4) << 6
        s[:, j] |= (mn[:, j] >> 4) << 6
    blocks[:, 4:16] = s.astype(np.uint8)
    got = oracle.dequant_rows(12, blocks.reshape(-1), 256 * nb, 1).reshape(nb, 8, 32)
    qs = blocks[:, 16:].reshape(nb, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(nb, 8, 32).astype(np.float32)
    d32, dm32 = d.astype(np.float32), dm.astype(np.float32)
    d1 = (d32[:, None] * sc.astype(np.float32)).astype(np.float32)
    m1 = (dm32[:, None] * mn.astype(np.float32)).astype(np.float32)
    want = ((d1[:, :, None] * q).astype(np.float32) - m1[:, :, None]).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4_k_q8_0_dequant_against_reference_build(oracle, refbuild):
    rng = np.random.default_rng(21)
    w = synth.constructed_rows(12, 8, 1024, rng)
    got = oracle.dequant_rows(12, w, 1024, 8).reshape(-1, 256)
    blocks = w.reshape(-1, 144)
    out = np.zeros(256, dtype=np.float32)
    mism = 0
    for b in range(blocks.shape[0]):
        blk = np.ascontiguousarray(blocks[b])
        refbuild.ref_dequant_q4_K(blk.ctypes.data, out.ctypes.data)
        # the reference writes d1*q - m1 as one expression: its compiler may or may not fuse it; this build's canonical
        # form is unfused, and the reference build here is compiled -ffp-contract=off, so they agree to the bit
        mism += int(np.count_nonzero(out.view(np.uint32) != got[b].view(np.uint32)))
    assert mism == 0
    w8 = synth.constructed_rows(8, 4, 512, rng)
    got8 = oracle.dequant_rows(8, w8, 512, 4).reshape(-1, 32)
    o32 = np.zeros(32, dtype=np.float32)
    for b, blk in enumerate(w8.reshape(-1, 34)):
        blk = np.ascontiguousarray(blk)
        refbuild.ref_dequant_q8_0(blk.ctypes.data, o32.ctypes.data)
        assert np.array_equal(o32.view(np.uint32), got8[b].view(np.uint32))


def test_iq2_s_dequant_structure(oracle):
    """|w| = d * (2 ls + 1) / 8 * g with g in {8, 25, 43}; sign bit j of the group's sign byte; exhaustively over the
    scale nibbles and over a sample of (index, sign byte) pairs that covers all 1024 indices and all 256 sign bytes."""
    rng = np.random.default_rng(2)
    nb = 512
    w = synth.constructed_rows(22, 1, 256 * nb, rng).reshape(nb, 82)
    # force coverage: block b, group g takes index (32 b + g) % 1024 and sign byte (32 b + g) % 256
    idx = (np.arange(nb)[:, None] * 32 + np.arange(32)[None, :]) % 1024
    w[:, 2:34] = (idx & 255).astype(np.uint8)
    qh = np.zeros((nb, 8), dtype=np.uint8)
    for il in range(4):
        qh |= (((idx.reshape(nb, 8, 4)[:, :, il] >> 8) & 3) << (2 * il)).astype(np.uint8)
    w[:, 66:74] = qh
    w[:, 34:66] = ((np.arange(nb)[:, None] * 32 + np.arange(32)[None, :] * 7) % 256).astype(np.uint8)
    got = oracle.dequant_rows(22, w.reshape(-1), 256 * nb, 1).reshape(nb, 32, 8)
    grid = np.ctypeslib.as_array(oracle.lib().mo_iq2s_grid(), shape=(1024,)).view(np.uint8).reshape(1024, 8)
    d = w[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(nb)
    sc = w[:, 74:82]
    ls = np.stack([sc & 15, sc & 15, sc >> 4, sc >> 4], axis=2).reshape(nb, 32).astype(np.float32)
    dl = ((d[:, None] * (np.float32(0.5) + ls)).astype(np.float32) * np.float32(0.25)).astype(np.float32)
    mag = grid[idx].astype(np.float32)
    sign = 1.0 - 2.0 * ((w[:, 34:66][:, :, None] >> np.arange(8)[None, None, :]) & 1).astype(np.float32)
    want = (dl[:, :, None] * mag).astype(np.float32) * sign
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
    # the alternative association the exact kernels use: (d/8) * (2 ls + 1): the same float outside the subnormals
    alt = ((d[:, None] * np.float32(0.125)) * (2 * ls + 1)).astype(np.float32)
    assert np.array_equal(alt, dl)


def test_iq2_xxs_dequant_structure(oracle):
    """IQ2_XXS from the format's definition (ggml-common.h:380-384: d, then per 32 values four index bytes and one word of
    four 7-bit sign indices and a 4-bit scale): |w| = d * (0.5 + s) * 0.25 * g, sign bit j of the sign index, bit 7 the
    parity of the other seven.  Every codebook index, every sign index and every scale occurs."""
    rng = np.random.default_rng(16)
    nb = 256
    w = synth.constructed_rows(16, 1, 256 * nb, rng).reshape(nb, 66)
    q = w[:, 2:66].reshape(nb, 8, 8)
    idx = (np.arange(nb)[:, None, None] + 32 * np.arange(8)[None, :, None] + 7 * np.arange(4)[None, None, :]) % 256
    sgn = (np.arange(nb)[:, None, None] * 5 + 16 * np.arange(8)[None, :, None] + 37 * np.arange(4)[None, None, :]) % 128
    scl = (np.arange(nb)[:, None] + np.arange(8)[None, :]) % 16
    q[:, :, 0:4] = idx.astype(np.uint8)
    aux = (sgn[:, :, 0] | (sgn[:, :, 1] << 7) | (sgn[:, :, 2] << 14) | (sgn[:, :, 3] << 21) | (scl << 28)).astype(np.uint32)
    q[:, :, 4:8] = aux[:, :, None].view(np.uint8).reshape(nb, 8, 4)
    assert len(np.unique(idx)) == 256 and len(np.unique(sgn)) == 128
    got = oracle.dequant_rows(16, w.reshape(-1), 256 * nb, 1).reshape(nb, 8, 4, 8)
    grid = np.ctypeslib.as_array(oracle.lib().mo_iq2xxs_grid(), shape=(256,)).view(np.uint8).reshape(256, 8)
    d = w[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(nb)
    db = ((d[:, None] * (np.float32(0.5) + scl.astype(np.float32))).astype(np.float32) * np.float32(0.25)).astype(np.float32)
    parity = np.zeros_like(sgn)
    for j in range(7):
        parity ^= (sgn >> j) & 1
    s8 = sgn | (parity << 7)
    sign = 1.0 - 2.0 * ((s8[..., None] >> np.arange(8)) & 1).astype(np.float32)
    want = (db[:, :, None, None] * grid[idx].astype(np.float32)).astype(np.float32) * sign
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
    # an even number of negative values in every group of 8
    assert np.all(np.count_nonzero(got < 0, axis=3) % 2 == 0)


def test_iq1_dequant_structure(oracle):
    rng = np.random.default_rng(9)
    for t in (19, 29):
        nb = 64
        w = synth.constructed_rows(t, 1, 256 * nb, rng)
        got = oracle.dequant_rows(t, w, 256 * nb, 1).reshape(nb, 16, 16)
        blocks = w.reshape(nb, synth.BLOCK_BYTES[t])
        if t == 19:
            d = blocks[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(nb)
        else:
            sc = blocks[:, 48:56].copy().view(np.uint16).reshape(nb, 4)
            bits = ((sc[:, 0] >> 12) | ((sc[:, 1] >> 8) & 0xF0) | ((sc[:, 2] >> 4) & 0xF00) | (sc[:, 3] & 0xF000))
            d = bits.astype(np.uint16).view(np.float16).astype(np.float64)
        # every value / d is (2s+1) * (g +- 1/8), g in {-1, 0, 1}, s in 0..7: 8 w / d is an odd multiple of (2s+1)
        r = got.astype(np.float64) / d[:, None, None] * 8.0
        assert np.allclose(r, np.round(r), atol=1e-3)
        r = np.round(r).astype(np.int64)
        for b in range(nb):
            for g in range(16):
                vals = set(np.abs(r[b, g]).tolist())
                ok = False
                for s in range(8):
                    m = 2 * s + 1
                    if vals <= {7 * m, 9 * m, m}:
                        ok = True
                assert ok, (t, b, g, vals)


def test_float_and_double_selection_agree(oracle):
    # the kernel selects on float p, the reference's host test on double p: no disagreement on N(0,1) logits
    rng = np.random.default_rng(8)
    logits = rng.standard_normal((2000, 256)).astype(np.float32)
    a, _ = oracle.router_topk(logits, 8)
    b, _ = oracle.router_topk(logits, 8, f64=True)
    assert np.array_equal(a, b)


def test_softmax_router_against_an_independent_statement(oracle):
    """The softmax router's ids and weights against numpy: softmax in double, the k largest by a stable descending sort
    (the lower index wins a tie), the chosen probabilities renormalised by max(sum, 2^-14) - the reference's host form
    (src/kernels/router_top10_parity.cpp:36-60).  Random rows, rows of quantised logits (many exact ties), all-equal rows."""
    rng = np.random.default_rng(81)
    k, ne = 8, 256
    rows = [rng.standard_normal((400, ne)), np.round(rng.standard_normal((150, ne)) * 2.0) / 2.0, np.zeros((3, ne)),
            np.full((2, ne), -3.25)]
    logits = np.concatenate(rows).astype(np.float32)
    ids, w = oracle.router_topk(logits, k)
    for t in range(logits.shape[0]):
        x = logits[t].astype(np.float64)
        p = np.exp(x - x.max())
        p /= p.sum()
        pf = p.astype(np.float32)   # (the device selects on the probabilities rounded to float: ties there go to the lower index too)
        order = np.argsort(-pf, kind="stable")[:k]
        assert np.array_equal(ids[t], order), t
        want = p[order] / max(p[order].sum(), 2.0 ** -14)
        assert np.max(np.abs(w[t] - want) / want) < 1e-5, t
    # closed forms: all-equal logits -> ids 0 .. k-1, every weight 1 / k
    assert np.array_equal(ids[-1], np.arange(k)) and np.allclose(w[-1], 1.0 / k, rtol=1e-6)
    # a wrong reading must differ: no renormalisation leaves the weights' sum below 1
    assert abs(float(w[0].sum()) - 1.0) < 1e-5


def test_combine_is_the_slot_order_rounded_sum(oracle):
    """mo_combine against its statement (src/kernels/cuda/native_moe.cu:36-52): sum = parts[0] * w[0]; sum += parts[i] * w[i]
    in slot order, every product and every sum rounded to float - bit for bit; a reversed order or a fused multiply-add
    gives different bits on random data."""
    rng = np.random.default_rng(82)
    parts = rng.standard_normal((8, 4096)).astype(np.float32)
    w = rng.random(8).astype(np.float32)
    got = oracle.combine(parts, w)
    want = (parts[0] * w[0]).astype(np.float32)
    for i in range(1, 8):
        want = (want + (parts[i] * w[i]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    rev = (parts[7] * w[7]).astype(np.float32)
    for i in range(6, -1, -1):
        rev = (rev + (parts[i] * w[i]).astype(np.float32)).astype(np.float32)
    assert not np.array_equal(rev.view(np.uint32), want.view(np.uint32))
    fused = (parts[0].astype(np.float64) * w[0]).astype(np.float32)
    for i in range(1, 8):
        fused = (fused.astype(np.float64) + parts[i].astype(np.float64) * float(w[i])).astype(np.float32)
    assert not np.array_equal(fused.view(np.uint32), want.view(np.uint32))
    # one slot: the product alone
    assert np.array_equal(oracle.combine(parts[:1], w[:1]).view(np.uint32), (parts[0] * w[0]).astype(np.float32).view(np.uint32))


# ---- the sigmoid router: the device arithmetic against the reference's host form (router_sigmoid_parity.cpp:36-86) restated
# here in double with a stable sort, on that test's own case shapes, to its bars (ids equal, weights 1e-5; :137-143)

def _ref_router_sigmoid(logits, bias, k, w_scale, norm_w, softmax=False, biased_weights=False, no_renorm=False, no_scale=False):
    nt, ne = logits.shape
    ids = np.zeros((nt, k), dtype=np.int32)
    w = np.zeros((nt, k), dtype=np.float32)
    for t in range(nt):
        x = logits[t].astype(np.float64)
        if softmax:
            p = np.exp(x - x.max())
            p /= p.sum()
        else:
            p = 1.0 / (1.0 + np.exp(-x))
        score = p + (bias.astype(np.float64) if bias is not None else 0.0)
        order = np.argsort(-score, kind="stable")[:k]
        ids[t] = order
        wf = p[order].astype(np.float32)
        s = p[order].sum()
        for i in range(k):
            v = float(wf[i]) + (float(bias[order[i]]) if (biased_weights and bias is not None) else 0.0)
            if norm_w and not no_renorm:
                v /= max(s, 6.103515625e-5)
            if not no_scale:
                v *= w_scale
            w[t, i] = np.float32(v)
    return ids, w


SIGMOID_CASES = [(4, 32, 8, 2.5, True, True, False, 11), (1, 288, 8, 2.5, True, True, False, 12),
                 (4, 32, 8, 2.5, True, True, True, 13), (4, 32, 8, 1.0, False, False, False, 14),
                 (16, 256, 8, 2.5, True, True, False, 15), (3, 384, 6, 1.0, True, True, True, 16)]


def sigmoid_case(nt, ne, with_bias, quantize, seed):
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((nt, ne)) * 2.0).astype(np.float32)
    bias = (rng.standard_normal(ne) * 0.1).astype(np.float32) if with_bias else None
    if quantize:   # exact selection-score ties on purpose
        logits = (np.round(logits * 4) / 4).astype(np.float32)
        if bias is not None:
            bias = (np.round(bias * 4) / 4).astype(np.float32)
    return logits, bias


@pytest.mark.parametrize("nt,ne,k,w_scale,norm_w,with_bias,quantize,seed", SIGMOID_CASES)
def test_sigmoid_router_against_the_reference_host_form(oracle, nt, ne, k, w_scale, norm_w, with_bias, quantize, seed):
    logits, bias = sigmoid_case(nt, ne, with_bias, quantize, seed)
    ids, w = oracle.router_sigmoid(logits, bias, k, w_scale, 1 if norm_w else 0)
    rid, rw = _ref_router_sigmoid(logits, bias, k, w_scale, norm_w)
    assert np.array_equal(ids, rid)
    assert np.max(np.abs(w - rw)) < 1e-5
    i64, w64 = oracle.router_sigmoid(logits, bias, k, w_scale, 1 if norm_w else 0, f64=True)
    assert np.array_equal(i64, rid) and np.max(np.abs(w64 - rw)) < 1e-6
    # the wrong readings the reference names must differ materially (:147-160)
    if with_bias and not quantize:
        assert np.max(np.abs(w - _ref_router_sigmoid(logits, bias, k, w_scale, norm_w, biased_weights=True)[1])) > 1e-3
    assert np.max(np.abs(w - _ref_router_sigmoid(logits, bias, k, w_scale, norm_w, softmax=True)[1])) > 1e-2
    if norm_w:
        assert np.max(np.abs(w - _ref_router_sigmoid(logits, bias, k, w_scale, norm_w, no_renorm=True)[1])) > 1e-2
    if w_scale != 1.0:
        assert np.max(np.abs(w - _ref_router_sigmoid(logits, bias, k, w_scale, norm_w, no_scale=True)[1])) > 1e-2


def test_sigmoid_router_closed_forms(oracle):
    ne, k = 64, 8
    logits = np.full((2, ne), 0.3, dtype=np.float32)
    ids, w = oracle.router_sigmoid(logits, None, k, 2.5, 1)
    assert np.array_equal(ids, np.tile(np.arange(k, dtype=np.int32), (2, 1)))          # a pure tie: the lower indices
    assert np.allclose(w, 2.5 / k, rtol=1e-6)
    # the bias selects but does not weigh: expert 40 has the smallest p and a large bias
    logits = np.linspace(1.0, 2.0, ne, dtype=np.float32)[None, :].copy()
    logits[0, 40] = -6.0
    bias = np.zeros(ne, dtype=np.float32)
    bias[40] = 5.0
    ids, w = oracle.router_sigmoid(logits, bias, k, 1.0, 0)
    assert ids[0, 0] == 40 and abs(w[0, 0] - 1.0 / (1.0 + np.exp(6.0))) < 1e-7
    assert np.array_equal(ids[0, 1:], np.arange(ne - 1, ne - k, -1))
    ids, w = oracle.router_sigmoid(logits, bias, k, 2.5, 1)
    assert abs(float(w.sum()) - 2.5) < 1e-5                                              # normalised, then scaled
    # all sigmoids tiny: the two normalisations part (max(sum, 2^-14) against sum + 1e-20)
    logits = np.full((1, ne), -30.0, dtype=np.float32)
    _, w1 = oracle.router_sigmoid(logits, None, k, 1.0, 1)
    _, w2 = oracle.router_sigmoid(logits, None, k, 1.0, 2)
    p = 1.0 / (1.0 + np.exp(30.0))
    assert np.allclose(w1, p / 6.103515625e-5, rtol=1e-5) and np.allclose(w2, 1.0 / k, rtol=1e-5)


def non_finite_rows(ne, seed):
    """Five rows: 0 and 4 ordinary, 1 with a NaN logit, 2 with +Inf, 3 with -Inf (its sigmoid is a finite 0)."""
    logits = (np.random.default_rng(seed).standard_normal((5, ne)) * 2).astype(np.float32)
    logits[1, ne // 3] = np.nan
    logits[2, ne - 1] = np.inf
    logits[3, 0] = -np.inf
    return logits


@pytest.mark.parametrize("ne", (64, 300))
def test_sigmoid_router_refuses_non_finite_rows(oracle, ne):
    """The engine's routers give a row with a non-finite logit or score no routes: ids -1, weights 0
    (src/kernels/cuda/glm_batch.cu:2077-2092, tests/hip/glm_handoff.cpp:186-207); the other rows are not touched."""
    k = 8
    logits = non_finite_rows(ne, 5)
    bias = (np.random.default_rng(6).standard_normal(ne) * 0.1).astype(np.float32)
    for f64 in (False, True):
        ids, w = oracle.router_sigmoid(logits, bias, k, 2.5, 1, f64=f64)
        good = [0, 4]
        gi, gw = oracle.router_sigmoid(logits[good], bias, k, 2.5, 1, f64=f64)
        assert np.array_equal(ids[good], gi) and np.array_equal(w[good], gw) and gi.min() >= 0
        assert np.all(ids[1:4] == -1) and np.all(w[1:4] == 0.0)
    # a bias that makes one score infinite refuses every row
    bias[5] = np.inf
    ids, w = oracle.router_sigmoid(logits, bias, k, 1.0, 2)
    assert np.all(ids == -1) and np.all(w == 0.0)


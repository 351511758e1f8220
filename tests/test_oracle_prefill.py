"""The CPU checker's prompt-chunk pieces against what the mathematics fixes: the grouped product against an
independent float64 numpy product of the dequantized operands, the plan against a brute-force scan, the per-32
quantizer's invariants and the Q4_K encoder's round trip."""
import numpy as np

Q4_K, Q8_0 = 12, 8


def test_grouped_ref_equals_numpy_product(oracle):
    import synth
    rng = np.random.default_rng(3)
    k, n, ne = 512, 24, 3
    mats = [synth.constructed_rows(Q4_K, n, k, rng) for _ in range(ne)]
    bounds = np.array([0, 5, 5, 12], dtype=np.int32)         # expert 1 has no rows
    x = rng.standard_normal((12, k)).astype(np.float32)
    xq = np.zeros((12, k), dtype=np.int8)
    xd = np.zeros((12, k // 32), dtype=np.float32)
    for r in range(12):
        xq[r], xd[r] = oracle.quant_i8x32(x[r])
    got = oracle.grouped_ref(Q4_K, [mats[0], None, mats[2]], bounds, k, n, xq, xd)
    xdq = xq.astype(np.float64) * np.repeat(xd.astype(np.float64), 32, axis=1)
    for e in (0, 2):
        w = oracle.dequant_rows(Q4_K, mats[e], k, n).astype(np.float64)
        want = xdq[bounds[e]:bounds[e + 1]] @ w.T
        assert np.allclose(got[bounds[e]:bounds[e + 1]], want, rtol=1e-6, atol=1e-6 * np.abs(want).max())
    # linear in the activation scale, and a transposed operand would not survive unequal k and n
    got2 = oracle.grouped_ref(Q4_K, [mats[0], None, mats[2]], bounds, k, n, xq, 2.0 * xd)
    assert np.allclose(got2, 2.0 * got, rtol=1e-6)


def test_plan_is_the_stable_sort(oracle):
    rng = np.random.default_rng(8)
    ids = rng.integers(-1, 7, (40, 3)).astype(np.int32)       # -1 and 6 are out of range for 6 experts
    resident = np.array([1, 1, 0, 1, 1, 1], dtype=bool)
    bounds, row_entry, entry_row = oracle.prefill_plan(ids, 6, resident)
    flat = ids.reshape(-1)
    rows = []
    for e in range(6):
        assert bounds[e] == len(rows)
        if resident[e]:
            rows += [i for i in range(flat.size) if flat[i] == e]      # brute force, in entry order
    assert bounds[6] == len(rows) and np.array_equal(row_entry, rows)
    for i in range(flat.size):
        assert (entry_row[i] == -1) == (i not in rows)
        if entry_row[i] >= 0:
            assert row_entry[entry_row[i]] == i


def test_i8x32_invariants(oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(256) * np.repeat(rng.uniform(1e-3, 50, 8), 32)).astype(np.float32)
    x[64:96] = 0.0
    q, d = oracle.quant_i8x32(x)
    for b in range(8):
        xb, qb = x[32 * b:32 * b + 32], q[32 * b:32 * b + 32].astype(np.int32)
        am = np.abs(xb).max()
        assert d[b] == np.float32(am / np.float32(127.0))
        if am == 0:
            assert not qb.any()
            continue
        assert np.abs(qb).max() == 127 and qb[np.argmax(np.abs(xb))] == 127 * np.sign(xb[np.argmax(np.abs(xb))])
        assert np.abs(qb * np.float64(d[b]) - xb).max() <= 0.5 * d[b] * (1 + 1e-5)
    # exact halves round to even
    xb = np.zeros(32, dtype=np.float32)
    xb[0], xb[1], xb[2], xb[3] = 127.0, 0.5, 1.5, -2.5
    q, d = oracle.quant_i8x32(xb)
    assert d[0] == 1.0 and list(q[:4]) == [127, 0, 2, -2]


def test_q4k_encoder_round_trip(oracle):
    rng = np.random.default_rng(6)
    w = (rng.standard_normal(4096) * 0.02).astype(np.float32)
    blob = oracle.encode_q4k(w)
    assert blob.size == 16 * 144
    back = oracle.dequant_rows(Q4_K, blob, 4096, 1)[0]
    err = np.abs(back - w).reshape(-1, 32)
    span = (w.reshape(-1, 32).max(axis=1) - np.minimum(w.reshape(-1, 32).min(axis=1), 0))
    assert np.all(err.max(axis=1) <= span / 15 * 0.75 + 1e-4)   # within about a step of the 4-bit grid of each sub-block
    assert np.sqrt(np.mean((back - w) ** 2)) / w.std() < 0.08

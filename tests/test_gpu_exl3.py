"""EXL3 experts on the GPU through the C ABI: the decoded W' bit for bit against exllamav3's own vectors and the CPU
checker, then gate/up, down and whole layers against the checker's mat-vec (FP16-rounded rotated input, FP32 sums) at
1e-3 relative L2: the sums run in a different order, the weights and rotations are the same bits."""
import glob
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from gpu_util import HostExpert, host_layer, swiglu, rel_l2  # noqa: E402
from test_oracle_exl3 import read_exh1, FILES  # noqa: E402

TOL = 1e-3


@pytest.fixture(scope="module")
def ex():
    from maya_amd import exl3
    exl3.load()
    return exl3


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
def test_inner_matches_exllamav3(ex, path):
    f = read_exh1(path)
    words = np.ascontiguousarray(f["trellis"]).view(np.uint32).reshape(-1)
    k, n = 16 * f["ki"], 16 * f["nj"]
    w = ex.reconstruct_inner(torch.from_numpy(words.copy()).cuda(), k, n, f["k2"], f["cb"])
    torch.cuda.synchronize()
    assert np.array_equal(w.cpu().numpy().view(np.uint16), f["w_hat"])


@pytest.mark.parametrize("k2,cb", [(2, 0), (4, 1), (6, 2), (8, 0), (16, 1), (3, 2), (5, 2), (7, 2)])
def test_inner_matches_checker_on_random_bits(ex, oracle, k2, cb):
    rng = np.random.default_rng(100 + k2 * 3 + cb)
    k, n = 64, 48
    words = rng.integers(0, 2 ** 32, (k // 16) * (n // 16) * 4 * k2, dtype=np.uint64).astype(np.uint32)
    want = oracle.exl3_inner(words, k, n, k2, cb).astype(np.float16)
    got = ex.reconstruct_inner(torch.from_numpy(words).cuda(), k, n, k2, cb)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_unsupported_k2_is_refused(ex):
    from maya_amd.lib import MayaError
    assert ex.supported(6, 2) and ex.supported(3, 2) and not ex.supported(3, 0) and not ex.supported(18, 2)
    with pytest.raises(MayaError):
        ex.reconstruct_inner(torch.zeros(64, dtype=torch.int32, device="cuda"), 16, 16, 9, 0)


CASES = [
    # n_embd, n_ff, k2 (gate, up, down), cb, n_expert, k, n_tokens, limit
    (256, 128, 4, 2, 6, 2, 1, 0.0),
    (512, 256, (6, 6, 8), 2, 8, 4, 1, 7.0),
    (384, 256, (2, 4, 6), 0, 8, 3, 3, 0.0),
    (256, 384, (8, 8, 4), 1, 5, 2, 5, 2.0),
    (512, 128, (3, 5, 7), 2, 6, 3, 4, 0.0),
    (4096, 2048, 6, 2, 8, 8, 1, 7.0),
    (1024, 512, 4, 2, 4, 4, 8, 0.0),
    (6144, 1536, 6, 2, 10, 8, 4, 0.0),      # the EXL3 configuration's expert shape and window
    (2048, 512, (4, 4, 16), 2, 5, 3, 2, 0.0),   # split gate/up with a general-walk down (16 bits a step)
]


@pytest.mark.parametrize("case", CASES, ids=[str(c[:4]) + "x%dt" % c[6] for c in CASES])
def test_layer_matches_checker(ex, oracle, case):
    n_embd, n_ff, k2, cb, n_expert, k, nt, limit = case
    l, nbytes = ex.make_layout(n_embd, n_ff, k2, cb)
    blobs = [ex.synth_blob(l, nbytes, 1000 + e) for e in range(n_expert)]
    from maya_amd import lib
    store = lib.ExpertStore(blobs)
    rng = np.random.default_rng(n_embd + nt)
    logits = rng.standard_normal((nt, n_expert)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    add = rng.standard_normal((nt, n_embd)).astype(np.float32)
    layer = ex.Exl3Layer(l, n_expert, k, max_tokens=nt)
    out = layer.forward(store.table, torch.from_numpy(logits).cuda(), torch.from_numpy(x).cuda(), limit=limit,
                        add=torch.from_numpy(add).cuda())
    torch.cuda.synchronize()
    ids, w = oracle.router_topk(logits, k)
    assert np.array_equal(layer.ids[:nt].cpu().numpy(), ids)
    experts = [HostExpert(ex, oracle, l, b) for b in blobs]
    want, _ = host_layer(oracle, experts, ids, w, x, limit)
    want = want + add
    got = out.cpu().numpy()
    for t in range(nt):
        assert rel_l2(got[t], want[t]) <= TOL, (t, rel_l2(got[t], want[t]))


def test_stages_null_slots_and_window_equals_single_token(ex, oracle):
    """gate/up and down called separately: h against the checker, a plan with empty slots, and a window's grouped pass
    giving each token what the token alone gets."""
    from maya_amd import lib
    n_embd, n_ff, k, nt, n_expert = 512, 256, 3, 4, 5
    l, nbytes = ex.make_layout(n_embd, n_ff, (4, 6, 4), 2)
    blobs = [ex.synth_blob(l, nbytes, 77 + e) for e in range(n_expert)]
    store = lib.ExpertStore(blobs)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    ids = np.stack([rng.permutation(n_expert)[:k] for _ in range(nt)]).astype(np.int32)
    w = rng.uniform(0.1, 1.0, (nt, k)).astype(np.float32)
    table = store.table.clone()
    table[2] = 0                                   # expert 2 is not resident: its slots are skipped
    ids_d = torch.from_numpy(ids).cuda()
    plan = lib.plan(ids_d.reshape(-1), table)
    w_d = torch.from_numpy(w).cuda()
    x_d = torch.from_numpy(x).cuda()
    experts = [HostExpert(ex, oracle, l, b) for b in blobs]
    want, want_h = host_layer(oracle, experts, ids, w, x, 0.0, skip=(2,))

    def run(groups, n_tok, sl):
        h = torch.zeros((n_tok * k, n_ff), dtype=torch.float32, device="cuda")
        part = torch.zeros((n_tok * k, n_embd), dtype=torch.float32, device="cuda")
        out = torch.zeros((n_tok, n_embd), dtype=torch.float32, device="cuda")
        a = ex.make_args(l, n_tok, k, plan[sl.start * k:sl.stop * k], w_d[sl], x_d[sl], h, part, out, groups=groups)
        ex.gate_up(a)
        ex.down(a)
        torch.cuda.synchronize()
        return h.cpu().numpy(), out.cpu().numpy()

    groups = lib.group(plan)
    h_win, out_win = run(groups, nt, slice(0, nt))
    for e in range(nt * k):
        if ids.reshape(-1)[e] == 2:
            assert not h_win[e].any()
        else:
            assert rel_l2(h_win[e], want_h[e]) <= TOL
    for t in range(nt):
        assert rel_l2(out_win[t], want[t]) <= TOL
        h1, out1 = run(None, 1, slice(t, t + 1))
        assert np.array_equal(out1[0], out_win[t])          # the same sums in the same order: the same bits
        assert np.array_equal(h1, h_win[t * k:(t + 1) * k])


def test_skip_flag_and_bad_shapes(ex):
    from maya_amd import lib
    l, nbytes = ex.make_layout(256, 128, 4, 2)
    store = lib.ExpertStore([ex.synth_blob(l, nbytes, 5)])
    plan = store.table.clone()
    w = torch.ones(1, device="cuda")
    x = torch.ones((1, 256), device="cuda")
    h = torch.full((1, 128), 3.0, device="cuda")
    part = torch.zeros((1, 256), device="cuda")
    out = torch.full((1, 256), 5.0, device="cuda")
    skip = torch.ones(1, dtype=torch.int32, device="cuda")
    a = ex.make_args(l, 1, 1, plan, w, x, h, part, out, skip=skip)
    ex.gate_up(a)
    ex.down(a)
    torch.cuda.synchronize()
    assert float(h.min()) == 3.0 and float(out.min()) == 5.0      # *skip != 0: nothing is written
    bad, _ = ex.make_layout(256, 128, 4, 2)
    bad.n_ff = 120
    with pytest.raises(lib.MayaError):
        ex.gate_up(ex.make_args(bad, 1, 1, plan, w, x, h, part, out))
    bad2, _ = ex.make_layout(256, 128, 9, 0)
    with pytest.raises(lib.MayaError):
        ex.gate_up(ex.make_args(bad2, 1, 1, plan, w, x, h, part, out))


def test_expert_matches_the_reference_cpu_lane(ex):
    """Whole experts against the reference's CPU lane for EXL3 (exl3_cpu.cpp: weights and rotated input unrounded): the
    vectors of tests/golden/refbuild_exl3cpu_vectors.npz, k = 1 with weight 1 so the layer's output is the expert's."""
    from maya_amd import lib
    from test_oracle_pins import _exl3cpu_case, _exl3cpu_golden
    g = _exl3cpu_golden()
    checked = 0
    for i, row in enumerate(g["cases"]):
        l, blob, x, crc = _exl3cpu_case(ex, row)
        if crc != int(g["crc_%d" % i]):
            continue
        store = lib.ExpertStore([blob])
        layer = ex.Exl3Layer(l, 1, 1, max_tokens=1)
        out = layer.forward(store.table, torch.zeros((1, 1), dtype=torch.float32, device="cuda"), torch.from_numpy(x[None]).cuda(),
                            limit=float(g["limits"][i])).cpu().numpy()[0]
        torch.cuda.synchronize()
        err = rel_l2(out, g["out_%d" % i])
        assert err <= TOL, (i, err)
        checked += 1
    assert checked == len(g["cases"])

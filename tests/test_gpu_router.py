"""GPU parity, routing: top-k ids bit-exact with the CPU checker on random, tied and degenerate logits; grouping."""
import numpy as np
import pytest
import torch

from bench_workloads import zipf_bias

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


def _check(lib, oracle, logits, k):
    ids, w = lib.route_topk(torch.from_numpy(logits).cuda(), k)
    wi, ww = oracle.router_topk(logits, k)
    assert np.array_equal(ids.cpu().numpy(), wi)
    got = w.cpu().numpy()
    assert np.max(np.abs(got - ww) / np.maximum(ww, 1e-30)) <= 1e-5   # the reference's weight tolerance
    return got


@pytest.mark.parametrize("ne,k", ((256, 8), (160, 8), (512, 10), (8, 8), (1000, 16)))
def test_random_normal(lib, oracle, ne, k):
    rng = np.random.default_rng(ne + k)
    _check(lib, oracle, rng.standard_normal((64, ne)).astype(np.float32), k)


def test_all_equal_is_pure_tie_rule(lib, oracle):
    logits = np.full((3, 256), 0.37, dtype=np.float32)
    w = _check(lib, oracle, logits, 8)
    ids, _ = lib.route_topk(torch.from_numpy(logits).cuda(), 8)
    assert np.array_equal(ids.cpu().numpy(), np.tile(np.arange(8, dtype=np.int32), (3, 1)))
    assert np.allclose(w, 1.0 / 8, rtol=1e-6)


def test_twelve_way_tie_and_dominant(lib, oracle):
    rng = np.random.default_rng(5)
    logits = rng.standard_normal((4, 256)).astype(np.float32)
    tie = rng.choice(256, 12, replace=False)
    logits[0, tie] = 4.0
    logits[1, 77] = 60.0                 # one dominant expert: the others' p underflow towards 0
    logits[2] = np.round(logits[2] * 2) / 2   # many equal logits
    logits[3, :] = -1e30
    logits[3, 5] = 0.0
    _check(lib, oracle, logits, 8)


def test_wide_routers_ties_and_degenerate_rows(lib, oracle):
    """More than 256 experts take the candidate path: ties by index, underflowed probabilities, k up to 16."""
    rng = np.random.default_rng(15)
    for ne, k in ((1024, 8), (512, 16), (384, 6)):
        logits = rng.standard_normal((5, ne)).astype(np.float32)
        logits[0, :] = 0.25                                   # all equal: ids 0 .. k-1
        logits[1, rng.choice(ne, 20, replace=False)] = 5.0    # a 20-way tie at the top
        logits[2, :] = -1e30
        logits[2, ne - 3] = 0.0                               # one expert, every other probability exactly 0
        logits[3] = np.round(logits[3] * 2) / 2
        _check(lib, oracle, logits, k)


def test_zipf_biased(lib, oracle):
    import synth
    rng = np.random.default_rng(6)
    logits = (rng.standard_normal((512, 256)) + zipf_bias(256)[None, :]).astype(np.float32)
    _check(lib, oracle, logits, 8)


def test_plan_and_group(lib):
    rng = np.random.default_rng(9)
    for trial in range(20):
        nt, k, ne = int(rng.integers(1, 17)), 8, 24
        ids = np.stack([rng.choice(ne, k, replace=False) for _ in range(nt)]).astype(np.int32)
        table = (np.arange(ne, dtype=np.int64) + 1) * 4096
        table[rng.choice(ne, 3, replace=False)] = 0          # not resident
        plan = lib.plan(torch.from_numpy(ids).cuda(), torch.from_numpy(table).cuda())
        p = plan.cpu().numpy()
        assert np.array_equal(p, table[ids.reshape(-1)])
        gp, gs, ge, ng = [t.cpu().numpy() for t in lib.group(plan)]
        # host restatement: distinct non-null blobs in first-appearance order, entries ascending
        order, members = [], {}
        for e, b in enumerate(p):
            if b == 0:
                continue
            if b not in members:
                members[b] = []
                order.append(b)
            members[b].append(e)
        assert ng[0] == len(order)
        assert np.array_equal(gp[:len(order)], np.array(order, dtype=np.int64))
        start = 0
        for g, b in enumerate(order):
            assert gs[g] == start
            assert list(ge[start:start + len(members[b])]) == members[b]
            start += len(members[b])
        assert gs[len(order)] == start


# ---- the sigmoid router (router_sigmoid / moe_route's selection): ids bit-exact with the CPU checker, weights to the
# reference's bar of 1e-5 (src/kernels/router_sigmoid_parity.cpp:137-143), on that test's case shapes and wider ones

from test_oracle_formats import SIGMOID_CASES, non_finite_rows, sigmoid_case


def _check_sigmoid(lib, oracle, logits, bias, k, w_scale, norm):
    b = None if bias is None else torch.from_numpy(bias).cuda()
    ids, w = lib.route_sigmoid(torch.from_numpy(logits).cuda(), b, k, w_scale, norm)
    wi, ww = oracle.router_sigmoid(logits, bias, k, w_scale, norm)
    assert np.array_equal(ids.cpu().numpy(), wi)
    assert np.max(np.abs(w.cpu().numpy() - ww)) < 1e-5
    return ids.cpu().numpy(), w.cpu().numpy()


@pytest.mark.parametrize("nt,ne,k,w_scale,norm_w,with_bias,quantize,seed", SIGMOID_CASES + [
    (8, 1024, 8, 2.5, True, True, False, 21), (5, 1000, 16, 1.0, True, True, True, 22), (64, 256, 8, 2.5, True, True, False, 23),
    (3, 8, 8, 1.0, True, False, False, 24), (7, 160, 6, 1.5, True, True, True, 25)])
def test_sigmoid_router(lib, oracle, nt, ne, k, w_scale, norm_w, with_bias, quantize, seed):
    logits, bias = sigmoid_case(nt, ne, with_bias, quantize, seed)
    _check_sigmoid(lib, oracle, logits, bias, k, w_scale, 1 if norm_w else 0)
    _check_sigmoid(lib, oracle, logits, bias, k, w_scale, 2)


def test_sigmoid_router_ties_bias_and_tiny_sums(lib, oracle):
    ne, k = 256, 8
    logits = np.full((2, ne), 0.3, dtype=np.float32)
    ids, w = _check_sigmoid(lib, oracle, logits, None, k, 2.5, 1)
    assert np.array_equal(ids, np.tile(np.arange(k, dtype=np.int32), (2, 1))) and np.allclose(w, 2.5 / k, rtol=1e-6)
    # a negative selection score and a bias that selects an expert whose weight stays its small unbiased p
    logits = np.linspace(-3.0, -1.0, ne, dtype=np.float32)[None, :].copy()
    bias = np.full(ne, -0.5, dtype=np.float32)      # every score negative: the order must still be the floats' order
    bias[17] = 5.0
    ids, w = _check_sigmoid(lib, oracle, logits, bias, k, 1.0, 0)
    assert ids[0, 0] == 17 and np.array_equal(ids[0, 1:], np.arange(ne - 1, ne - k, -1))
    assert abs(w[0, 0] - 1.0 / (1.0 + np.exp(-float(logits[0, 17])))) < 1e-6
    # all sigmoids tiny: the clamp and the HF form part
    logits = np.full((1, ne), -30.0, dtype=np.float32)
    _, w1 = _check_sigmoid(lib, oracle, logits, None, k, 1.0, 1)
    _, w2 = _check_sigmoid(lib, oracle, logits, None, k, 1.0, 2)
    assert np.allclose(w2, 1.0 / k, rtol=1e-5) and float(w1.max()) < 1e-8
    L = lib.load()
    assert L.maya_moe_route_sigmoid(0, 0, 1, 8, 8, 1.0, 1, 0, 0, 0) == 3       # MAYA_E_ARG
    x = torch.zeros((1, 8), device="cuda")
    o = torch.zeros((1, 8), device="cuda")
    assert L.maya_moe_route_sigmoid(x.data_ptr(), 0, 1, 8, 8, 1.0, 3, o.data_ptr(), o.data_ptr(), 0) == 1   # MAYA_E_UNSUPPORTED
    assert L.maya_moe_route_sigmoid(x.data_ptr(), 0, 1, 8, 9, 1.0, 1, o.data_ptr(), o.data_ptr(), 0) == 2   # k > experts


def test_route_plan_in_one_launch(lib):
    rng = np.random.default_rng(31)
    for ne, k, nt in ((256, 8, 5), (300, 6, 3), (8, 2, 1)):
        logits = torch.from_numpy(rng.standard_normal((nt, ne)).astype(np.float32)).cuda()
        table = (torch.arange(1, ne + 1, dtype=torch.int64, device="cuda") * 4096)
        table[::7] = 0
        bias = torch.from_numpy((rng.standard_normal(ne) * 0.1).astype(np.float32)).cuda()
        for router in (None, lib.Router(lib.ROUTER_SIGMOID, 1, bias.data_ptr(), 2.5)):
            ids, w, pl = lib.route_plan(logits, k, table, router)
            wi, ww = lib.route_topk(logits, k) if router is None else lib.route_sigmoid(logits, bias, k, 2.5, 1)
            torch.cuda.synchronize()
            assert torch.equal(ids, wi) and torch.equal(w, ww)
            assert torch.equal(pl, lib.plan(wi.reshape(-1), table))


@pytest.mark.parametrize("ne", (64, 256, 300))
def test_sigmoid_router_refuses_non_finite_rows(lib, oracle, ne):
    """A row with a NaN / Inf logit or score gets no routes (ids -1, weights 0, null plan entries), in the router call and
    in the route-and-plan launch; its neighbours route as if it were not there."""
    k = 8
    logits = non_finite_rows(ne, 5)
    bias = (np.random.default_rng(6).standard_normal(ne) * 0.1).astype(np.float32)
    ids, w = _check_sigmoid(lib, oracle, logits, bias, k, 2.5, 1)
    assert np.all(ids[1:4] == -1) and np.all(w[1:4] == 0.0) and ids[[0, 4]].min() >= 0
    table = torch.arange(1, ne + 1, dtype=torch.int64, device="cuda") * 4096
    bias_d = torch.from_numpy(bias).cuda()
    pi, pw, pl = lib.route_plan(torch.from_numpy(logits).cuda(), k, table, lib.Router(lib.ROUTER_SIGMOID, 1, bias_d.data_ptr(), 2.5))
    torch.cuda.synchronize()
    assert np.array_equal(pi.cpu().numpy(), ids) and np.array_equal(pw.cpu().numpy(), w)
    pl = pl.cpu().numpy().reshape(5, k)
    assert np.all(pl[1:4] == 0) and np.array_equal(pl[[0, 4]], (ids[[0, 4]].astype(np.int64) + 1) * 4096)
    bias[5] = np.inf
    ids, w = _check_sigmoid(lib, oracle, logits, bias, k, 1.0, 2)
    assert np.all(ids == -1) and np.all(w == 0.0)



def _window_logits(rng, nt, ne):
    """Rows that press the router's rules: random, all equal, a many-way tie at the top, one dominant expert, many equal
    values, one expert with every other probability exactly 0."""
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    for t in range(nt):
        kind = t % 6
        if kind == 1:
            logits[t, :] = 0.25
        elif kind == 2:
            logits[t, rng.choice(ne, min(12, ne), replace=False)] = 4.0
        elif kind == 3:
            logits[t, rng.integers(ne)] = 60.0
        elif kind == 4:
            logits[t] = np.round(logits[t] * 2) / 2
        elif kind == 5:
            logits[t, :] = -1e30
            logits[t, ne - 1] = 0.0
    return logits


@pytest.mark.parametrize("nt,ne,k", ((2, 256, 8), (3, 160, 6), (4, 256, 8), (5, 64, 8), (8, 256, 8), (16, 256, 16), (16, 8, 1),
                                     (7, 200, 10), (12, 65, 3), (1, 256, 8)))
def test_window_routing_in_one_launch(lib, oracle, nt, ne, k):
    """maya_moe_route_window = maya_moe_route_plan + maya_moe_group, bit for bit (ids, weights, plan, groups), with experts
    that are not resident and tokens that share experts; ids also against the CPU checker."""
    rng = np.random.default_rng(1000 + 31 * nt + ne + k)
    logits = _window_logits(rng, nt, ne)
    table = torch.from_numpy((rng.integers(1, 1 << 40, ne) * 16).astype(np.int64)).cuda()
    table[rng.choice(ne, max(1, ne // 8), replace=False)] = 0      # not resident: null plan entries, no group
    if ne >= 4:
        table[2] = table[3]                                        # two experts behind one blob: one group
    ld = torch.from_numpy(logits).cuda()
    assert lib.load().maya_moe_route_window_ok(None, nt, ne, k) == 1
    ids, w, pl, (gp, gs, ge, ng) = lib.route_window(ld, k, table)
    ids2, w2, pl2 = lib.route_plan(ld, k, table)
    gp2, gs2, ge2, ng2 = lib.group(pl2)
    torch.cuda.synchronize()
    assert torch.equal(ids, ids2) and torch.equal(w, w2) and torch.equal(pl, pl2)
    n = int(ng.item())
    assert n == int(ng2.item())
    assert torch.equal(gp[:n], gp2[:n]) and torch.equal(gs[:n + 1], gs2[:n + 1]) and torch.equal(ge, ge2)
    wi, _ = oracle.router_topk(logits, k)
    assert np.array_equal(ids.cpu().numpy(), wi)


def test_window_routing_refuses_what_it_does_not_cover(lib):
    L = lib.load()
    assert L.maya_moe_route_window_ok(None, 4, 512, 8) == 0        # more than 256 experts
    assert L.maya_moe_route_window_ok(None, 16, 256, 16) == 1
    assert L.maya_moe_route_window_ok(None, 17, 256, 8) == 0
    r = lib.Router(lib.ROUTER_SIGMOID, 1, None, 1.0)
    import ctypes as C
    assert L.maya_moe_route_window_ok(C.byref(r), 4, 256, 8) == 0   # the sigmoid router keeps its own launches

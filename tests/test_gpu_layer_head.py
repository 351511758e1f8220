"""GPU parity of the single-token layer whose head rides in the gate/up launch (IQ2_S first, the other types below): every gate/up workgroup picks the
token's experts from the ORDER of the logits and rounds x itself, so the cases here are the ones where the order of the
logits and the order of the rounded probabilities can differ (ties, near ties, probabilities in the sub-normal range,
NaN / Inf) - the layer must give the ids, weights and output, bit for bit, of the layer that routes with the exact
router in a launch of its own.  That layer is reached by handing x over at an address that is not 16-byte aligned."""
import numpy as np
import pytest
import torch

from gpu_util import dev, make_experts, oracle_layer, rel_l2

pytestmark = pytest.mark.gpu

N_EMBD, N_FF, NE, K = 2048, 512, 40, 8


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


@pytest.fixture(scope="module")
def layer(lib):
    blobs = make_experts(22, 22, N_EMBD, N_FF, NE, 77)
    gguf_layout, _ = lib.layout(22, 22, N_EMBD, N_FF)
    store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
    return blobs, store, lib.MoeLayer(22, 22, N_EMBD, N_FF, NE, K, packing=1), lib.MoeLayer(22, 22, N_EMBD, N_FF, NE, K, packing=1)


def logit_cases():
    rng = np.random.default_rng(5)
    base = rng.standard_normal(NE).astype(np.float32)
    cases = {"random": base.copy()}
    c = base.copy()
    c[[31, 7, 19]] = np.float32(2.5)           # three equal logits at the top: the lower index first
    cases["ties at the top"] = c
    c = base.copy()
    order = np.argsort(-c)
    c[order[8]] = c[order[7]]                  # the 8th and 9th equal: the lower index is in, the other out
    cases["tie at the cut"] = c
    c = base.copy()
    c[order[3]] = np.nextafter(c[order[2]], np.float32(-10))   # one unit in the last place apart
    c[order[8]] = np.nextafter(c[order[7]], np.float32(-10))
    cases["one ulp apart"] = c
    c = np.zeros(NE, dtype=np.float32)
    c[5] = -0.0
    c[9] = -0.0
    cases["all equal, signed zeros"] = c
    c = base.copy()
    c[17] = np.float32(300.0)                  # every other probability underflows to zero: ties at p = 0
    cases["one logit far above"] = c
    c = (base * np.float32(40.0)).astype(np.float32)   # probabilities down to the sub-normal range
    cases["wide range"] = c
    c = base.copy()
    c[11] = np.float32(np.inf)
    cases["+inf"] = c
    c = base.copy()
    c[3] = np.float32(-np.inf)
    cases["-inf"] = c
    c = base.copy()
    c[20] = np.float32(np.nan)
    cases["nan"] = c
    c = np.arange(NE, dtype=np.float32) * np.float32(5e-7)   # a ladder of steps below the bar
    cases["ladder below the bar"] = c
    return cases


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16, torch.float16))
def test_head_in_the_gate_up_launch_is_the_exact_router(lib, oracle, layer, dtype):
    blobs, store, fused, plain = layer
    rng = np.random.default_rng(9)
    x32 = rng.standard_normal(N_EMBD).astype(np.float32)
    x32[256:512] = 0.0                                          # a block of zeros
    x32[600], x32[700] = 9.0, -9.0                              # equal magnitudes of either sign: the first one's sign
    xa = torch.zeros(N_EMBD + 16, dtype=dtype, device="cuda")
    off = 8 // xa.element_size()                                # 8 bytes off a 16-byte boundary
    x_al = xa[:N_EMBD].view(1, N_EMBD)
    x_un = xa[off:off + N_EMBD].view(1, N_EMBD)
    assert x_al.data_ptr() % 16 == 0 and x_un.data_ptr() % 16 == 8
    for name, lg in logit_cases().items():
        print("case", name, dtype, flush=True)
        logits = dev(lg.reshape(1, NE))
        x_al.copy_(torch.from_numpy(x32).to(dtype).view(1, -1))
        out_f = fused.forward(store.table, logits, x_al).clone()
        ids_f, w_f = fused.ids.clone(), fused.weights.clone()
        x_un.copy_(torch.from_numpy(x32).to(dtype).view(1, -1))
        out_p = plain.forward(store.table, logits, x_un).clone()
        torch.cuda.synchronize()
        assert torch.equal(ids_f, plain.ids), (name, ids_f, plain.ids)
        assert torch.equal(w_f.view(torch.int32), plain.weights.view(torch.int32)), name
        assert torch.equal(out_f.view(torch.int32), out_p.view(torch.int32)), name
    # and against the CPU path on the plain case
    lg = logit_cases()["random"].reshape(1, NE)
    xin = torch.from_numpy(x32).to(dtype)
    out = fused.forward(store.table, dev(lg), xin.cuda().view(1, -1)).cpu().numpy()
    wi, ww, wout = oracle_layer(oracle, 22, 22, blobs, K, N_EMBD, N_FF, lg, xin.float().numpy().reshape(1, -1))
    assert np.array_equal(fused.ids.cpu().numpy(), wi) and rel_l2(out[0], wout[0]) <= 1e-3


def test_absent_experts_and_k_next_to_the_expert_count(lib, oracle):
    """k = n_expert - 1 (the order-only pick needs one expert beyond the slots) and k = n_expert (the head then stays a
    launch of its own); experts missing from the table give no contribution on either path."""
    n_embd, n_ff = 2048, 512
    for ne, k in ((5, 4), (4, 4), (9, 8)):
        blobs = make_experts(22, 22, n_embd, n_ff, ne, 90 + ne)
        gguf_layout, _ = lib.layout(22, 22, n_embd, n_ff)
        store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
        table = store.table.clone()
        table[1] = 0
        rng = np.random.default_rng(ne)
        logits = dev(rng.standard_normal((1, ne)).astype(np.float32))
        xa = torch.zeros(n_embd + 8, dtype=torch.float32, device="cuda")
        x32 = torch.from_numpy(rng.standard_normal(n_embd).astype(np.float32)).cuda()
        a, b = lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1), lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1)
        x_al, x_un = xa[:n_embd].view(1, -1), xa[2:2 + n_embd].view(1, -1)
        x_al.copy_(x32.view(1, -1))
        out_a = a.forward(table, logits, x_al).clone()
        x_un.copy_(x32.view(1, -1))
        out_b = b.forward(table, logits, x_un).clone()
        torch.cuda.synchronize()
        assert torch.equal(a.ids, b.ids) and torch.equal(a.weights.view(torch.int32), b.weights.view(torch.int32))
        assert torch.equal(out_a.view(torch.int32), out_b.view(torch.int32)), (ne, k)
        assert float(out_a.abs().max()) > 0


def test_order_only_pick_against_the_exact_router_on_adversarial_rows(lib):
    """Rows built to sit on the order-only pick's edges: values on a coarse grid (many exact ties), values a few units in
    the last place apart at magnitudes from 1e-3 to 1e3 and of either sign (one 256-ulp bucket holds several), steps just
    under and just over the 1e-6 bar, everything within 1e-6 of zero.  ids and weights must be the exact router's
    (maya_moe_route_topk), and the output - which depends on what the gate/up workgroups picked for themselves - the
    output of the layer that routes in a launch of its own (x handed over unaligned), all bit for bit."""
    n_embd, n_ff, ne, k = 2048, 512, 256, 8
    blobs = make_experts(22, 22, n_embd, n_ff, ne, 123)
    gguf_layout, _ = lib.layout(22, 22, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
    fused, plain = lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1), lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1)
    xa = torch.zeros(n_embd + 8, dtype=torch.float32, device="cuda")
    x32 = torch.randn(n_embd, device="cuda")
    x_al, x_un = xa[:n_embd].view(1, -1), xa[2:2 + n_embd].view(1, -1)
    rng = np.random.default_rng(2024)
    rows = []
    for trial in range(25):
        base = rng.standard_normal(ne).astype(np.float32)
        rows.append(base)
        rows.append((np.round(base * 4) / 4).astype(np.float32))              # a coarse grid: ties everywhere
        for mag in (1e-3, 0.3, 1.0, 3.0, 50.0, 1e3):
            for sign in (1.0, -1.0):
                c = (-np.abs(base) * np.float32(mag) - np.float32(2 * mag)).astype(np.float32)
                top = rng.permutation(ne)[:12]
                steps = rng.integers(0, 6, size=12)                           # 0 .. 5 ulps apart, some equal
                v = np.float32(sign * mag)
                for j, st in zip(top, steps):
                    c[j] = v
                    for _ in range(int(st)):
                        v = np.nextafter(v, np.float32(-np.inf))
                rows.append(c)
        c = base.copy()
        top = np.argsort(-c)[:10]
        c[top] = np.float32(1.0) - np.arange(10, dtype=np.float32) * np.float32(rng.choice([0.9e-6, 1.1e-6, 2e-6]))
        rows.append(c)
        rows.append((base * np.float32(1e-7)).astype(np.float32))             # everything within 1e-6 of zero, both signs
    rows = np.stack(rows).astype(np.float32)
    want_ids, want_w = lib.route_topk(dev(rows), k)
    bad = 0
    for i in range(rows.shape[0]):
        lg = dev(rows[i:i + 1])
        x_al.copy_(x32.view(1, -1))
        out_f = fused.forward(store.table, lg, x_al).clone()
        x_un.copy_(x32.view(1, -1))
        out_p = plain.forward(store.table, lg, x_un)
        ok = (torch.equal(fused.ids[0], want_ids[i]) and torch.equal(fused.weights[0].view(torch.int32), want_w[i].view(torch.int32))
              and torch.equal(plain.ids[0], want_ids[i]) and torch.equal(out_f.view(torch.int32), out_p.view(torch.int32)))
        if not ok:
            bad += 1
            print("row", i, fused.ids[0].tolist(), want_ids[i].tolist(), flush=True)
    torch.cuda.synchronize()
    assert bad == 0, bad


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt", ((22, 22, 2048, 512, 12, 4, 1), (22, 22, 2048, 1024, 12, 4, 3),
                                                      (12, 12, 2048, 2048, 6, 3, 1), (22, 12, 1024, 512, 8, 8, 6)))
def test_the_layer_in_two_calls_is_the_layer(lib, gt, dt, n_embd, n_ff, ne, k, nt):
    """maya_moe_layer_decode_begin + maya_moe_layer_decode_end on the same arguments = maya_moe_layer_decode, bit for bit."""
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 31 + nt)
    gguf_layout, _ = lib.layout(gt, dt, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
    rng = np.random.default_rng(nt)
    logits = dev(rng.standard_normal((nt, ne)).astype(np.float32))
    x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    add = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    whole = lib.MoeLayer(gt, dt, n_embd, n_ff, ne, k, max_tokens=nt, packing=1)
    halves = lib.MoeLayer(gt, dt, n_embd, n_ff, ne, k, max_tokens=nt, packing=1)
    want = whole.forward(store.table, logits, x, add=add).clone()
    halves.out.zero_()
    halves.forward(store.table, logits, x, add=add, half="begin")
    torch.cuda.synchronize()
    assert float(halves.out.abs().max()) == 0.0          # nothing of the second half has run
    got = halves.forward(store.table, logits, x, add=add, half="end")
    torch.cuda.synchronize()
    assert torch.equal(whole.ids, halves.ids) and torch.equal(whole.weights.view(torch.int32), halves.weights.view(torch.int32))
    assert torch.equal(want.view(torch.int32), got.view(torch.int32))


@pytest.mark.parametrize("norm,with_bias", ((1, True), (0, False), (2, True)))
def test_sigmoid_router_in_the_gate_up_launch(lib, norm, with_bias):
    """The sigmoid router (bias, weight scale, the three normalisations) with the head in the gate/up launch: ids, weights
    and output bit for bit those of the three-launch layer (x unaligned) and of maya_moe_route_sigmoid, on random rows,
    equal scores (equal logits with equal bias; a bias that makes different logits meet), saturated sigmoids (p = 1 for
    many experts: ties at the top), scores a unit in the last place apart, and rows with NaN / Inf (refused: ids -1,
    weights 0, the output just `add`)."""
    n_embd, n_ff, ne, k = 2048, 512, 64, 6
    blobs = make_experts(22, 22, n_embd, n_ff, ne, 321)
    gguf_layout, _ = lib.layout(22, 22, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
    fused, plain = lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1), lib.MoeLayer(22, 22, n_embd, n_ff, ne, k, packing=1)
    rng = np.random.default_rng(77 + norm)
    bias = (rng.standard_normal(ne) * 0.1).astype(np.float32)
    bias[[3, 9]] = 0.25
    bias_d = dev(bias)
    router = lib.Router(lib.ROUTER_SIGMOID, norm, bias_d.data_ptr() if with_bias else 0, 2.5)
    rows = []
    for trial in range(12):
        base = rng.standard_normal(ne).astype(np.float32)
        rows.append(base)
        c = base.copy()
        c[[3, 9, 20]] = np.float32(1.75)                                      # equal logits (3 and 9 with equal bias too)
        rows.append(c)
        rows.append((base * np.float32(30.0)).astype(np.float32))             # saturated: p = 1 (or 0) for most experts
        c = base.copy()
        top = np.argsort(-c)[:8]
        v = np.float32(2.0)
        for j in top:
            c[j] = v
            v = np.nextafter(v, np.float32(-np.inf))                          # neighbours in the last place
        rows.append(c)
        rows.append((np.round(base * 2) / 2).astype(np.float32))              # a coarse grid
    c = rng.standard_normal(ne).astype(np.float32)
    c[11] = np.float32(np.nan)
    rows.append(c)
    c = rng.standard_normal(ne).astype(np.float32)
    c[5] = np.float32(np.inf)
    rows.append(c)
    rows = np.stack(rows).astype(np.float32)
    want_ids, want_w = lib.route_sigmoid(dev(rows), bias_d if with_bias else None, k, 2.5, norm)
    xa = torch.zeros(n_embd + 8, dtype=torch.float32, device="cuda")
    x32 = torch.randn(n_embd, device="cuda")
    add = torch.randn(1, n_embd, device="cuda")
    x_al, x_un = xa[:n_embd].view(1, -1), xa[2:2 + n_embd].view(1, -1)
    bad = 0
    for i in range(rows.shape[0]):
        lg = dev(rows[i:i + 1])
        x_al.copy_(x32.view(1, -1))
        out_f = fused.forward(store.table, lg, x_al, add=add, router=router).clone()
        x_un.copy_(x32.view(1, -1))
        out_p = plain.forward(store.table, lg, x_un, add=add, router=router)
        ok = (torch.equal(fused.ids[0], want_ids[i]) and torch.equal(fused.weights[0].view(torch.int32), want_w[i].view(torch.int32))
              and torch.equal(plain.ids[0], want_ids[i]) and torch.equal(out_f.view(torch.int32), out_p.view(torch.int32)))
        if not ok:
            bad += 1
            print("row", i, fused.ids[0].tolist(), want_ids[i].tolist(), flush=True)
    torch.cuda.synchronize()
    assert bad == 0, bad
    assert int(want_ids[-1, 0]) == -1 and int(want_ids[-2, 0]) == -1          # the refused rows were in the set


@pytest.mark.parametrize("ty,n_embd,n_ff,ne,k", ((12, 2048, 512, 40, 8), (12, 2048, 2048, 12, 8), (12, 3072, 512, 9, 4), (12, 7168, 256, 6, 1),
                                                   (19, 2048, 512, 40, 8), (19, 3072, 256, 9, 4), (19, 5120, 256, 7, 2)))
def test_other_types_head_in_the_gate_up_launch(lib, oracle, ty, n_embd, n_ff, ne, k):
    """The same for Q4_K and IQ1_S experts (their position-mapped gate/up kernels with the head in them): for Q4_K
    the 8-row launch of few entries and the 16-row one; row lengths whose middle wave holds gate and up lanes (3072,
    5120); one slot (k = 1); F32, BF16 and F16 x; edge logits; the sigmoid router.  ids, weights and output bit for bit
    those of the three-launch layer, and the CPU path's within 1e-3."""
    blobs = make_experts(ty, ty, n_embd, n_ff, ne, 500 + ne)
    gguf_layout, _ = lib.layout(ty, ty, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf_layout)
    fused, plain = lib.MoeLayer(ty, ty, n_embd, n_ff, ne, k, packing=1), lib.MoeLayer(ty, ty, n_embd, n_ff, ne, k, packing=1)
    rng = np.random.default_rng(n_embd + ne)
    x32 = rng.standard_normal(n_embd).astype(np.float32)
    x32[256:512] = 0.0
    x32[600], x32[700] = 9.0, -9.0
    rows = [rng.standard_normal(ne).astype(np.float32) for _ in range(6)]
    c = rows[0].copy()
    c[[1, 4]] = np.float32(2.5)                                   # a tie at the top
    rows.append(c)
    c = rows[1].copy()
    order = np.argsort(-c)
    c[order[k]] = c[order[k - 1]]                                 # a tie at the cut
    rows.append(c)
    c = rows[2].copy()
    c[order[0]] = np.nextafter(c[order[1]], np.float32(10))       # one unit in the last place apart
    rows.append(c)
    rows.append(np.zeros(ne, dtype=np.float32))
    c = rows[3].copy()
    c[2] = np.float32(np.nan)
    rows.append(c)
    bias = dev((rng.standard_normal(ne) * 0.1).astype(np.float32))
    routers = (None, lib.Router(lib.ROUTER_SIGMOID, 1, bias.data_ptr(), 2.5))
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        xa = torch.zeros(n_embd + 16, dtype=dtype, device="cuda")
        off = 8 // xa.element_size()
        x_al, x_un = xa[:n_embd].view(1, n_embd), xa[off:off + n_embd].view(1, n_embd)
        for router in routers:
            for i, lg in enumerate(rows):
                print("case", n_embd, n_ff, dtype, router is not None, i, flush=True)
                logits = dev(lg.reshape(1, ne))
                x_al.copy_(torch.from_numpy(x32).to(dtype).view(1, -1))
                out_f = fused.forward(store.table, logits, x_al, router=router).clone()
                ids_f, w_f = fused.ids.clone(), fused.weights.clone()
                x_un.copy_(torch.from_numpy(x32).to(dtype).view(1, -1))
                out_p = plain.forward(store.table, logits, x_un, router=router).clone()
                torch.cuda.synchronize()
                assert torch.equal(ids_f, plain.ids), (i, ids_f, plain.ids)
                assert torch.equal(w_f.view(torch.int32), plain.weights.view(torch.int32)), i
                assert torch.equal(out_f.view(torch.int32), out_p.view(torch.int32)), i
    lg = rows[0].reshape(1, ne)
    xin = torch.from_numpy(x32)
    out = fused.forward(store.table, dev(lg), xin.cuda().view(1, -1)).cpu().numpy()
    wi, ww, wout = oracle_layer(oracle, ty, ty, blobs, k, n_embd, n_ff, lg, x32.reshape(1, -1))
    assert np.array_equal(fused.ids.cpu().numpy(), wi) and rel_l2(out[0], wout[0]) <= 1e-3

"""GPU parity, the residency tiers of the routed experts: route + plan against the tables (bit for bit with the CPU
checker's plan over the same ids), the fetch of second-tier blobs, the table edits, and a layer whose experts arrive
through them against the same layer with every expert resident."""
import numpy as np
import pytest
import torch

from gpu_util import dev, make_experts

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


def u64(t):
    return t.cpu().numpy().view(np.uint64)


def random_tables(rng, nl, ne, p_hbm, p_ram, p_spare):
    tab = np.zeros(nl * (2 * ne + 3), dtype=np.uint64)
    n = nl * ne
    hbm = rng.random(n) < p_hbm
    tab[:n][hbm] = (rng.integers(1, 1 << 30, size=int(hbm.sum())) * 256).astype(np.uint64)
    ram = rng.random(n) < p_ram
    tab[n:2 * n][ram] = (rng.integers(1, 1 << 30, size=int(ram.sum())) * 256 + (1 << 40)).astype(np.uint64)
    sp = rng.random(nl * 3) < p_spare
    tab[2 * n:][sp] = (rng.integers(1, 1 << 30, size=int(sp.sum())) * 256 + (1 << 41)).astype(np.uint64)
    return tab


@pytest.mark.parametrize("ne,k,nt,sigmoid,promote_min,seed", (
    (64, 8, 1, False, 0, 1), (256, 8, 4, True, 0, 2), (300, 6, 3, True, 2, 3), (16, 4, 8, False, 3, 4), (160, 8, 16, True, 0, 5)))
def test_route_tiered_matches_the_checker_over_a_run_of_routes(lib, oracle, ne, k, nt, sigmoid, promote_min, seed):
    rng = np.random.default_rng(seed)
    nl = 3
    tab = random_tables(rng, nl, ne, 0.4, 0.6, 0.8)
    scratch = (np.arange(1, 6, dtype=np.uint64) * 4096 + (1 << 42)).astype(np.uint64)
    tiers = lib.Tiers(nl, ne, dev(scratch.view(np.int64)), nt * k, with_counts=True)
    tiers.tab.copy_(dev(tab.view(np.int64)))
    tiers.seq.fill_(4096 - 3)     # the counts age during the run
    counts = np.zeros(nl * ne, dtype=np.uint32)
    seq = np.array([4096 - 3], dtype=np.uint32)
    bias = (rng.standard_normal(ne) * 0.1).astype(np.float32)
    bias_d = dev(bias)
    router = lib.Router(lib.ROUTER_SIGMOID, 1, bias_d.data_ptr(), 2.5) if sigmoid else None
    for step in range(6):
        layer = int(rng.integers(0, nl))
        logits = (rng.standard_normal((nt, ne)) * 2).astype(np.float32)
        if step == 4 and sigmoid:
            logits[nt // 2, 3] = np.nan        # a refused row plans nothing and counts nothing
        if step == 3:                          # the engine hands slots back between tokens
            keys = np.array([2 * nl * ne + 3 * layer + 1, 2 * nl * ne + 3 * layer + 2, -5, 10 ** 9], dtype=np.int32)
            vals = np.array([(1 << 43) + 256 * step, (1 << 43) + 512 * step, 77, 78], dtype=np.uint64)
            tiers.update(dev(keys), dev(vals.view(np.int64)))
            tab[keys[0]], tab[keys[1]] = vals[0], vals[1]
        print("step", step, "layer", layer, flush=True)
        ids, w, pl = tiers.route(dev(logits), layer, k, router, promote_min)
        torch.cuda.synchronize()
        wi, ww = (lib.route_sigmoid(dev(logits), bias_d, k, 2.5, 1) if sigmoid else lib.route_topk(dev(logits), k))
        assert torch.equal(ids, wi) and torch.equal(w, ww)
        plan, src, masks = oracle.plan_tiered(ids.cpu().numpy(), layer, ne, tab, scratch, counts, seq, promote_min)
        assert np.array_equal(u64(pl).reshape(nt, k), plan)
        assert np.array_equal(u64(tiers.fetch_src[:nt * k]).reshape(nt, k), src)
        assert np.array_equal(tiers.masks[:4 * nt].cpu().numpy().view(np.uint32).reshape(nt, 4), masks)
        assert np.array_equal(u64(tiers.tab), tab)
        assert np.array_equal(tiers.counts.cpu().numpy().view(np.uint32), counts)
        assert int(tiers.seq.item()) == int(seq[0])


def test_route_tiered_argument_checks(lib):
    L = lib.load()
    tiers = lib.Tiers(2, 8, torch.zeros(2, dtype=torch.int64, device="cuda"), 8)
    logits = torch.zeros((1, 8), device="cuda")
    ids = torch.zeros(8, dtype=torch.int32, device="cuda")
    w = torch.zeros(8, device="cuda")
    pl = torch.zeros(8, dtype=torch.int64, device="cuda")
    import ctypes as C
    call = lambda layer, ne, k: L.maya_moe_route_tiered(None, logits.data_ptr(), 1, layer, ne, k, C.byref(tiers.c), 0, ids.data_ptr(),
                                                        w.data_ptr(), pl.data_ptr(), None)
    assert call(0, 8, 4) == 0
    assert call(2, 8, 4) == 2 and call(-1, 8, 4) == 2      # MAYA_E_SHAPE: no such layer
    assert call(0, 4, 4) == 2                              # the tables are not this many experts a layer
    assert L.maya_moe_route_tiered(None, None, 1, 0, 8, 4, C.byref(tiers.c), 0, ids.data_ptr(), w.data_ptr(), pl.data_ptr(), None) == 3
    assert L.maya_moe_fetch(None, pl.data_ptr(), 8, 16, None) == 3 and L.maya_moe_fetch(pl.data_ptr(), pl.data_ptr(), 0, 16, None) == 2
    torch.cuda.synchronize()


@pytest.mark.parametrize("nbytes,src_off,dst_off,pinned", ((4096, 0, 0, False), (100000, 0, 0, True), (65537, 2, 2, False), (12345, 2, 6, True),
                                                         (3 << 20, 0, 0, True)))
def test_fetch_copies_the_entries_with_a_source(lib, nbytes, src_off, dst_off, pinned):
    n = 6
    stride = (nbytes + 511) & ~255
    g = torch.Generator().manual_seed(nbytes)
    host = torch.randint(0, 256, (n * stride + 256,), dtype=torch.uint8, generator=g)
    if pinned:
        ram = torch.empty(n * stride + 256, dtype=torch.uint8, pin_memory=True)   # the second tier in mapped host memory
        ram.copy_(host)
    else:
        ram = host.cuda()
    slots = torch.full((n * stride + 256,), 0xEE, dtype=torch.uint8, device="cuda")
    src = torch.zeros(n, dtype=torch.int64)
    dst = torch.zeros(n, dtype=torch.int64)
    sbase, dbase = ram.data_ptr() + (-ram.data_ptr()) % 256, slots.data_ptr() + (-slots.data_ptr()) % 256
    for e in (0, 2, 3, 5):
        src[e] = sbase + e * stride + src_off
    for e in range(n):
        dst[e] = dbase + (n - 1 - e) * stride + dst_off      # entry e -> slot n-1-e
    dst[3] = 0                                              # an entry the plan left out: nothing is written for it
    tiers = lib.Tiers(1, 8, torch.zeros(0, dtype=torch.int64, device="cuda"), n)
    tiers.fetch_src.copy_(src.cuda())
    tiers.fetch(dst.cuda(), nbytes)
    torch.cuda.synchronize()
    got = slots.cpu().numpy()
    want = np.full_like(got, 0xEE)
    h = host.numpy()
    so, do = sbase - ram.data_ptr(), dbase - slots.data_ptr()
    for e in (0, 2, 5):
        a = do + (n - 1 - e) * stride + dst_off
        b = so + e * stride + src_off
        want[a:a + nbytes] = h[b:b + nbytes]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt,packing", ((22, 22, 7168, 2048, 12, 8, 1, 1), (22, 12, 1024, 512, 16, 4, 3, 0)))
def test_a_layer_whose_experts_arrive_through_the_tiers(lib, gt, dt, n_embd, n_ff, ne, k, nt, packing):
    """HBM holds a third of the experts, mapped host memory all of them; the route promotes into three spares, takes
    scratch slots for the rest, the fetch fills them, and the layer over that plan gives bit for bit what it gives with
    every expert resident."""
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 400 + gt + dt)
    gguf, bb = lib.layout(gt, dt, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf if packing else None)
    rng = np.random.default_rng(9)
    logits = (rng.standard_normal((nt, ne)) * 2).astype(np.float32)
    x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    router = lib.Router(lib.ROUTER_SIGMOID, 1, 0, 2.5)
    layer = lib.MoeLayer(gt, dt, n_embd, n_ff, ne, k, max_tokens=nt, packing=packing)
    ref = layer.forward(store.table, dev(logits), x, router=router).clone()
    ref_ids = layer.ids[:nt].clone()
    # the second tier: every (packed) blob in mapped host memory
    stride = (bb + 255) & ~255
    ram = torch.empty(ne * stride + 256, dtype=torch.uint8, pin_memory=True)
    rbase = ram.data_ptr() + (-ram.data_ptr()) % 256
    roff = rbase - ram.data_ptr()
    pool_host = store.pool.cpu()
    for e in range(ne):
        o = store.addrs[e] - store.pool.data_ptr()
        ram[roff + e * stride:roff + e * stride + bb].copy_(pool_host[o:o + bb])
    n_slots = 3 + nt * k
    slots = torch.zeros(n_slots * stride + 256, dtype=torch.uint8, device="cuda")
    sb = slots.data_ptr() + (-slots.data_ptr()) % 256
    scratch = torch.tensor([sb + (3 + i) * stride for i in range(nt * k)], dtype=torch.int64, device="cuda")
    tiers = lib.Tiers(1, ne, scratch, nt * k)
    tab = np.zeros(2 * ne + 3, dtype=np.int64)
    for e in range(0, ne, 3):
        tab[e] = store.addrs[e]
    for e in range(ne):
        tab[ne + e] = rbase + e * stride
    tab[2 * ne:] = [sb, sb + stride, sb + 2 * stride]
    tiers.tab.copy_(dev(tab))
    ids, w, pl = tiers.route(dev(logits), 0, k, router)
    tiers.fetch(pl, bb)
    torch.cuda.synchronize()
    masks = tiers.masks[:4 * nt].cpu().numpy().reshape(nt, 4)
    assert torch.equal(ids, ref_ids) and np.all(masks[:, 0] == 0) and np.all(masks[:, 3] == 0) and masks[:, 1].any() and masks[0, 2] != 0
    assert int((pl == 0).sum()) == 0
    # the layer over this plan: a table that holds, for every routed expert, where the plan put it
    table = torch.zeros(ne, dtype=torch.int64, device="cuda")
    table[ids.reshape(-1).long()] = pl
    out = layer.forward(table, None, x, router=router, routed=(ids, w))
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


@pytest.mark.parametrize("nbytes,src_off,dst_off,pinned,count,wgs", ((4096, 0, 0, False, 3, 0), (100000, 0, 0, True, 6, 4), (65537, 2, 2, False, 9, 1),
                                                                    (12345, 2, 6, True, 2, 7), (3 << 20, 0, 0, True, 4, 0), (4096, 0, 0, False, 0, 0)))
def test_prefetch_copies_the_counted_entries_of_the_list(lib, nbytes, src_off, dst_off, pinned, count, wgs):
    """maya_moe_prefetch: the first *pf_n entries of the list (a device count; past the list's length it is clamped), a null
    source or slot skipped, nothing else written - from HBM and from mapped host memory, aligned and not, by 1 ... n workgroups."""
    n = 6
    stride = (nbytes + 511) & ~255
    g = torch.Generator().manual_seed(nbytes + count)
    host = torch.randint(0, 256, (n * stride + 256,), dtype=torch.uint8, generator=g)
    if pinned:
        ram = torch.empty(n * stride + 256, dtype=torch.uint8, pin_memory=True)
        ram.copy_(host)
    else:
        ram = host.cuda()
    slots = torch.full((n * stride + 256,), 0xEE, dtype=torch.uint8, device="cuda")
    src = torch.zeros(n, dtype=torch.int64)
    dst = torch.zeros(n, dtype=torch.int64)
    sbase, dbase = ram.data_ptr() + (-ram.data_ptr()) % 256, slots.data_ptr() + (-slots.data_ptr()) % 256
    for e in range(n):
        src[e] = sbase + e * stride + src_off
        dst[e] = dbase + (n - 1 - e) * stride + dst_off      # entry e -> slot n-1-e
    src[1] = 0                                              # an entry without a source
    dst[4] = 0                                              # ... and one without a slot
    pf_n = torch.tensor([count], dtype=torch.int32, device="cuda")
    lib.prefetch(src.cuda(), dst.cuda(), pf_n, nbytes, n_workgroups=wgs)
    torch.cuda.synchronize()
    got = slots.cpu().numpy()
    want = np.full_like(got, 0xEE)
    h = host.numpy()
    so, do = sbase - ram.data_ptr(), dbase - slots.data_ptr()
    for e in range(min(count, n)):
        if e in (1, 4):
            continue
        a = do + (n - 1 - e) * stride + dst_off
        b = so + e * stride + src_off
        want[a:a + nbytes] = h[b:b + nbytes]
    assert np.array_equal(got, want)
    L = lib.load()
    assert L.maya_moe_prefetch(None, dst.cuda().data_ptr(), pf_n.data_ptr(), n, nbytes, 0, None) == 3
    assert L.maya_moe_prefetch(src.cuda().data_ptr(), dst.cuda().data_ptr(), pf_n.data_ptr(), 0, nbytes, 0, None) == 2

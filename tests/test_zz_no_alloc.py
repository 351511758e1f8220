"""maya_moe_layer_decode_static, the layer call that allocates nothing (its workspace is a device array inside the library):
through the C ABI its ids, weights and output equal maya_moe_layer_decode_routed's with a caller workspace, bit for bit, on two
calls in a row - the second on a smaller input, so whatever the first left in the shared array does not leak into it - and a
call that would not fit is refused before anything is launched."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import dev, make_experts

pytestmark = pytest.mark.gpu


def _static(lib, L, layer, table, logits, x, router=None):
    nt = x.shape[0]
    ids = torch.full((nt, layer.k), -7, dtype=torch.int32, device="cuda")
    w = torch.zeros((nt, layer.k), dtype=torch.float32, device="cuda")
    out = torch.full((nt, layer.n_embd), float("nan"), dtype=torch.float32, device="cuda")
    rc = L.maya_moe_layer_decode_static(C.byref(layer.layout), lib._p(table), layer.n_expert, layer.k, router, lib._p(logits), lib._p(x),
                                        lib.dtype_id(x), nt, float("inf"), None, lib._p(ids), lib._p(w), lib._p(out), lib._stream())
    return rc, ids, w, out


def test_static_layer_equals_the_workspace_layer_twice_in_a_row():
    from maya_amd import lib
    L = lib.load()
    lib.check(L.maya_init())
    L.maya_moe_layer_decode_static.argtypes = [C.POINTER(lib.Layout), C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    rng = np.random.default_rng(2026)
    # first call: 3 tokens of a 4096 x 2048 IQ2_S layer (stream packing: the position-mapped kernels), top-8 of 12;
    # second call: 1 token of a 1024 x 512 IQ2_S / Q4_K layer (GGUF packing: the generic kernels), top-4 of 6
    for gt, dt, n_embd, n_ff, ne, k, nt, packing in ((22, 22, 4096, 2048, 12, 8, 3, 1), (22, 12, 1024, 512, 6, 4, 1, 0)):
        blobs = make_experts(gt, dt, n_embd, n_ff, ne, 900 + n_embd)
        gguf, _ = lib.layout(gt, dt, n_embd, n_ff)
        store = lib.ExpertStore(blobs, pack_layout=gguf if packing else None)
        layer = lib.MoeLayer(gt, dt, n_embd, n_ff, ne, k, max_tokens=nt, packing=packing)
        logits = dev(rng.standard_normal((nt, ne)).astype(np.float32))
        x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
        print("static layer call", gt, dt, n_embd, n_ff, ne, k, nt, packing, flush=True)
        rc, ids, w, out = _static(lib, L, layer, store.table, logits, x)
        assert rc == 0, L.maya_last_error().decode()
        want = layer.forward(store.table, logits, x).clone()
        torch.cuda.synchronize()
        assert torch.equal(ids, layer.ids[:nt]) and torch.equal(w, layer.weights[:nt])
        assert torch.equal(out.view(torch.int32), want.view(torch.int32)) and float(want.abs().max()) > 0
    # a call whose scratch would not fit in the static array is refused, nothing launched
    gguf, _ = lib.layout(22, 22, 8192, 4096)
    big = lib.MoeLayer(22, 22, 8192, 4096, 4, 4, max_tokens=8)
    assert int(L.maya_moe_workspace_bytes(C.byref(big.layout), 8, 4)) > (1 << 20)
    logits = torch.zeros((8, 4), device="cuda")
    x = torch.zeros((8, 8192), device="cuda")
    rc, ids, w, out = _static(lib, L, big, torch.zeros(4, dtype=torch.int64, device="cuda"), logits, x)
    torch.cuda.synchronize()
    assert rc == 2 and b"static" in L.maya_last_error()
    assert int(ids[0, 0]) == -7 and bool(torch.isnan(out).all())


def test_static_layer_is_capturable_and_leaves_device_memory_alone():
    """Nothing is allocated: the call is captured into a HIP graph (a capture fails when anything under it allocates device
    memory or copies synchronously), the device's free memory is the same before and after, and the replayed graph gives the
    eager call's bits."""
    from maya_amd import lib
    L = lib.load()
    lib.check(L.maya_init())
    L.maya_moe_layer_decode_static.argtypes = [C.POINTER(lib.Layout), C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    rng = np.random.default_rng(2027)
    gt, dt, n_embd, n_ff, ne, k, nt = 22, 22, 4096, 2048, 12, 8, 2
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 950)
    gguf, _ = lib.layout(gt, dt, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf)
    layer = lib.MoeLayer(gt, dt, n_embd, n_ff, ne, k, max_tokens=nt, packing=1)
    logits = dev(rng.standard_normal((nt, ne)).astype(np.float32))
    x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    rc, ids, w, out = _static(lib, L, layer, store.table, logits, x)   # (eager first: every kernel's code is on the device)
    assert rc == 0, L.maya_last_error().decode()
    torch.cuda.synchronize()
    want = out.clone()
    ids2 = torch.full_like(ids, -7)
    w2 = torch.zeros_like(w)
    out2 = torch.full_like(out, float("nan"))
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        rc = L.maya_moe_layer_decode_static(C.byref(layer.layout), lib._p(store.table), ne, k, None, lib._p(logits), lib._p(x), lib.dtype_id(x), nt,
                                            float("inf"), None, lib._p(ids2), lib._p(w2), lib._p(out2), lib._stream())
    assert rc == 0, L.maya_last_error().decode()
    for _ in range(2):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ids2, ids) and torch.equal(w2, w) and torch.equal(out2.view(torch.int32), want.view(torch.int32))
        out2.fill_(float("nan"))
        torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before - (4 << 20)   # (the graph's own launch records, nothing else)

"""The routed layer with the shared expert beside it (maya_moe_layer_decode_shared): the shared expert's launches run on
the library's second stream while the routed experts' head and gate/up run on the caller's.  The result must be the bits
of the two calls it replaces - the shared expert through the stage calls, then the routed layer with add = its output -
eagerly, call after call on changing inputs, and replayed from a HIP graph."""
import numpy as np
import pytest
import torch

from gpu_util import oracle_layer, rel_l2
import bench_workloads as workloads

pytestmark = pytest.mark.gpu
IQ2_S, Q4_K, Q8_0 = 22, 12, 8
FIELDS = {IQ2_S: (82, {0: (2e-3, 6e-3)}), Q4_K: (144, {0: (2e-4, 6e-4), 2: (2e-4, 6e-4)}), Q8_0: (34, {0: (1e-4, 4e-4)})}


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


def build(lib, gt, dt, st, E, FF, NE, TK, T, seed):
    gguf, bb = lib.layout(gt, dt, E, FF)
    pool = torch.empty(NE * bb, dtype=torch.uint8, device="cuda")
    view = pool.view(NE, bb)
    view[:, :gguf.down_off] = workloads.random_blocks(NE * gguf.down_off, *FIELDS[gt], seed).view(NE, -1)
    view[:, gguf.down_off:] = workloads.random_blocks(NE * (bb - gguf.down_off), *FIELDS[dt], seed + 1).view(NE, -1)
    packed = torch.empty_like(pool)
    for e in range(NE):
        lib.repack(gguf, view[e], packed[e * bb:(e + 1) * bb])
    table = torch.tensor([packed.data_ptr() + e * bb for e in range(NE)], dtype=torch.int64, device="cuda")
    sg, sbb = lib.layout(st, st, E, FF)
    sh = workloads.random_blocks(sbb, *FIELDS[st], seed + 2)
    sh_packed = torch.empty_like(sh)
    lib.repack(sg, sh, sh_packed)
    torch.cuda.synchronize()
    layer = lib.MoeLayer(gt, dt, E, FF, NE, TK, max_tokens=T, packing=lib.PACK_STREAM)
    dense = lib.DenseExpert(st, st, E, FF, T, sh_packed.data_ptr(), packing=lib.PACK_STREAM)
    return dict(gguf=gguf, view=view, packed=packed, table=table, sg=sg, sh=sh, sh_packed=sh_packed, layer=layer, dense=dense)


def inputs(E, NE, T, seed):
    rng = np.random.default_rng(seed)
    return (torch.from_numpy(rng.standard_normal((T, NE)).astype(np.float32)).cuda(),
            torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).cuda(),
            torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).cuda())


def two_calls(w, logits, x, add, limit):
    """The shared expert through the stage calls (the residual in its down launch), then the routed layer on top of it."""
    a = w["dense"].args
    a.add = add.data_ptr() if add is not None else None
    sh = w["dense"].forward(x, limit=limit)
    a.add = None
    return w["layer"].forward(w["table"], logits, x, add=sh).clone()


@pytest.mark.parametrize("gt,dt,st,E,FF,NE,TK,T", [
    (IQ2_S, Q4_K, Q8_0, 7168, 2048, 32, 8, 8),    # configs[2]'s types and shape (fewer experts resident)
    (IQ2_S, IQ2_S, Q8_0, 7168, 2048, 16, 8, 1),   # one token: the down kernel that rounds h itself waits for the join
    (Q4_K, Q4_K, Q4_K, 4096, 1024, 8, 2, 3),
])
def test_layer_with_shared_expert_is_the_two_calls(lib, gt, dt, st, E, FF, NE, TK, T):
    w = build(lib, gt, dt, st, E, FF, NE, TK, T, 500 + T)
    for rep in range(3):   # call after call: the second stream's buffers are reused without a host synchronisation
        logits, x, add = inputs(E, NE, T, 510 + rep)
        use_add = add if rep != 1 else None
        got = w["layer"].forward(w["table"], logits, x, add=use_add, shared=w["dense"], shared_limit=7.0).clone()
        ids = w["layer"].ids[:T].clone()
        want = two_calls(w, logits, x, use_add, 7.0)
        torch.cuda.synchronize()
        assert torch.equal(ids, w["layer"].ids[:T])
        assert torch.equal(got, want), rep
        assert float(got.abs().max()) > 0


def test_against_the_cpu_path(lib, oracle):
    gt, dt, st, E, FF, NE, TK, T = IQ2_S, Q4_K, Q8_0, 7168, 2048, 32, 8, 4
    w = build(lib, gt, dt, st, E, FF, NE, TK, T, 530)
    logits, x, _ = inputs(E, NE, T, 531)
    out = w["layer"].forward(w["table"], logits, x, shared=w["dense"]).cpu().numpy()

    class Blobs:
        def __getitem__(self, e):
            return w["view"][e].cpu().numpy()
    ids, _, want = oracle_layer(oracle, gt, dt, Blobs(), TK, E, FF, logits.cpu().numpy(), x.cpu().numpy())
    assert np.array_equal(w["layer"].ids[:T].cpu().numpy(), ids)
    shb, sg = w["sh"].cpu().numpy(), w["sg"]
    for t in range(T):
        s = oracle.expert(st, st, shb, shb[sg.up_off:], shb[sg.down_off:], E, FF, x[t:t + 1].cpu().numpy())[0]
        assert rel_l2(out[t], want[t] + s) <= 1e-3, (t, rel_l2(out[t], want[t] + s))


def test_replayed_from_a_graph(lib):
    """Captured once, replayed with eager work and synchronisations in between, on inputs that change between replays."""
    gt, dt, st, E, FF, NE, TK, T = IQ2_S, Q4_K, Q8_0, 7168, 2048, 32, 8, 8
    w = build(lib, gt, dt, st, E, FF, NE, TK, T, 540)
    logits, x, _ = inputs(E, NE, T, 541)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=s)   # (warm: nothing is set up under capture)
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=torch.cuda.current_stream())
    for rep in range(4):
        l2, x2, _ = inputs(E, NE, T, 550 + rep)
        logits.copy_(l2)
        x.copy_(x2)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = w["layer"].out[:T].clone()
        want = two_calls(w, logits, x, None, float("inf"))
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_refusals_leave_the_stream_usable(lib):
    gt, dt, st, E, FF, NE, TK, T = Q4_K, Q4_K, Q4_K, 4096, 1024, 8, 2, 3
    w = build(lib, gt, dt, st, E, FF, NE, TK, T, 560)
    logits, x, _ = inputs(E, NE, T, 561)
    other = lib.DenseExpert(st, st, E, FF, T + 1, w["sh_packed"].data_ptr(), packing=lib.PACK_STREAM)
    with pytest.raises(AssertionError):
        w["layer"].forward(w["table"], logits, x, shared=other)
    a = other.args
    import ctypes as C
    L = lib.load()
    rc = L.maya_moe_layer_decode_shared(C.byref(w["layer"].layout), w["table"].data_ptr(), NE, TK, None, logits.data_ptr(), x.data_ptr(), 0, T,
                                        float("inf"), C.byref(a), w["layer"].ids.data_ptr(), w["layer"].weights.data_ptr(),
                                        w["layer"].out.data_ptr(), w["layer"].ws.data_ptr(), w["layer"].ws_bytes, None)
    assert rc != 0 and b"tokens" in L.maya_last_error()
    # a routed layer that is refused (k above the number of experts): asked before the fork, so the status is > 0, nothing
    # was launched on either stream, and the next call works
    rc = L.maya_moe_layer_decode_shared(C.byref(w["layer"].layout), w["table"].data_ptr(), 1, TK, None, logits.data_ptr(), x.data_ptr(), 0, T,
                                        float("inf"), C.byref(w["dense"].args), w["layer"].ids.data_ptr(), w["layer"].weights.data_ptr(),
                                        w["layer"].out.data_ptr(), w["layer"].ws.data_ptr(), w["layer"].ws_bytes, None)
    assert rc > 0 and b"n_expert" in L.maya_last_error()
    torch.cuda.synchronize()
    got = w["layer"].forward(w["table"], logits, x, shared=w["dense"]).clone()
    want = two_calls(w, logits, x, None, float("inf"))
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_another_stream_is_refused_while_the_side_stream_is_inside_a_capture(lib):
    """The device's one side stream belongs to an open capture until that capture ends: a call from another stream in between
    gets MAYA_E_BUSY and launches nothing, the capture stays valid (the same capture may call again), and its graph replays
    with the right bits."""
    import ctypes as C
    gt, dt, st, E, FF, NE, TK, T = IQ2_S, Q4_K, Q8_0, 4096, 2048, 16, 4, 2
    w = build(lib, gt, dt, st, E, FF, NE, TK, T, 570)
    logits, x, _ = inputs(E, NE, T, 571)
    L = lib.load()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s1):
        w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=s1)
    s1.synchronize()
    out2 = torch.zeros_like(w["layer"].out)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s1):
        w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=torch.cuda.current_stream())
        rc = L.maya_moe_layer_decode_shared(C.byref(w["layer"].layout), w["table"].data_ptr(), NE, TK, None, logits.data_ptr(), x.data_ptr(),
                                            0, T, float("inf"), C.byref(w["dense"].args), w["layer"].ids.data_ptr(),
                                            w["layer"].weights.data_ptr(), out2.data_ptr(), w["layer"].ws.data_ptr(), w["layer"].ws_bytes,
                                            C.c_void_p(s2.cuda_stream))
        busy_msg = L.maya_last_error()
        w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=torch.cuda.current_stream())   # the same capture again
    assert rc == 5 and b"capture" in busy_msg
    s2.synchronize()
    assert not out2.any()   # nothing ran for the refused call
    l2, x2, _ = inputs(E, NE, T, 572)
    logits.copy_(l2)
    x.copy_(x2)
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    got = w["layer"].out[:T].clone()
    want = two_calls(w, logits, x, None, float("inf"))
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # after the capture has ended the other stream is served
    with torch.cuda.stream(s2):
        got2 = w["layer"].forward(w["table"], logits, x, shared=w["dense"], stream=s2).clone()
    s2.synchronize()
    assert torch.equal(got2, want)

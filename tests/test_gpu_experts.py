"""GPU parity, expert rows: the HIP layer against the CPU checker (the reference's CPU expert path in the ggml
contract) on the same seeded inputs.  Bar: top-k ids bit-exact, expert outputs within 1e-3 relative L2."""
import numpy as np
import pytest
import torch

from gpu_util import dev, make_experts, oracle_layer, rel_l2
import synth

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


def run_layer(lib, gate_type, down_type, blobs, k, n_embd, n_ff, logits, x, limit=float("inf"), up_type=None,
              misalign=0, add=None, resident=None, packing=0, router=None):
    gguf_layout, _ = lib.layout(gate_type, down_type, n_embd, n_ff, up_type)
    store = lib.ExpertStore(blobs, misalign=misalign, pack_layout=gguf_layout if packing else None)
    table = store.table
    if resident is not None:
        table = table.clone()
        mask = torch.ones(len(blobs), dtype=torch.bool)
        mask[list(resident)] = False
        table[mask.cuda()] = 0
    layer = lib.MoeLayer(gate_type, down_type, n_embd, n_ff, len(blobs), k, max_tokens=x.shape[0], up_type=up_type,
                         packing=packing)
    out = layer.forward(table, dev(logits), x if torch.is_tensor(x) else dev(x), limit=limit,
                        add=None if add is None else dev(add), router=router)
    torch.cuda.synchronize()
    return layer.ids.cpu().numpy(), layer.weights.cpu().numpy(), out.cpu().numpy(), store


CASES = [
    # gate/up type, down type, n_embd, n_ff, experts, k, tokens
    (22, 22, 1024, 512, 16, 4, 1),
    (12, 12, 1024, 512, 16, 4, 1),
    (8, 8, 512, 256, 8, 2, 1),
    (19, 19, 1024, 512, 8, 4, 1),
    (29, 29, 1024, 512, 8, 4, 1),
    (22, 12, 1024, 512, 16, 8, 1),
    (22, 22, 1024, 512, 16, 8, 4),
    (22, 12, 1024, 768, 12, 8, 8),
    (12, 12, 768, 512, 6, 4, 3),
    (29, 22, 512, 512, 6, 4, 5),
    # the single-token streaming kernels (n_embd and n_ff multiples of 1024, n_embd a multiple of 14)
    (22, 22, 7168, 1024, 10, 8, 1),
    (22, 22, 7168, 2048, 9, 8, 1),
    (22, 22, 14336, 1024, 4, 3, 1),
    # the position-mapped kernels on several tokens' entries, and the Q4_K ones (stream packing; n_ff 2048 for down)
    (22, 22, 4096, 2048, 12, 8, 5),
    (12, 12, 4096, 2048, 6, 4, 1),
    (12, 12, 7168, 2048, 5, 3, 4),
    (22, 12, 6144, 2048, 9, 8, 3),
    (12, 22, 8192, 2048, 4, 2, 2),
    # stream-packed Q8_0 (the shared expert's format): one token, a window, mixed with other types
    (8, 8, 4096, 2048, 5, 3, 1),
    (8, 8, 7168, 2048, 3, 2, 7),
    (8, 12, 6144, 2048, 4, 2, 3),
    (22, 8, 4096, 2048, 6, 4, 2),
    # stream-packed IQ1_S on the position-mapped kernels: one token, a window, mixed with IQ2_S
    (19, 19, 4096, 2048, 6, 4, 1),
    (19, 19, 7168, 2048, 9, 8, 3),
    (19, 22, 6144, 2048, 4, 2, 2),
    (22, 19, 4096, 2048, 4, 3, 2),
    # and IQ1_M
    (29, 29, 4096, 2048, 6, 4, 1),
    (29, 29, 7168, 2048, 9, 8, 3),
    (29, 19, 6144, 2048, 4, 2, 2),
    (12, 29, 8192, 2048, 4, 3, 2),
    # IQ2_XXS (the general kernels): one token, a window, mixed with IQ2_S either side
    (16, 16, 1024, 512, 8, 4, 1),
    (16, 16, 7168, 2048, 9, 8, 3),
    (16, 22, 4096, 2048, 6, 4, 2),
    (22, 16, 2048, 1024, 4, 2, 5),
    # other expert shapes on the position-mapped kernels: rows of 2048 / 3072 / 5120 values, n_ff 1024 / 1536 (the down
    # rows then leave lanes of their wave idle)
    (22, 22, 5120, 1536, 6, 4, 1),
    (22, 22, 2048, 1024, 6, 4, 3),
    (12, 12, 3072, 1536, 5, 3, 2),
    (22, 12, 5120, 1024, 5, 3, 1),
    (12, 22, 2048, 1536, 4, 2, 2),
    (8, 8, 5120, 1536, 3, 2, 1),
    (8, 8, 3072, 1024, 3, 1, 6),
    (8, 22, 2048, 1536, 4, 2, 3),
    (19, 19, 5120, 1536, 4, 3, 1),
    (29, 29, 3072, 1024, 4, 2, 2),
    (19, 29, 2048, 1536, 3, 2, 3),
    # IQ2_S down rows with n_embd / 256 rows a workgroup (24, 28, 32; 28 has an odd number of row quads), windows too
    (22, 22, 6144, 2048, 5, 3, 2),
    (22, 22, 7168, 2048, 9, 8, 4),
    (22, 22, 8192, 1536, 4, 4, 3),
]


@pytest.mark.parametrize("packing", (0, 1))
@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt", CASES)
def test_layer_matches_cpu_path(lib, oracle, gt, dt, n_embd, n_ff, ne, k, nt, packing):
    seed = gt * 1000 + dt * 10 + nt
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, seed)
    rng = np.random.default_rng(seed + 1)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    print("case", gt, dt, n_embd, n_ff, ne, k, nt, packing, flush=True)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, packing=packing)
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, x)
    assert np.array_equal(ids, wi)
    for t in range(nt):
        assert rel_l2(out[t], wout[t]) <= TOL, (t, rel_l2(out[t], wout[t]))


def encoded_q4k_expert(oracle, n_embd, n_ff, seed):
    """One expert as BASELINE's single-expert configuration states it: gate / up [n_ff x n_embd] and down [n_embd x n_ff]
    drawn from N(0, 0.02) in F32 and quantized to Q4_K (the checker's own encoder: the reference never quantizes weights)."""
    rng = np.random.default_rng(seed)
    return np.concatenate([oracle.encode_q4k((rng.standard_normal(rows * cols) * 0.02).astype(np.float32))
                           for rows, cols in ((n_ff, n_embd), (n_ff, n_embd), (n_embd, n_ff))])


@pytest.mark.parametrize("ne,k,nt,packing", ((1, 1, 1, 1), (2, 2, 2, 1), (1, 1, 1, 0), (2, 1, 2, 1)))
def test_single_expert_glu_q4k_from_gaussian_weights(lib, oracle, ne, k, nt, packing):
    """BASELINE's first configuration at its full size: one Q4_K expert GLU of 7168 x 2048 on one F32 token (and two experts
    on two tokens).  One or two plan slots on few tokens select the kernels' smallest tiles - 8 gate/up row pairs and 8
    down rows a workgroup - which no other case reaches."""
    n_embd, n_ff = 7168, 2048
    blobs = [encoded_q4k_expert(oracle, n_embd, n_ff, 500 + e) for e in range(ne)]
    rng = np.random.default_rng(510 + nt)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    ids, w, out, _ = run_layer(lib, 12, 12, blobs, k, n_embd, n_ff, logits, x, packing=packing)
    wi, ww, wout = oracle_layer(oracle, 12, 12, blobs, k, n_embd, n_ff, logits, x)
    assert np.array_equal(ids, wi)
    for t in range(nt):
        assert np.abs(wout[t]).max() > 0
        assert rel_l2(out[t], wout[t]) <= TOL, (t, rel_l2(out[t], wout[t]))
    if ne == 1:
        # out = down(silu(gate x) * (up x)) with weight 1: the expert alone
        want = oracle.expert(12, 12, blobs[0], blobs[0][n_ff * (n_embd // 256) * 144:], blobs[0][2 * n_ff * (n_embd // 256) * 144:],
                             n_embd, n_ff, x)
        assert rel_l2(out[0], want[0]) <= TOL


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt,packing,norm", (
    (22, 22, 7168, 2048, 9, 8, 1, 1, 1), (22, 22, 1024, 512, 16, 4, 3, 0, 2), (12, 12, 4096, 2048, 6, 4, 2, 1, 1),
    (8, 8, 512, 256, 8, 2, 1, 0, 0), (22, 12, 1024, 768, 300, 8, 2, 0, 1)))
def test_layer_with_the_sigmoid_router(lib, oracle, gt, dt, n_embd, n_ff, ne, k, nt, packing, norm):
    """The layer's head routes as router_sigmoid / moe_route do (a selection bias, a scaling factor): ids bit-exact, weights
    1e-5, the layer against the CPU path's experts combined with those weights."""
    seed = gt * 1000 + dt * 10 + nt + 7
    blobs = make_experts(gt, dt, n_embd, n_ff, min(ne, 12), seed)
    blobs = [blobs[i % len(blobs)] for i in range(ne)]   # (many experts: the same few blobs again)
    rng = np.random.default_rng(seed + 1)
    logits = (rng.standard_normal((nt, ne)) * 2).astype(np.float32)
    bias = (rng.standard_normal(ne) * 0.1).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    bias_d = dev(bias)
    router = lib.Router(lib.ROUTER_SIGMOID, norm, bias_d.data_ptr(), 2.5)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, packing=packing, router=router)
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, x,
                                route=lambda l, kk: oracle.router_sigmoid(l, bias, kk, 2.5, norm))
    assert np.array_equal(ids, wi) and np.max(np.abs(w - ww)) < 1e-5
    for t in range(nt):
        assert rel_l2(out[t], wout[t]) <= TOL, (t, rel_l2(out[t], wout[t]))


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt,packing", (
    (22, 22, 7168, 2048, 9, 8, 1, 1), (22, 22, 1024, 512, 16, 4, 3, 0), (12, 12, 4096, 2048, 6, 4, 3, 1), (22, 12, 1024, 768, 300, 8, 2, 0)))
def test_layer_refuses_a_token_with_non_finite_logits(lib, gt, dt, n_embd, n_ff, ne, k, nt, packing):
    """A token whose router row holds a NaN gets no routes: ids -1, weights 0, and its output is the added part alone; the
    other tokens' outputs are bit for bit what the layer gives without the bad row's NaN."""
    seed = gt * 100 + dt + nt + 3
    blobs = make_experts(gt, dt, n_embd, n_ff, min(ne, 12), seed)
    blobs = [blobs[i % len(blobs)] for i in range(ne)]
    rng = np.random.default_rng(seed + 1)
    logits = (rng.standard_normal((nt, ne)) * 2).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    add = rng.standard_normal((nt, n_embd)).astype(np.float32)
    router = lib.Router(lib.ROUTER_SIGMOID, 1, 0, 2.5)
    wi, ww, wout, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, packing=packing, router=router, add=add)
    bad = nt // 2
    logits[bad, ne // 2] = np.nan
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, packing=packing, router=router, add=add)
    assert np.all(ids[bad] == -1) and np.all(w[bad] == 0.0) and np.array_equal(out[bad], add[bad])
    for t in range(nt):
        if t != bad:
            assert np.array_equal(ids[t], wi[t]) and np.array_equal(w[t], ww[t]) and np.array_equal(out[t], wout[t])


def test_mixed_gate_up_types(lib, oracle):
    gt, ut, dt, n_embd, n_ff, ne, k = 22, 29, 22, 512, 256, 6, 3
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 77, up_type=ut)
    rng = np.random.default_rng(78)
    logits = rng.standard_normal((2, ne)).astype(np.float32)
    x = rng.standard_normal((2, n_embd)).astype(np.float32)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, up_type=ut)
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, x, up_type=ut)
    assert np.array_equal(ids, wi)
    assert rel_l2(out, wout) <= TOL


def test_two_byte_aligned_blobs_clamp_and_add(lib, oracle):
    """Blobs at a +2 byte offset (GGUF slices are only 2-byte aligned), GLM's clamped SwiGLU, a shared-expert part added."""
    gt, dt, n_embd, n_ff, ne, k, nt = 22, 12, 1024, 512, 8, 4, 2
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 91)
    rng = np.random.default_rng(92)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = (rng.standard_normal((nt, n_embd)) * 3).astype(np.float32)
    add = rng.standard_normal((nt, n_embd)).astype(np.float32)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, limit=0.75, misalign=2, add=add)
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, x, limit=0.75)
    assert np.array_equal(ids, wi)
    assert rel_l2(out, wout + add) <= TOL


def test_null_plan_slots_are_left_out(lib, oracle):
    gt, dt, n_embd, n_ff, ne, k, nt = 22, 22, 512, 256, 8, 4, 3
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 55)
    rng = np.random.default_rng(56)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    resident = {0, 2, 3, 5, 6}
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, resident=resident)
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, x, skip=set(range(ne)) - resident)
    assert np.array_equal(ids, wi)
    assert rel_l2(out, wout) <= TOL


def test_zero_input_and_bf16_input(lib, oracle):
    gt, dt, n_embd, n_ff, ne, k = 22, 22, 512, 256, 4, 2
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 60)
    rng = np.random.default_rng(61)
    logits = rng.standard_normal((1, ne)).astype(np.float32)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, np.zeros((1, n_embd), dtype=np.float32))
    assert not out.any()
    xb = torch.from_numpy(rng.standard_normal((1, n_embd)).astype(np.float32)).to(torch.bfloat16)
    ids, w, out, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, xb.cuda())
    wi, ww, wout = oracle_layer(oracle, gt, dt, blobs, k, n_embd, n_ff, logits, xb.to(torch.float32).numpy())
    assert np.array_equal(ids, wi) and rel_l2(out, wout) <= TOL


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,ne,k,nt", ((22, 12, 1024, 512, 10, 4, 6), (22, 22, 7168, 1024, 6, 4, 3), (22, 12, 4096, 2048, 7, 4, 4), (8, 8, 4096, 2048, 1, 1, 8),
                                                     (19, 19, 4096, 2048, 5, 4, 4), (29, 29, 4096, 2048, 5, 4, 3)))
def test_window_rows_equal_token_rows(lib, gt, dt, n_embd, n_ff, ne, k, nt):
    """A verify window's rows carry the bits its tokens give one at a time (the reference's window contract), in either
    row packing."""
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 33)
    rng = np.random.default_rng(34)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    _, _, win, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x)
    _, _, winp, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits, x, packing=1)
    for t in range(nt):
        _, _, one, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits[t:t + 1], x[t:t + 1])
        assert np.array_equal(win[t].view(np.uint32), one[0].view(np.uint32)), t
        _, _, onep, _ = run_layer(lib, gt, dt, blobs, k, n_embd, n_ff, logits[t:t + 1], x[t:t + 1], packing=1)
        assert np.array_equal(winp[t].view(np.uint32), onep[0].view(np.uint32)), t
        # the stream packing's kernels sum a row's sub-blocks in another order than the GGUF packing's: same integers,
        # float sums that differ in their last bits (and, rarely, one Q8_K code of h): held to the parity bar
        assert rel_l2(onep[0], win[t]) <= TOL, t


def test_unsupported_and_bad_shapes_fail_cleanly(lib):
    import ctypes as C
    L = lib.load()
    l = lib.Layout()
    assert L.maya_moe_layout_init(C.byref(l), 22, 22, 22, 1000, 512) == 0      # not whole blocks
    assert L.maya_moe_layout_init(C.byref(l), 22, 8, 22, 1024, 512) == 0        # gate/up activation formats differ
    assert L.maya_moe_layout_init(C.byref(l), 99, 99, 99, 1024, 512) == 0
    assert L.maya_moe_supported(22) == 1 and L.maya_moe_supported(10) == 0
    with pytest.raises(lib.MayaError):
        lib.route_topk(torch.zeros((1, 4), device="cuda"), 8)


@pytest.mark.parametrize("dt", (22, 12, 19, 29))
def test_down_rounds_h_itself_like_the_quantizer(lib, dt):
    """The stream-packed IQ2_S / Q4_K / IQ1_S / IQ1_M down kernels given no rounded h round it in their prologue: the same Q8_K codes as
    maya_quant_act (an all-zero block, equal magnitudes of both signs inside a lane's values, across lanes, and where
    the lower index sits in the higher lane), so the same output bits."""
    import ctypes as C
    L = lib.load()
    n_embd, n_ff, ne, k = 1024, 2048, 8, 8
    blobs = make_experts(22, dt, n_embd, n_ff, ne, 77)
    gguf, _ = lib.layout(22, dt, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf)
    rng = np.random.default_rng(3)
    h = rng.standard_normal((k, n_ff)).astype(np.float32)
    h[0, 256:512] = 0.0
    h[1, 512:768] = 0.5
    h[2, 100], h[2, 200] = -7.0, 7.0          # the first (negative) maximum sets the sign of the scale
    h[3, 900], h[3, 300] = 9.0, -9.0
    h[4, 300], h[4, 310] = 9.0, -9.0          # both in one run of 32
    h[4, 600], h[4, 590] = 8.0, -8.0
    h[5, 256 + 44], h[5, 256 + 20] = -5.0, 5.0
    h[5, 512 + 20], h[5, 512 + 44] = -5.0, 5.0
    h[6, 1024:1280] = -0.0
    h[7, 1030] = -6.5                         # the largest magnitude of its block, and negative: no tie
    h[7, 1100] = 6.25
    h_d = dev(h)
    hq = lib.quant_act(22, h_d)           # Q8_K serves both down types
    w = dev(rng.uniform(0.05, 0.3, k).astype(np.float32))
    plan = store.table.clone()
    outs = []
    for given in (True, False):
        a = lib.Args()
        a.layout = lib.copy_layout(gguf, lib.PACK_STREAM)
        a.n_tokens, a.k = 1, k
        a.plan_ptr, a.plan_w = plan.data_ptr(), w.data_ptr()
        a.limit = float("inf")
        a.h = h_d.data_ptr()
        part = torch.zeros((k, n_embd), device="cuda")
        out = torch.zeros((1, n_embd), device="cuda")
        a.out = out.data_ptr()
        if given:
            a.hq, a.part = hq.c(), part.data_ptr()
        assert L.maya_moe_down_rounds_h(C.byref(a)) == 1
        lib.check(L.maya_moe_down(C.byref(a), lib._stream()))
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    assert np.abs(outs[0]).max() > 0


@pytest.mark.parametrize("gt,dt,n_embd,n_ff,k,nt,packing", ((22, 22, 4096, 2048, 4, 1, 1), (12, 12, 1024, 512, 3, 2, 0), (8, 8, 4096, 2048, 2, 3, 1)))
def test_down_adds_the_flagged_part_and_then_the_unconditional_one(lib, gt, dt, n_embd, n_ff, k, nt, packing):
    """out = sum_i w_i part_i [+ add when *add_flag] + add2: the order of glmf::moe_down's cpu_part and sh_out
    (include/strata/kernels/glm_fast.hpp:499-501), each sum rounded."""
    import ctypes as C
    L = lib.load()
    ne = k + 1
    blobs = make_experts(gt, dt, n_embd, n_ff, ne, 41)
    gguf, _ = lib.layout(gt, dt, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf if packing else None)
    rng = np.random.default_rng(42)
    h = dev(rng.standard_normal((nt * k, n_ff)).astype(np.float32))
    hq = lib.quant_act(dt, h)
    ids = torch.from_numpy(np.stack([rng.permutation(ne)[:k] for _ in range(nt)]).astype(np.int32)).cuda()
    plan = lib.plan(ids.view(-1), store.table)
    w = dev(rng.uniform(0.05, 0.3, nt * k).astype(np.float32))
    add = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    add2 = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    outs = {}
    for name, flag, second in (("plain", None, False), ("off", 0, False), ("on", 1, False), ("both", 1, True), ("second", None, True)):
        a = lib.Args()
        a.layout = lib.copy_layout(gguf, packing)
        a.n_tokens, a.k = nt, k
        a.plan_ptr, a.plan_w = plan.data_ptr(), w.data_ptr()
        a.limit = float("inf")
        a.h = h.data_ptr()
        a.hq = hq.c()
        part = torch.zeros((nt * k, n_embd), device="cuda")
        out = torch.zeros((nt, n_embd), device="cuda")
        a.part, a.out = part.data_ptr(), out.data_ptr()
        fl = None
        if flag is not None:
            fl = torch.tensor([flag], dtype=torch.int32, device="cuda")
            a.add, a.add_flag = add.data_ptr(), fl.data_ptr()
        if second:
            a.add2 = add2.data_ptr()
        lib.check(L.maya_moe_down(C.byref(a), lib._stream()))
        torch.cuda.synchronize()
        outs[name] = out.clone()
    assert torch.equal(outs["off"], outs["plain"]) and float(outs["plain"].abs().max()) > 0
    assert torch.equal(outs["on"], outs["plain"] + add)
    assert torch.equal(outs["both"], (outs["plain"] + add) + add2)
    assert torch.equal(outs["second"], outs["plain"] + add2)


def test_layers_take_tokens_that_are_already_routed(lib, oracle):
    """logits NULL: ids / weights are inputs.  The sigmoid router's ids and weights through the decode layer, the prompt-chunk
    layer and (in test_gpu_exl3) the EXL3 layer give what the routed layer gives."""
    from maya_amd import prefill
    gt, n_embd, n_ff, ne, k, nt = 12, 1024, 512, 10, 3, 6
    blobs = make_experts(gt, gt, n_embd, n_ff, ne, 321)
    rng = np.random.default_rng(322)
    logits = (rng.standard_normal((nt, ne)) * 2).astype(np.float32)
    bias = (rng.standard_normal(ne) * 0.1).astype(np.float32)
    x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    bias_d = dev(bias)
    ids, w = lib.route_sigmoid(dev(logits), bias_d, k, 2.5, 1)
    store = lib.ExpertStore(blobs)
    layer = lib.MoeLayer(gt, gt, n_embd, n_ff, ne, k, max_tokens=nt)
    a = layer.forward(store.table, dev(logits), x, router=lib.Router(lib.ROUTER_SIGMOID, 1, bias_d.data_ptr(), 2.5)).clone()
    b = layer.forward(store.table, None, x, routed=(ids, w)).clone()
    torch.cuda.synchronize()
    assert torch.equal(layer.ids, ids) and rel_l2(b.cpu().numpy(), a.cpu().numpy()) <= 1e-6 and float(a.abs().max()) > 0
    # the prompt-chunk layer on the same routing: the same tokens' outputs (another summation order)
    layout, _ = lib.layout(gt, gt, n_embd, n_ff)
    pl = prefill.PrefillLayer(layout, ne, k, nt, out_dtype=torch.float32)
    c = pl.forward(store.table, None, x, limit=0.0, routed=(ids, w))
    torch.cuda.synchronize()
    for t in range(nt):
        assert rel_l2(c[t].cpu().numpy(), a[t].cpu().numpy()) <= 1e-4, t


def test_dense_expert_through_the_stage_calls(lib, oracle):
    """The expert every token takes, with a static plan and no routing launch: the same rows as a k = 1 layer over one expert."""
    t, n_embd, n_ff, nt = 8, 4096, 2048, 5
    blobs = make_experts(t, t, n_embd, n_ff, 1, 77)
    gguf, _ = lib.layout(t, t, n_embd, n_ff)
    store = lib.ExpertStore(blobs, pack_layout=gguf)
    rng = np.random.default_rng(78)
    x = dev(rng.standard_normal((nt, n_embd)).astype(np.float32))
    dense = lib.DenseExpert(t, t, n_embd, n_ff, nt, int(store.table[0].item()), packing=lib.PACK_STREAM)
    a = dense.forward(x, limit=6.0).clone()
    layer = lib.MoeLayer(t, t, n_embd, n_ff, 1, 1, max_tokens=nt, packing=lib.PACK_STREAM)
    b = layer.forward(store.table, dev(np.zeros((nt, 1), dtype=np.float32)), x, limit=6.0)
    torch.cuda.synchronize()
    assert torch.equal(a, b) and float(a.abs().max()) > 0
    want = oracle.expert(t, t, blobs[0], blobs[0][gguf.up_off:], blobs[0][gguf.down_off:], n_embd, n_ff, x.cpu().numpy(), 6.0)
    for i in range(nt):
        assert rel_l2(a[i].cpu().numpy(), want[i]) <= TOL, i

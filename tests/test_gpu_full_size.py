"""GPU parity at the BASELINE configurations' full sizes (256 experts of 7168 x 2048 resident: gigabytes of synthetic
blobs made on the device).  The CPU checker cannot run a whole step at these sizes in seconds, so each test checks the
routing in full and the layer on the tokens it samples (their routed experts' blobs are pulled to the host one by one),
plus a property that holds at any size: a prompt chunk's token row is the decode layer's row for that token."""
import numpy as np
import pytest
import torch

from gpu_util import oracle_layer, rel_l2
import bench_workloads as workloads
from bench_workloads import zipf_bias

pytestmark = pytest.mark.gpu
TOL = 1e-3
E, FF, NE, TK = 7168, 2048, 256, 8
IQ2_S, Q4_K, Q8_0 = 22, 12, 8
FIELDS = {IQ2_S: (82, {0: (2e-3, 6e-3)}), Q4_K: (144, {0: (2e-4, 6e-4), 2: (2e-4, 6e-4)}), Q8_0: (34, {0: (1e-4, 4e-4)})}


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    return L


class DeviceBlobs:
    """Expert e's GGUF blob, pulled from the device pool when the checker asks for it."""

    def __init__(self, view):
        self.view = view

    def __getitem__(self, e):
        return self.view[e].cpu().numpy()


def make_pool(lib, gt, dt, n_expert, seed):
    """GGUF blobs [gate | up | down] of random blocks on the device, and the same experts in the stream packing."""
    gguf, bb = lib.layout(gt, dt, E, FF)
    pool = torch.empty(n_expert * bb, dtype=torch.uint8, device="cuda")
    view = pool.view(n_expert, bb)
    view[:, :gguf.down_off] = workloads.random_blocks(n_expert * gguf.down_off, *FIELDS[gt], seed).view(n_expert, -1)
    view[:, gguf.down_off:] = workloads.random_blocks(n_expert * (bb - gguf.down_off), *FIELDS[dt], seed + 1).view(n_expert, -1)
    packed = torch.empty_like(pool)
    for e in range(n_expert):
        lib.repack(gguf, view[e], packed[e * bb:(e + 1) * bb])
    torch.cuda.synchronize()
    table = torch.tensor([packed.data_ptr() + e * bb for e in range(n_expert)], dtype=torch.int64, device="cuda")
    return gguf, bb, view, packed, table


def test_decode_layer_256_iq2s_experts(lib, oracle):
    """configs[1]: one token (bf16), 256 resident IQ2_S experts, top-8."""
    gguf, bb, view, packed, table = make_pool(lib, IQ2_S, IQ2_S, NE, 101)
    layer = lib.MoeLayer(IQ2_S, IQ2_S, E, FF, NE, TK, max_tokens=1, packing=lib.PACK_STREAM)
    rng = np.random.default_rng(102)
    for step in range(3):
        logits = rng.standard_normal((1, NE)).astype(np.float32)
        x = torch.from_numpy(rng.standard_normal((1, E)).astype(np.float32)).to(torch.bfloat16)
        out = layer.forward(table, torch.from_numpy(logits).cuda(), x.cuda()).cpu().numpy()
        ids, w, want = oracle_layer(oracle, IQ2_S, IQ2_S, DeviceBlobs(view), TK, E, FF, logits, x.to(torch.float32).numpy())
        assert np.array_equal(layer.ids[:1].cpu().numpy(), ids) and np.max(np.abs(layer.weights[:1].cpu().numpy() - w)) < 1e-5
        assert rel_l2(out[0], want[0]) <= TOL


def test_eight_tokens_mixed_experts_and_the_shared_expert(lib, oracle):
    """configs[2]: 8 tokens, 256 experts with IQ2_S gate/up and Q4_K down, top-8, plus a Q8_0 shared expert every token
    takes (its rows are the layer's added part)."""
    T = 8
    gguf, bb, view, packed, table = make_pool(lib, IQ2_S, Q4_K, NE, 201)
    sg, sbb = lib.layout(Q8_0, Q8_0, E, FF)
    sh = workloads.random_blocks(sbb, *FIELDS[Q8_0], 203)
    sh_packed = torch.empty_like(sh)
    lib.repack(sg, sh, sh_packed)
    layer = lib.MoeLayer(IQ2_S, Q4_K, E, FF, NE, TK, max_tokens=T, packing=lib.PACK_STREAM)
    dense = lib.DenseExpert(Q8_0, Q8_0, E, FF, T, sh_packed.data_ptr(), packing=lib.PACK_STREAM)
    rng = np.random.default_rng(204)
    logits = rng.standard_normal((T, NE)).astype(np.float32)
    x = rng.standard_normal((T, E)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    shared = dense.forward(xd)
    out = layer.forward(table, torch.from_numpy(logits).cuda(), xd, add=shared).cpu().numpy()
    ids, w, want = oracle_layer(oracle, IQ2_S, Q4_K, DeviceBlobs(view), TK, E, FF, logits, x)
    assert np.array_equal(layer.ids[:T].cpu().numpy(), ids)
    shb = sh.cpu().numpy()
    for t in range(T):
        s = oracle.expert(Q8_0, Q8_0, shb, shb[sg.up_off:], shb[sg.down_off:], E, FF, x[t:t + 1])[0]
        assert rel_l2(shared[t].cpu().numpy(), s) <= TOL
        assert rel_l2(out[t], want[t] + s) <= TOL, (t, rel_l2(out[t], want[t] + s))


def test_prompt_chunk_512_tokens_256_q4k_experts(lib, oracle):
    """configs[3]: 512 tokens, 256 Q4_K experts, top-8, Zipf(1.1)-skewed routing: the ids of every token, the chunk's rows of
    sampled tokens against the CPU path, and every sampled row against the decode layer's for that token alone."""
    from maya_amd import prefill
    import synth
    T = 512
    gguf, bb, view, packed, table = make_pool(lib, Q4_K, Q4_K, NE, 301)
    rng = np.random.default_rng(302)
    logits = (rng.standard_normal((T, NE)) + zipf_bias(NE)).astype(np.float32)
    x = rng.standard_normal((T, E)).astype(np.float32)
    xd, ld = torch.from_numpy(x).cuda(), torch.from_numpy(logits).cuda()
    chunk = prefill.PrefillLayer(lib.copy_layout(gguf, lib.PACK_STREAM), NE, TK, T, out_dtype=torch.float32)
    out = chunk.forward(table, ld, xd).cpu().numpy()
    ids, w = oracle.router_topk(logits, TK)
    assert np.array_equal(chunk.ids[:T].cpu().numpy(), ids)
    one = lib.MoeLayer(Q4_K, Q4_K, E, FF, NE, TK, max_tokens=1, packing=lib.PACK_STREAM)
    hot = int(np.bincount(ids.reshape(-1), minlength=NE).argmax())
    sample = [0, 1, 255, 511] + [int(t) for t in np.nonzero((ids == hot).any(axis=1))[0][:2]]   # (two rows of the busiest expert)
    for t in sample:
        _, _, want = oracle_layer(oracle, Q4_K, Q4_K, DeviceBlobs(view), TK, E, FF, logits[t:t + 1], x[t:t + 1])
        assert rel_l2(out[t], want[0]) <= TOL, (t, rel_l2(out[t], want[0]))
        dec = one.forward(table, ld[t:t + 1].contiguous(), xd[t:t + 1].contiguous()).cpu().numpy()
        assert rel_l2(out[t], dec[0]) <= 1e-5, (t, rel_l2(out[t], dec[0]))


def test_exl3_verify_window_160_experts(oracle):
    """configs[4]: 160 EXL3 experts (3 bits a weight, mul1), hidden 6144, intermediate 1536, top-8, a 4-token window:
    every token's ids, and the rows of sampled tokens against the checker's decode of the routed experts' own bytes."""
    from maya_amd import exl3
    from gpu_util import HostExpert
    E4, FF4, NE4, T = 6144, 1536, 160, 4
    l, bb, pool, view, table = workloads.exl3_pool(E4, FF4, NE4, 6)
    layer = exl3.Exl3Layer(l, NE4, TK, max_tokens=T)
    rng = np.random.default_rng(401)
    logits = rng.standard_normal((T, NE4)).astype(np.float32)
    x = rng.standard_normal((T, E4)).astype(np.float16).astype(np.float32)   # FP16 activations, handed over as F32
    out = layer.forward(table, torch.from_numpy(logits).cuda(), torch.from_numpy(x).cuda()).cpu().numpy()
    ids, w = oracle.router_topk(logits, TK)
    assert np.array_equal(layer.ids[:T].cpu().numpy(), ids)
    assert np.max(np.abs(layer.weights[:T].cpu().numpy() - w)) < 1e-5
    experts = {}
    for t in (0, 3):
        for e in ids[t]:
            if int(e) not in experts:
                experts[int(e)] = HostExpert(exl3, oracle, l, view[int(e), :bb].cpu().numpy())
        parts = [experts[int(e)].part(experts[int(e)].h(x[t], 0.0)) for e in ids[t]]
        want = oracle.combine(np.stack(parts), np.ascontiguousarray(w[t], dtype=np.float32))
        assert rel_l2(out[t], want) <= TOL, (t, rel_l2(out[t], want))

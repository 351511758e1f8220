"""EXL3 expert blobs built on the device from a model directory's pieces (maya_exl3_pack_experts): byte-equal to the host
concatenation in both piece orders, and a layer run from the packed blobs against the CPU checker on the same bytes."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
from gpu_util import dev, rel_l2  # noqa: E402
from test_exl3_files import PREFIX, synth_model  # noqa: E402
from test_gpu_exl3 import HostExpert, host_layer  # noqa: E402


@pytest.mark.parametrize("order", (0, 1))
@pytest.mark.parametrize("k2,cb", (((6, 6, 8), 2), ((4, 4, 4), 0), ((7, 7, 5), 2)))
def test_pack_equals_the_host_concatenation_and_runs_a_layer(tmp_path, oracle, order, k2, cb):
    from maya_amd import exl3, exl3_files as xf, lib
    exl3.load()
    n_embd, n_ff, ne, k, nt = 256, 128, 6, 3, 2
    d, _ = synth_model(tmp_path, layer=1, n_expert=ne, n_embd=n_embd, n_ff=n_ff, k2=k2, cb=cb, seed=11 + order)
    st = xf.SafeTensorsDir(d)
    L = xf.expert_layer(st, 1, PREFIX % 1, ne)
    store = xf.LayerStore(d, st.files, L, order=order)
    l, nbytes = store.layout, store.blob_bytes
    # the library's offsets are the documented ones: compact pieces, or the engine's 256-byte pieces with the trellis first
    if order == 0:
        ml, mb = exl3.make_layout(n_embd, n_ff, list(k2), cb)
        assert mb == nbytes and all(ml.suh[r] == l.suh[r] and ml.svh[r] == l.svh[r] and ml.trellis[r] == l.trellis[r] for r in range(3))
    else:
        assert all(l.trellis[r] % 256 == 0 and l.suh[r] % 256 == 0 and l.svh[r] % 256 == 0 and l.trellis[r] < l.suh[r] < l.svh[r] for r in range(3))
    pool = store.pool.cpu().numpy().reshape(ne, store.stride)
    blobs = [xf.host_blob(L, l, nbytes, st.mm, st.files, row) for row in L["rows"]]
    for e in range(ne):
        assert np.array_equal(pool[e, :nbytes], blobs[e]), e
    # the layer from the packed blobs against the checker's experts decoded from the same bytes
    rng = np.random.default_rng(7)
    logits = rng.standard_normal((nt, ne)).astype(np.float32)
    x = rng.standard_normal((nt, n_embd)).astype(np.float32)
    layer = exl3.Exl3Layer(l, ne, k, max_tokens=nt)
    out = layer.forward(store.table, dev(logits), dev(x)).cpu().numpy()
    torch.cuda.synchronize()
    ids, w = oracle.router_topk(logits, k)
    assert np.array_equal(layer.ids.cpu().numpy(), ids)
    experts = [HostExpert(exl3, oracle, l, b) for b in blobs]
    want, _ = host_layer(oracle, experts, ids, w, x, 0.0)
    for t in range(nt):
        assert rel_l2(out[t], want[t]) <= 1e-3, (t, rel_l2(out[t], want[t]))


def test_layout_init_refuses_what_the_kernels_do_not_take():
    from maya_amd import exl3
    from maya_amd.lib import MayaError
    exl3.load()
    with pytest.raises(MayaError):
        exl3.layout_init(200, 128, 6, 2)          # not whole 128-value blocks
    with pytest.raises(MayaError):
        exl3.layout_init(256, 128, 7, 1)          # K 3.5 without the mul1 codebook
    l, n = exl3.layout_init(256, 128, (6, 6, 8), 2, exl3.ORDER_TRELLIS_FIRST)
    assert n % 256 == 0 and n >= 2 * (256 * 128 * 6 // 16) + 128 * 256 * 8 // 16

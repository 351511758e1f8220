"""GPU parity, experts from files: a synthetic GGUF's stacked expert tensors -> blobs built on the device
(maya_moe_pack_experts) -> the routed layer, against the CPU checker run on the host concatenation of the same bytes;
the same layer loaded through a pack directory (native_experts.txt + experts.bin) gives bit-identical results."""
import numpy as np
import pytest
import torch

from gpu_util import dev, oracle_layer, rel_l2
from maya_amd import expert_files as ef
from test_expert_files import synth_model

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("spec,n_embd,n_ff,tokens", [((3, 22, 22, 22), 2048, 1024, 1), ((5, 22, 22, 12), 1024, 512, 3),
                                                     ((7, 12, 12, 8), 2048, 1024, 2)])
def test_layer_from_files(tmp_path, spec, n_embd, n_ff, tokens):
    import oracle_py as oracle
    from maya_amd import lib
    ne, k = 6, 4
    p = tmp_path / "m.gguf"
    synth_model(p, [spec], n_embd, n_ff, ne, seed=spec[0])
    g = ef.GgufFile(p)
    (L,) = ef.expert_layers(g)
    blobs = ef.layer_blobs(g, L)
    rng = np.random.default_rng(spec[0] + 100)
    logits = rng.standard_normal((tokens, ne)).astype(np.float32)
    x = rng.standard_normal((tokens, n_embd)).astype(np.float32)
    ids, w, want = oracle_layer(oracle, L.gate_type, L.down_type, list(blobs), k, n_embd, n_ff, logits, x, up_type=L.up_type)

    def run(store, packing):
        layer = lib.MoeLayer(L.gate_type, L.down_type, n_embd, n_ff, ne, k, max_tokens=tokens, up_type=L.up_type, packing=packing)
        out = layer.forward(store.table, dev(logits), dev(x))
        torch.cuda.synchronize()
        return layer.ids.cpu().numpy(), out.cpu().numpy()

    # straight from the GGUF, regrouped for the streaming kernels on the way in
    store = ef.LayerStore.from_gguf(g, L, packing=lib.PACK_STREAM)
    got_ids, got = run(store, lib.PACK_STREAM)
    assert np.array_equal(got_ids, ids)
    assert rel_l2(got, want) < 1e-3
    # the device-built GGUF-order blobs are the host concatenation, byte for byte
    plain = ef.LayerStore.from_gguf(g, L, packing=lib.PACK_GGUF)
    pad = (-plain.pool.data_ptr()) % 256
    dev_blobs = plain.pool[pad:pad + plain.stride * ne].view(ne, plain.stride)[:, :L.blob_bytes].cpu().numpy()
    assert np.array_equal(dev_blobs, blobs)
    # through a pack directory
    ef.write_index(tmp_path / "native_experts.txt", [L], p.name)
    ef.write_experts_bin(tmp_path / "experts.bin", g, [L])
    rows, n_expert, total = ef.read_index(tmp_path / "native_experts.txt", n_embd, n_ff)
    assert n_expert == ne and total == (tmp_path / "experts.bin").stat().st_size
    packed = ef.LayerStore.from_experts_bin(tmp_path / "experts.bin", rows[0], n_expert, n_embd, n_ff, packing=lib.PACK_STREAM)
    ids2, got2 = run(packed, lib.PACK_STREAM)
    assert np.array_equal(ids2, ids) and np.array_equal(got2, got)

"""Expert tensors on disk: the GGUF v3 directory, the expert blobs cut from a layer's three stacked tensors, and the
pack directory's index (native_experts.txt) under the reference parser's rules.  The reader is pinned on header bytes
laid out by hand from the format (not by this package's writer); the blobs against a per-expert concatenation; the
index against a row written out by hand in the reference's format (tools/iq_pack.py:470-489)."""
import struct

import numpy as np
import pytest

from maya_amd import expert_files as ef
import synth


def _s(x):
    return struct.pack("<Q", len(x)) + x.encode()


def test_reader_on_hand_laid_header(tmp_path):
    # magic, version 3, 1 tensor, 3 metadata entries: a u32, a string, an array of two strings
    h = struct.pack("<IIQQ", 0x46554747, 3, 1, 3)
    h += _s("general.alignment") + struct.pack("<II", 4, 64)
    h += _s("general.name") + struct.pack("<I", 8) + _s("tiny")
    h += _s("tok") + struct.pack("<IIQ", 9, 8, 2) + _s("a") + _s("bc")
    h += _s("blk.0.w") + struct.pack("<I", 2) + struct.pack("<2Q", 32, 3) + struct.pack("<IQ", 8, 128)
    pad = (-len(h)) % 64
    data = bytes(range(200)) + bytes(200)
    p = tmp_path / "m.gguf"
    p.write_bytes(h + b"\0" * pad + data)
    g = ef.GgufFile(p)
    assert g.version == 3 and g.alignment == 64 and g.data_start == len(h) + pad
    assert g.meta == {"general.alignment": 64, "general.name": "tiny", "tok": ["a", "bc"]}
    t = g.tensors["blk.0.w"]
    assert t.dims == (32, 3) and t.type_id == 8 and t.offset == g.data_start + 128 and t.nbytes == 3 * 34
    assert g.bytes_of("blk.0.w").tobytes() == data[128:128 + 102]


def test_reader_refusals(tmp_path):
    p = tmp_path / "x.gguf"
    p.write_bytes(struct.pack("<IIQQ", 0x46554746, 3, 0, 0))
    with pytest.raises(ValueError, match="not a GGUF file"):
        ef.GgufFile(p)
    p.write_bytes(struct.pack("<IIQQ", 0x46554747, 2, 0, 0))
    with pytest.raises(ValueError, match="GGUF v2"):
        ef.GgufFile(p)
    p.write_bytes(struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 50) + b"abc")
    with pytest.raises(ValueError, match="ends inside a string"):
        ef.GgufFile(p)
    p.write_bytes(b"GGUF")
    with pytest.raises(ValueError, match="too short"):
        ef.GgufFile(p)


def test_writer_round_trip(tmp_path):
    rng = np.random.default_rng(1)
    a = rng.integers(0, 256, 3 * 34, dtype=np.uint8)
    b = rng.integers(0, 256, 2 * 144, dtype=np.uint8)
    p = tmp_path / "w.gguf"
    ef.write_gguf(p, [("n", 4, 7), ("f", 6, 0.5), ("names", 9, (8, ["x", "yz"])), ("ids", 9, (5, [1, -2, 3]))],
                  [("a", (32, 3), 8, a), ("b", (256, 2), 12, b)])
    g = ef.GgufFile(p)
    assert g.meta == {"n": 7, "f": 0.5, "names": ["x", "yz"], "ids": [1, -2, 3]}
    assert g.tensors["a"].offset % 32 == 0 and g.tensors["b"].offset == g.tensors["a"].offset + 128
    assert np.array_equal(g.bytes_of("a"), a) and np.array_equal(g.bytes_of("b"), b)


def synth_model(path, specs, n_embd, n_ff, n_expert, seed):
    """A GGUF with one MoE layer per spec (layer id, gate type, up type, down type), constructed blocks; returns the
    per-layer per-expert (gate, up, down) row arrays."""
    rng = np.random.default_rng(seed)

    def mk(t, n_rows, k):   # (a type the kernels do not take still has a size: plain random bytes)
        if t in synth.BLOCK_VALUES:
            return synth.constructed_rows(t, n_rows, k, rng)
        return rng.integers(0, 256, n_rows * ef.row_bytes(t, k), dtype=np.uint8)

    tensors, rows = [("token_embd.weight", (n_embd, 4), 0, rng.integers(0, 256, n_embd * 16, dtype=np.uint8))], {}
    for l, gt, ut, dt in specs:
        per = []
        for _ in range(n_expert):
            per.append((mk(gt, n_ff, n_embd), mk(ut, n_ff, n_embd), mk(dt, n_embd, n_ff)))
        rows[l] = per
        tensors.append(("blk.%d.ffn_gate_inp.weight" % l, (n_embd, n_expert), 0, np.zeros(n_embd * n_expert * 4, np.uint8)))
        for i, (r, t) in enumerate(zip(ef.ROLES, (gt, ut, dt))):
            dims = (n_embd, n_ff, n_expert) if i < 2 else (n_ff, n_embd, n_expert)
            tensors.append(("blk.%d.ffn_%s_exps.weight" % (l, r), dims, t, np.concatenate([np.ravel(e[i]) for e in per])))
    ef.write_gguf(path, [("general.architecture", 8, "synthetic")], tensors)
    return rows


def test_layers_and_blobs(tmp_path):
    from maya_amd import lib
    n_embd, n_ff, ne = 512, 256, 3
    p = tmp_path / "m.gguf"
    rows = synth_model(p, [(1, 22, 22, 12), (2, 22, 16, 8), (3, 29, 29, 19)], n_embd, n_ff, ne, 5)
    g = ef.GgufFile(p)
    layers = ef.expert_layers(g)
    assert [l.layer for l in layers] == [1, 2, 3]
    for L in layers:
        assert (L.n_embd, L.n_ff, L.n_expert) == (n_embd, n_ff, ne)
        # the library's own sizes for the same formats
        for t, k in ((L.gate_type, n_embd), (L.down_type, n_ff)):
            assert ef.row_bytes(t, k) == lib.row_bytes(t, k)
        if L.up_type in (8, 12, 16, 19, 22, 29):
            lay, nbytes = lib.layout(L.gate_type, L.down_type, n_embd, n_ff, L.up_type)
            assert nbytes == L.blob_bytes and lay.up_off - lay.gate_off == L.part_bytes[0] and lay.down_off - lay.up_off == L.part_bytes[1]
        blobs = ef.layer_blobs(g, L)
        assert blobs.shape == (ne, L.blob_bytes)
        for e in range(ne):
            want = np.concatenate([np.ravel(x) for x in rows[L.layer][e]])
            assert np.array_equal(blobs[e], want)
        for i, r in enumerate(ef.ROLES):
            assert L.gguf_off[i] == g.tensors["blk.%d.ffn_%s_exps.weight" % (L.layer, r)].offset


def test_index_text_and_rules(tmp_path):
    n_embd, n_ff, ne = 512, 256, 3
    p = tmp_path / "model-00001-of-00001.gguf"
    synth_model(p, [(1, 22, 22, 12), (2, 22, 16, 8)], n_embd, n_ff, ne, 6)
    g = ef.GgufFile(p)
    layers = ef.expert_layers(g)
    idx = tmp_path / "native_experts.txt"
    total = ef.write_index(idx, layers, p.name)
    b1 = 256 * 164 * 2 + 512 * 144                   # IQ2_S rows of 512 = 164 B; Q4_K rows of 256 = 144 B
    b2 = 256 * 164 + 256 * 132 + 512 * 272           # IQ2_XXS rows of 512 = 132 B; Q8_0 rows of 256 = 272 B
    assert total == ne * (b1 + b2)
    lines = idx.read_text().split("\n")
    assert lines[0].startswith("# strata native experts v3: layer gu_type d_type offset blob_bytes gate_off up_off down_off")
    assert "(n_expert 3, total %d;" % total in lines[0]
    o = [l.gguf_off for l in layers]
    assert lines[1] == "1 22 12 0 %d %d %d %d" % ((b1,) + o[0])
    assert lines[2] == "2 22:16 8 %d %d %d %d %d" % ((ne * b1, b2) + o[1])
    assert lines[3] == "" and len(lines) == 4
    rows, n_expert, tot = ef.read_index(idx, n_embd, n_ff, n_expert=512)   # (the header's count wins)
    assert n_expert == 3 and tot == total
    assert [(r.layer, r.gate_type, r.up_type, r.down_type, r.offset, r.blob_bytes) for r in rows] == \
        [(1, 22, 22, 12, 0, b1), (2, 22, 16, 8, ne * b1, b2)]
    assert rows[1].gguf_off == o[1] and rows[1].shards == ()
    # experts.bin: the blobs in index order
    ef.write_experts_bin(tmp_path / "experts.bin", g, layers)
    raw = np.fromfile(tmp_path / "experts.bin", dtype=np.uint8)
    assert raw.size == total
    assert np.array_equal(raw[ne * b1:].reshape(ne, b2), ef.layer_blobs(g, layers[1]))
    # the parser's refusals
    head = lines[0] + "\n"
    for body, what in (("1 22 12 0\n", "malformed line"), ("1 22 x 0 %d\n" % b1, "malformed line"),
                       ("1 22 12 0 %d\n" % (b1 + 2), "blob is %d B but its formats make %d" % (b1 + 2, b1)),
                       ("1 22 12 64 %d\n" % b1, "layer 1 is missing or not contiguous"),
                       ("1 22 12 0 %d\n3 22 12 %d %d\n" % (b1, 2 * b1, b1), "layer 3 is missing or not contiguous"),
                       ("1 22 12 0 %d 1 2 3 a b\n" % b1, "malformed line")):
        idx.write_text(head + body)
        with pytest.raises(ValueError, match=what):
            ef.read_index(idx, n_embd, n_ff)
    # a v1 row (no file offsets), a shard name, per-role shard names
    idx.write_text(head + "1 22 12 0 %d\n2 22 12 %d %d 10 20 30 s2.gguf\n3 22 12 %d %d 1 2 3 a b c\n" % (b1, ne * b1, b1, 2 * ne * b1, b1))
    rows, _, _ = ef.read_index(idx, n_embd, n_ff)
    assert rows[0].gguf_off is None and rows[1].shards == ("s2.gguf",) and rows[2].shards == ("a", "b", "c")
    idx.write_text("1 22 12 0 %d\n" % b1)
    with pytest.raises(ValueError, match="no expert count"):
        ef.read_index(idx, n_embd, n_ff)


def test_layers_refused(tmp_path):
    rng = np.random.default_rng(0)
    z = lambda n: rng.integers(0, 256, n, dtype=np.uint8)
    p = tmp_path / "bad.gguf"
    ef.write_gguf(p, [], [("blk.0.ffn_gate_exps.weight", (256, 32, 2), 22, z(2 * 32 * 82)),
                          ("blk.0.ffn_up_exps.weight", (256, 32, 2), 22, z(2 * 32 * 82))])
    with pytest.raises(ValueError, match="lacks blk.0.ffn_down_exps.weight"):
        ef.expert_layers(ef.GgufFile(p))
    ef.write_gguf(p, [], [("blk.0.ffn_gate_exps.weight", (256, 32, 2), 22, z(2 * 32 * 82)),
                          ("blk.0.ffn_up_exps.weight", (256, 32, 2), 22, z(2 * 32 * 82)),
                          ("blk.0.ffn_down_exps.weight", (256, 32, 2), 22, z(2 * 32 * 82))])
    with pytest.raises(ValueError, match="do not make one expert"):
        ef.expert_layers(ef.GgufFile(p))

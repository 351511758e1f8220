"""The EXL3 file side on the CPU: a safetensors model directory laid out by hand from the format (8-byte header length, JSON
header with dtype / shape / data_offsets, the data), the experts' nine pieces found in place, exl3.txt's rows written and read
back, the refusals the reference's packer makes (tools/exl3_pack.py:315-349), and the host concatenation of a blob."""
import json
import os
import struct

import numpy as np
import pytest

from maya_amd import exl3_files as xf

PREFIX = "model.language_model.layers.%d.mlp."


def write_safetensors(path, tensors):
    """tensors: [(name, dtype string, shape, uint8 data)] -> one .safetensors file; returns name -> absolute offset."""
    head, at = {}, 0
    for name, dt, shape, data in tensors:
        head[name] = {"dtype": dt, "shape": list(shape), "data_offsets": [at, at + data.size]}
        at += data.size
    hj = json.dumps(head).encode()
    hj += b" " * ((-len(hj)) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for _, _, _, data in tensors:
            f.write(data.tobytes())
    return {name: 8 + len(hj) + head[name]["data_offsets"][0] for name in head}


def synth_model(tmp, layer=3, n_expert=5, n_embd=256, n_ff=128, k2=(6, 6, 8), cb=2, seed=1, split=True):
    """A model directory whose routed experts of one layer are spread over two files; returns (dir, pieces) with pieces[e][r] =
    (trellis, suh, svh) as numpy arrays."""
    rng = np.random.default_rng(seed)
    d = str(tmp)
    files = [[], []]
    pieces = []
    for e in range(n_expert):
        row = []
        for r, role in enumerate(xf.ROLES):
            k, n = (n_ff, n_embd) if r == 2 else (n_embd, n_ff)
            words = 8 * k2[r]                    # int16 words a tile = 16 K = 8 k2
            tr = rng.integers(0, 65536, (k // 16, n // 16, words), dtype=np.uint16)
            suh = (rng.integers(0, 2, k) * 2 - 1).astype(np.float16)
            svh = ((rng.integers(0, 2, n) * 2 - 1) * rng.uniform(0.02, 0.1, n)).astype(np.float16)
            p = (PREFIX % layer) + "experts.%d.%s_proj." % (e, role)
            f = files[(e + r) % 2 if split else 0]
            f.append((p + "trellis", "I16", tr.shape, tr.view(np.uint8).reshape(-1)))
            f.append((p + "suh", "F16", suh.shape, suh.view(np.uint8)))
            f.append((p + "svh", "F16", svh.shape, svh.view(np.uint8)))
            if cb == 2:
                f.append((p + "mul1", "I32", (1,), np.zeros(4, dtype=np.uint8)))
            elif cb == 1:
                f.append((p + "mcg", "I32", (1,), np.zeros(4, dtype=np.uint8)))
            row.append((tr, suh, svh))
        pieces.append(row)
    names = ["model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors"]
    wm = {}
    for fn, ts in zip(names, files):
        if ts:
            write_safetensors(os.path.join(d, fn), ts)
            wm.update({t[0]: fn for t in ts})
    json.dump({"weight_map": wm}, open(os.path.join(d, "model.safetensors.index.json"), "w"))
    return d, pieces


def test_pieces_are_found_in_place_and_the_index_round_trips(tmp_path):
    d, pieces = synth_model(tmp_path)
    st = xf.SafeTensorsDir(d)
    L = xf.expert_layer(st, 3, PREFIX % 3, 5)
    assert L["cb"] == 2 and L["k2"] == (6, 6, 8) and L["shape"] == (256, 128, 128, 256)
    # a part's bytes: 16 k2 bytes a 16 x 16 tile + the two FP16 vectors
    assert L["gu_bytes"] == 256 * 128 * 6 // 16 + 2 * 256 + 2 * 128 and L["dn_bytes"] == 128 * 256 * 8 // 16 + 2 * 128 + 2 * 256
    for e, parts in L["rows"]:
        for r in range(3):
            for w in range(3):
                fi, off = parts[r][2 * w], parts[r][2 * w + 1]
                want = pieces[e][r][w].view(np.uint8).reshape(-1)
                assert xf.piece_bytes(L, r, w) == want.size
                got = st.mm[st.files[fi]][off:off + want.size]
                assert np.array_equal(got, want), (e, r, w)
    ix = os.path.join(d, "exl3.txt")
    xf.write_index(ix, st, [L])
    files, layers = xf.read_index(ix)
    assert files == st.files and len(layers) == 1
    for key in ("layer", "cb", "k2", "shape", "gu_bytes", "dn_bytes", "rows"):
        assert layers[0][key] == L[key], key
    # a row written out by hand from the format's description
    lines = [l for l in open(ix).read().splitlines() if l.startswith("layer")]
    assert lines == ["layer 3 2 3 3 4 256 128 128 256 %d %d" % (L["gu_bytes"], L["dn_bytes"])]
    e0 = [l for l in open(ix).read().splitlines() if l.startswith("e 3 0 ")][0].split()
    assert len(e0) == 21 and [int(v) for v in e0[3:9]] == list(L["rows"][0][1][0])


def test_half_integer_bitrates_and_their_text(tmp_path):
    assert xf.tile_k2(48, 2, "x") == 6 and xf.tile_k2(24, 2, "x") == 3 and xf.tile_k2(56, 2, "x") == 7 and xf.tile_k2(128, 0, "x") == 16
    assert xf.k_text(6) == "3" and xf.k_text(7) == "3.5" and xf.k2_of_text("3.5") == 7 and xf.k2_of_text("4") == 8
    with pytest.raises(ValueError):
        xf.tile_k2(24, 1, "x")           # K 1.5 without the mul1 codebook
    with pytest.raises(ValueError):
        xf.tile_k2(20, 2, "x")
    d, _ = synth_model(tmp_path, k2=(7, 7, 5), cb=2, n_expert=2)
    L = xf.expert_layer(xf.SafeTensorsDir(d), 3, PREFIX % 3, 2)
    assert L["k2"] == (7, 7, 5)
    ix = os.path.join(d, "exl3.txt")
    xf.write_index(ix, xf.SafeTensorsDir(d), [L])
    assert "layer 3 2 3.5 3.5 2.5 " in open(ix).read()
    assert xf.read_index(ix)[1][0]["k2"] == (7, 7, 5)


def test_refusals(tmp_path):
    (tmp_path / "a").mkdir()
    d, _ = synth_model(tmp_path / "a", n_expert=3)
    st = xf.SafeTensorsDir(d)
    with pytest.raises(ValueError, match="no "):
        xf.expert_layer(st, 3, PREFIX % 3, 4)        # expert 3 is not in the files
    # an expert whose down part has another bitrate than expert 0's
    (tmp_path / "b").mkdir()
    d2, _ = synth_model(tmp_path / "b", n_expert=2, split=False)
    extra = []
    rng = np.random.default_rng(5)
    for r, role in enumerate(xf.ROLES):
        k, n = (128, 256) if r == 2 else (256, 128)
        words = 8 * (4 if r == 2 else 6)
        p = (PREFIX % 3) + "experts.2.%s_proj." % role
        extra += [(p + "trellis", "I16", (k // 16, n // 16, words), rng.integers(0, 256, k // 16 * (n // 16) * words * 2, dtype=np.uint8)),
                  (p + "suh", "F16", (k,), np.zeros(2 * k, dtype=np.uint8)), (p + "svh", "F16", (n,), np.zeros(2 * n, dtype=np.uint8)),
                  (p + "mul1", "I32", (1,), np.zeros(4, dtype=np.uint8))]
    write_safetensors(os.path.join(d2, "extra.safetensors"), extra)
    with pytest.raises(ValueError, match="differ from expert 0"):
        xf.expert_layer(xf.SafeTensorsDir(d2), 3, PREFIX % 3, 3)
    # index rows: an expert before its layer, a wrong field count, an unknown file
    ix = os.path.join(d2, "bad.txt")
    open(ix, "w").write("file 0 a.safetensors\ne 3 0 " + " ".join(["0"] * 18) + "\n")
    with pytest.raises(ValueError, match="before its layer"):
        xf.read_index(ix)
    open(ix, "w").write("file 0 a.safetensors\nlayer 3 2 3 3 4 256 128 128 256 1 2\ne 3 0 1 2 3\n")
    with pytest.raises(ValueError, match="fields"):
        xf.read_index(ix)
    open(ix, "w").write("file 0 a.safetensors\nlayer 3 2 3 3 4 256 128 128 256 1 2\ne 3 0 " + " ".join(["7 0"] * 9) + "\n")
    with pytest.raises(ValueError, match="no file row"):
        xf.read_index(ix)
    # a truncated file
    open(os.path.join(d2, "short.safetensors"), "wb").write(struct.pack("<Q", 1 << 40))
    with pytest.raises(ValueError, match="header"):
        xf.SafeTensorsDir(d2)

"""EXL3 routed experts from the model's files to the expert blobs the kernels read: the host side of the reference's
tools/exl3_pack.py for this path (its SafeTensors reader :61-110, the experts' plan :315-349, exl3.txt's `layer` / `e` rows
:596-612), with the assembly of the blobs done on the device by maya_exl3_pack_experts.

An EXL3 model is a directory of .safetensors files; a routed expert e of a layer is nine tensors
`<prefix>experts.<e>.{gate,up,down}_proj.{trellis,suh,svh}` (trellis int16 [k/16][n/16][16 K words], suh / svh F16) plus a
marker tensor naming the codebook (`mul1`, `mcg`, neither = 3inst).  Nothing is converted: the pieces are copied, byte for
byte, to their offsets in the blob (maya_exl3_layout).  numpy for the files, torch for device memory.
"""
import json
import os
import struct

import numpy as np

ROLES = ("gate", "up", "down")
PIECES = ("trellis", "suh", "svh")


class SafeTensorsDir:
    """Every tensor of a model directory, read in place: name -> (file index, dtype, shape, absolute offset, bytes).  The
    files of model.safetensors.index.json first (a name goes to the file the index names), then any other .safetensors
    beside them for names the index does not have (tools/exl3_pack.py:61-92)."""

    def __init__(self, path):
        self.dir = path
        ix_path = os.path.join(path, "model.safetensors.index.json")
        ix = json.load(open(ix_path))["weight_map"] if os.path.exists(ix_path) else {}
        primary = sorted(set(ix.values()))
        others = sorted(f for f in os.listdir(path) if f.endswith(".safetensors") and f not in primary)
        self.files, self.t, self.mm = [], {}, {}
        for fn in primary + others:
            p = os.path.join(path, fn)
            with open(p, "rb") as f:
                head = f.read(8)
                if len(head) != 8:
                    raise ValueError("%s: not a safetensors file" % fn)
                n = struct.unpack("<Q", head)[0]
                if n > os.path.getsize(p) - 8:
                    raise ValueError("%s: header of %d bytes in a file of %d" % (fn, n, os.path.getsize(p)))
                h = json.loads(f.read(n))
            base = 8 + n
            self.files.append(fn)
            for k, v in h.items():
                if k == "__metadata__" or k in self.t:
                    continue
                if fn in primary and ix.get(k) not in (None, fn):
                    continue
                s, e = v["data_offsets"]
                if e < s or base + e > os.path.getsize(p):
                    raise ValueError("%s: %s lies outside the file" % (fn, k))
                self.t[k] = (len(self.files) - 1, v["dtype"], list(v["shape"]), base + s, e - s)
            self.mm[fn] = np.memmap(p, dtype=np.uint8, mode="r")

    def has(self, name):
        return name in self.t

    def raw(self, name):
        fi, _, _, off, nb = self.t[name]
        return self.mm[self.files[fi]][off:off + nb]


def tile_k2(words, cb, what):
    """A trellis tile's int16 words -> k2 = twice the bits a weight: 16 K words for K 1..8; 24 / 40 / 56 for the half-integer
    K 1.5 / 2.5 / 3.5, which only the mul1 codebook has (tools/exl3_pack.py:134-145)."""
    if words % 16 == 0 and 1 <= words // 16 <= 8:
        return words // 8
    if words in (24, 40, 56):
        if cb != 2:
            raise ValueError("%s: half-integer bitrate K %g without the mul1 codebook" % (what, words / 16))
        return words // 8
    raise ValueError("%s: %d words a tile is no EXL3 bitrate" % (what, words))


def k_text(k2):
    """exl3.txt's bits field: "3", or "3.5" for a half-integer K (tools/exl3_pack.py:148-150)."""
    return "%d.5" % (k2 // 2) if k2 % 2 else "%d" % (k2 // 2)


def k2_of_text(s):
    return int(round(float(s) * 2))


def expert_layer(st, layer, prefix, n_expert):
    """One MoE layer's experts: every expert's nine pieces where the files keep them, and the layer's geometry.  Every expert
    must share the parts' shapes, bits and codebook; gate and up must be alike (tools/exl3_pack.py:315-349).  Returns
    {"layer", "cb", "k2": (gate, up, down), "shape": (k_gate, n_gate, k_down, n_down), "gu_bytes", "dn_bytes",
     "rows": [(expert, [(file, trellis_off, file, suh_off, file, svh_off) per part])]}."""
    lay, rows = None, []
    for e in range(n_expert):
        parts, shape = [], []
        for r in ROLES:
            p = "%sexperts.%d.%s_proj." % (prefix, e, r)
            for x in PIECES:
                if not st.has(p + x):
                    raise ValueError("layer %d expert %d: no %s%s" % (layer, e, p, x))
            kt, nt, w = st.t[p + "trellis"][2]
            if st.t[p + "suh"][1] != "F16" or st.t[p + "svh"][1] != "F16":
                raise ValueError("layer %d expert %d %s: suh / svh are not F16" % (layer, e, r))
            cb = 2 if st.has(p + "mul1") else 1 if st.has(p + "mcg") else 0
            shape.append((kt * 16, nt * 16, tile_k2(w, cb, "layer %d expert %d %s" % (layer, e, r)), cb))
            parts.append((st.t[p + "trellis"][0], st.t[p + "trellis"][3], st.t[p + "suh"][0], st.t[p + "suh"][3],
                          st.t[p + "svh"][0], st.t[p + "svh"][3]))
        shape = tuple(shape)
        if lay is None:
            lay = shape
        elif shape != lay:
            raise ValueError("layer %d expert %d: shapes / bits differ from expert 0's" % (layer, e))
        rows.append((e, parts))
    (gk, gn, gk2, gcb), (uk, un, uk2, ucb), (dk, dn, dk2, dcb) = lay
    if (gk, gn) != (uk, un) or gk2 != uk2 or not (gcb == ucb == dcb):
        raise ValueError("layer %d: gate and up differ, or the codebooks do" % layer)
    if (dk, dn) != (gn, gk):
        raise ValueError("layer %d: down is %d x %d beside a %d x %d gate" % (layer, dk, dn, gk, gn))

    def part(k, n, k2):
        return k * n * k2 // 16 + 2 * k + 2 * n       # 16 k2 bytes a 16 x 16 tile

    return {"layer": layer, "cb": gcb, "k2": (gk2, uk2, dk2), "shape": (gk, gn, dk, dn), "gu_bytes": part(gk, gn, gk2),
            "dn_bytes": part(dk, dn, dk2), "rows": rows}


def write_index(path, st, layers):
    """exl3.txt's `file`, `layer` and `e` rows (tools/exl3_pack.py:596-612)."""
    with open(path, "w", newline="\n") as f:
        f.write("# maya exl3 pack v1\n")
        for i, fn in enumerate(st.files):
            f.write("file %d %s\n" % (i, fn))
        for L in layers:
            f.write("layer %d %d %s %s %s %d %d %d %d %d %d\n" % (L["layer"], L["cb"], *(k_text(x) for x in L["k2"]), *L["shape"],
                                                                  L["gu_bytes"], L["dn_bytes"]))
            for e, parts in L["rows"]:
                f.write("e %d %d %s\n" % (L["layer"], e, " ".join("%d %d %d %d %d %d" % p for p in parts)))


def read_index(path):
    """(files, layers) back from exl3.txt; a row of another kind (`mat`: the dense matrices) is left to its reader.  Refuses a
    row with the wrong number of fields, an expert of a layer without a `layer` row, a file index without a `file` row."""
    files, layers, by_id = {}, [], {}
    for ln, line in enumerate(open(path), 1):
        t = line.split()
        if not t or t[0].startswith("#"):
            continue
        if t[0] == "file":
            if len(t) != 3:
                raise ValueError("%s:%d: file row" % (path, ln))
            files[int(t[1])] = t[2]
        elif t[0] == "layer":
            if len(t) != 12:
                raise ValueError("%s:%d: layer row has %d fields" % (path, ln, len(t)))
            L = {"layer": int(t[1]), "cb": int(t[2]), "k2": tuple(k2_of_text(x) for x in t[3:6]), "shape": tuple(int(x) for x in t[6:10]),
                 "gu_bytes": int(t[10]), "dn_bytes": int(t[11]), "rows": []}
            layers.append(L)
            by_id[L["layer"]] = L
        elif t[0] == "e":
            if len(t) != 3 + 18:
                raise ValueError("%s:%d: expert row has %d fields" % (path, ln, len(t)))
            if int(t[1]) not in by_id:
                raise ValueError("%s:%d: expert of layer %s before its layer row" % (path, ln, t[1]))
            v = [int(x) for x in t[3:]]
            parts = [tuple(v[6 * r:6 * r + 6]) for r in range(3)]
            for p in parts:
                for fi in p[0::2]:
                    if fi not in files:
                        raise ValueError("%s:%d: file %d has no file row" % (path, ln, fi))
            by_id[int(t[1])]["rows"].append((int(t[2]), parts))
    return [files[i] for i in sorted(files)], layers


def piece_bytes(L, role, what):
    gk, gn, dk, dn = L["shape"]
    k, n = (dk, dn) if role == 2 else (gk, gn)
    return k * n * L["k2"][role] // 16 if what == 0 else 2 * k if what == 1 else 2 * n


def host_blob(L, layout, blob_bytes, mm, files, expert_row):
    """One expert's blob as the host would concatenate it (the checker of maya_exl3_pack_experts): numpy uint8 [blob_bytes]."""
    blob = np.zeros(blob_bytes, dtype=np.uint8)
    _, parts = expert_row
    for r in range(3):
        for w, dst in enumerate((layout.trellis[r], layout.suh[r], layout.svh[r])):
            fi, off = parts[r][2 * w], parts[r][2 * w + 1]
            nb = piece_bytes(L, r, w)
            blob[dst:dst + nb] = mm[files[fi]][off:off + nb]
    return blob


class LayerStore:
    """A layer's EXL3 experts resident in HBM: file pages -> pinned staging -> maya_exl3_pack_experts.  `table` is the device
    array of blob addresses the plans are built from."""

    def __init__(self, model_dir, files, L, order=None, device="cuda"):
        import torch
        from . import exl3
        gk, gn, dk, dn = L["shape"]
        self.layout, self.blob_bytes = exl3.layout_init(gk, gn, list(L["k2"]), L["cb"], exl3.ORDER_TRELLIS_FIRST if order is None else order)
        n = len(L["rows"])
        self.stride = (self.blob_bytes + 255) & ~255
        self.pool = torch.zeros(n * self.stride, dtype=torch.uint8, device=device)
        mm = {fn: np.memmap(os.path.join(model_dir, fn), dtype=np.uint8, mode="r") for fn in files}
        # the pieces, expert after expert, into one pinned staging buffer (each piece on a 16-byte boundary), then one copy
        sizes = [[piece_bytes(L, r, w) for w in range(3)] for r in range(3)]
        per = sum((s + 15) & ~15 for row in sizes for s in row)
        staging = torch.empty(n * per, dtype=torch.uint8, pin_memory=True)
        sview = staging.numpy()
        offs = np.zeros((n, 9), dtype=np.int64)
        at = 0
        for i, (_, parts) in enumerate(L["rows"]):
            for r in range(3):
                for w in range(3):
                    fi, off = parts[r][2 * w], parts[r][2 * w + 1]
                    nb = sizes[r][w]
                    sview[at:at + nb] = mm[files[fi]][off:off + nb]
                    offs[i, 3 * r + w] = at
                    at += (nb + 15) & ~15
        dev_staging = staging.to(device)
        pieces = torch.from_numpy(offs + dev_staging.data_ptr()).to(device)
        exl3.pack_experts(self.layout, pieces, n, self.pool, self.stride)
        torch.cuda.synchronize()
        base = self.pool.data_ptr()
        self.table = torch.tensor([base + i * self.stride for i in range(n)], dtype=torch.int64, device=device)
        self.n_expert = n

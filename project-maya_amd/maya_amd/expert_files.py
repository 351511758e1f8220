"""Expert tensors on disk -> expert blobs in HBM.

The reference keeps routed experts in two on-disk forms, and both feed the expert-rows kernels unchanged:

* the model's GGUF v3 file(s): per MoE layer three stacked tensors `blk.<l>.ffn_{gate,up,down}_exps.weight`, ggml
  dimensions `[row length, rows, n_expert]`, expert e's rows contiguous (header layout as read by the reference's
  tools/gguf_reader.py:83-121; the engine reads the experts straight from the file at the offsets the index names);
* a pack directory: `native_experts.txt`, one row a layer `layer gu_type d_type offset blob_bytes gate_off up_off down_off
  [shard]` (written by tools/iq_pack.py:470-500, parsed by `expert_layout_load`, src/kernels/cpu/expert_layout.cpp:165-253)
  and optionally `experts.bin`, per layer n_expert blobs `[gate rows | up rows | down rows]` (tools/iq_pack.py:505-518).

This module reads and writes those forms (header only is parsed; tensor bytes are memory-mapped, never loaded whole) and
hands a layer's three tensors to `maya_moe_pack_experts`, which builds the blobs on the device in either packing.  The
rules of the reference's parser are kept: the `#` header's `(n_expert N` wins over the caller's count, the type column
may be `gate:up`, a row whose blob size disagrees with its formats is refused, layers must be contiguous in experts.bin.
"""
import mmap
import os
import struct
from collections import namedtuple

import numpy as np

GGUF_MAGIC = 0x46554747  # "GGUF"
ROLES = ("gate", "up", "down")

# ggml type id -> (values a block, bytes a block) for the types the expert kernels take, and the float types
BLOCK = {0: (1, 4), 1: (1, 2), 30: (1, 2), 8: (32, 34), 12: (256, 144), 16: (256, 66), 19: (256, 50), 22: (256, 82),
         29: (256, 56)}
TYPE_NAME = {0: "F32", 1: "F16", 30: "BF16", 8: "Q8_0", 12: "Q4_K", 16: "IQ2_XXS", 19: "IQ1_S", 22: "IQ2_S", 29: "IQ1_M"}

Tensor = namedtuple("Tensor", "name dims type_id offset nbytes")   # offset: absolute in the file; nbytes None = unknown type
ExpertLayer = namedtuple("ExpertLayer", "layer gate_type up_type down_type n_embd n_ff n_expert blob_bytes part_bytes "
                                        "gguf_off shard")
IndexRow = namedtuple("IndexRow", "layer gate_type up_type down_type offset blob_bytes gguf_off shards")

_SCALAR = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}


def row_bytes(type_id, k):
    vals, nbytes = BLOCK[type_id]
    if k % vals:
        raise ValueError("a row of %d values is not whole blocks of type %d" % (k, type_id))
    return k // vals * nbytes


class GgufFile:
    """The directory of one GGUF v3 file: `meta` (key -> value), `tensors` (name -> Tensor), `data_start`.  The file stays
    memory-mapped; `bytes_of(name)` is a uint8 view of a tensor's data."""

    def __init__(self, path):
        self.path = str(path)
        self._fh = open(self.path, "rb")
        size = os.fstat(self._fh.fileno()).st_size
        if size < 24:
            raise ValueError("%s: not a GGUF file (too short)" % os.path.basename(self.path))
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self._at = 0
        magic, self.version, n_tensors, n_kv = self._take("<IIQQ")
        if magic != GGUF_MAGIC:
            raise ValueError("%s: not a GGUF file (magic %#x)" % (os.path.basename(self.path), magic))
        if self.version != 3:
            raise ValueError("%s: GGUF v%d, this reader handles v3" % (os.path.basename(self.path), self.version))
        self.meta = {}
        for _ in range(n_kv):
            key = self._string()
            self.meta[key] = self._value()
        raw = []
        for _ in range(n_tensors):
            name = self._string()
            (nd,) = self._take("<I")
            dims = self._take("<%dQ" % nd)
            type_id, rel = self._take("<IQ")
            raw.append((name, tuple(int(d) for d in dims), int(type_id), int(rel)))
        align = self.meta.get("general.alignment")
        self.alignment = int(align) if isinstance(align, int) and align else 32
        self.data_start = (self._at + self.alignment - 1) // self.alignment * self.alignment
        self.tensors = {}
        for name, dims, type_id, rel in raw:
            n = 1
            for d in dims:
                n *= d
            geom = BLOCK.get(type_id)
            nbytes = n // geom[0] * geom[1] if geom and n % geom[0] == 0 else None
            self.tensors[name] = Tensor(name, dims, type_id, self.data_start + rel, nbytes)

    def _take(self, fmt):
        n = struct.calcsize(fmt)
        if self._at + n > len(self._mm):
            raise ValueError("%s: the header ends early" % os.path.basename(self.path))
        out = struct.unpack_from(fmt, self._mm, self._at)
        self._at += n
        return out

    def _string(self):
        (n,) = self._take("<Q")
        if self._at + n > len(self._mm):
            raise ValueError("%s: the header ends inside a string" % os.path.basename(self.path))
        s = self._mm[self._at:self._at + n].decode("utf-8", "replace")
        self._at += n
        return s

    def _value(self, t=None):
        if t is None:
            (t,) = self._take("<I")
        if t == 8:
            return self._string()
        if t == 9:
            et, count = self._take("<IQ")
            if et == 8:
                return [self._string() for _ in range(count)]
            if et not in _SCALAR:
                raise ValueError("%s: metadata array of type %d" % (os.path.basename(self.path), et))
            return list(self._take("<%d%s" % (count, _SCALAR[et])))
        if t not in _SCALAR:
            raise ValueError("%s: metadata value of type %d" % (os.path.basename(self.path), t))
        return self._take("<" + _SCALAR[t])[0]

    def bytes_of(self, name):
        t = self.tensors[name]
        if t.nbytes is None:
            raise ValueError("%s: tensor %s has type %d, whose size is unknown here" % (self.path, name, t.type_id))
        if t.offset + t.nbytes > len(self._mm):
            raise ValueError("%s: tensor %s runs past the end of the file" % (self.path, name))
        return np.frombuffer(self._mm, dtype=np.uint8, count=t.nbytes, offset=t.offset)

    def close(self):
        # (views handed out by bytes_of keep the mapping alive; closing with a view outstanding raises BufferError)
        self._mm.close()
        self._fh.close()


def write_gguf(path, meta, tensors, alignment=32):
    """A GGUF v3 file from `meta` = [(key, gguf value type id, value)] (arrays: (key, 9, (element type id, list))) and
    `tensors` = [(name, ggml dims, type id, uint8 data)], data aligned to `alignment`.  For synthetic models and tests."""

    def s(x):
        b = x.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    def val(t, v):
        if t == 8:
            return s(v)
        if t == 9:
            et, items = v
            body = b"".join(s(i) for i in items) if et == 8 else struct.pack("<%d%s" % (len(items), _SCALAR[et]), *items)
            return struct.pack("<IQ", et, len(items)) + body
        return struct.pack("<" + _SCALAR[t], v)

    head = struct.pack("<IIQQ", GGUF_MAGIC, 3, len(tensors), len(meta))
    for key, t, v in meta:
        head += s(key) + struct.pack("<I", t) + val(t, v)
    rel, infos = 0, b""
    for name, dims, type_id, data in tensors:
        infos += s(name) + struct.pack("<I", len(dims)) + struct.pack("<%dQ" % len(dims), *dims) + struct.pack("<IQ", type_id, rel)
        rel += (int(data.size) + alignment - 1) // alignment * alignment
    head += infos
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * ((-len(head)) % alignment))
        for _, _, _, data in tensors:
            b = np.ascontiguousarray(data, dtype=np.uint8).tobytes()
            f.write(b)
            f.write(b"\0" * ((-len(b)) % alignment))


def expert_layers(g, shard=None):
    """The MoE layers of a GGUF file, in layer order: for each, the three stacked expert tensors' types, shapes and
    absolute offsets (tools/iq_pack.py:455-467).  Refuses a layer whose gate / up shapes or expert counts disagree."""
    ids = sorted({int(n.split(".")[1]) for n in g.tensors if n.startswith("blk.") and n.endswith("_exps.weight")})
    out = []
    for l in ids:
        try:
            ts = [g.tensors["blk.%d.ffn_%s_exps.weight" % (l, r)] for r in ROLES]
        except KeyError as e:
            raise ValueError("layer %d lacks %s" % (l, e.args[0]))
        if any(len(t.dims) != 3 for t in ts):
            raise ValueError("layer %d: an expert tensor is not [row length, rows, n_expert]" % l)
        (ke, nf, ne), up, (kd, nd, ned) = ts[0].dims, ts[1].dims, ts[2].dims
        if up != ts[0].dims or (kd, nd) != (nf, ke) or ned != ne:
            raise ValueError("layer %d: gate %s, up %s and down %s do not make one expert" % (l, ts[0].dims, up, ts[2].dims))
        if any(t.type_id not in BLOCK for t in ts):
            raise ValueError("layer %d: expert type %s is not handled" % (l, [t.type_id for t in ts]))
        part = (nf * row_bytes(ts[0].type_id, ke), nf * row_bytes(ts[1].type_id, ke), ke * row_bytes(ts[2].type_id, nf))
        out.append(ExpertLayer(l, ts[0].type_id, ts[1].type_id, ts[2].type_id, ke, nf, ne, sum(part), part,
                               tuple(t.offset for t in ts), shard))
    return out


def layer_blobs(g, layer):
    """[n_expert, blob_bytes] uint8: expert e's [gate rows | up rows | down rows], the host concatenation the
    reference's packer writes into experts.bin (tools/iq_pack.py:510-514)."""
    parts = [g.bytes_of("blk.%d.ffn_%s_exps.weight" % (layer.layer, r)).reshape(layer.n_expert, -1) for r in ROLES]
    return np.concatenate(parts, axis=1)


def write_index(path, layers, gguf_name):
    """native_experts.txt (v3 rows) for `layers`, experts.bin offsets running in layer order."""
    n_expert = layers[0].n_expert
    if any(l.n_expert != n_expert for l in layers):
        raise ValueError("the layers disagree on the expert count; a per-layer pruned model cannot be packed")
    total = sum(l.blob_bytes * n_expert for l in layers)
    with open(path, "w", encoding="utf-8", newline="\n") as f:
        f.write("# strata native experts v3: layer gu_type d_type offset blob_bytes gate_off up_off down_off [shard] "
                "(n_expert %d, total %d; absolute offsets in %s, or in the named shard beside it)\n"
                % (n_expert, total, gguf_name))
        at = 0
        for l in layers:
            gt = str(l.gate_type) if l.gate_type == l.up_type else "%d:%d" % (l.gate_type, l.up_type)
            row = "%d %s %d %d %d %d %d %d" % ((l.layer, gt, l.down_type, at, l.blob_bytes) + tuple(l.gguf_off))
            f.write(row + (" " + l.shard if l.shard else "") + "\n")
            at += l.blob_bytes * n_expert
    return total


def write_experts_bin(path, g, layers):
    with open(path, "wb") as f:
        for l in layers:
            f.write(layer_blobs(g, l).tobytes())


def read_index(path, n_embd, n_ff, n_expert=None):
    """(rows, n_expert, total bytes of experts.bin) of a native_experts.txt, under the rules of `expert_layout_load`
    (src/kernels/cpu/expert_layout.cpp:184-250)."""
    rows = {}
    with open(path, "r", encoding="utf-8") as f:
        for line in f.read().split("\n"):
            if not line:
                continue
            if line[0] == "#":
                at = line.find("(n_expert ")
                if at >= 0:
                    digits = line[at + 10:].split(",")[0].split()[0]
                    n_expert = int(digits)
                continue
            w = line.split()
            try:
                if len(w) < 5:
                    raise ValueError
                l = int(w[0])
                gt, _, ut = w[1].partition(":")
                gt, ut, dt = int(gt), int(ut) if ut else int(gt), int(w[2])
                off, blob = int(w[3]), int(w[4])
                gguf_off = tuple(int(x) for x in w[5:8]) if len(w) >= 8 else None
                shards = tuple(w[8:])
                if l < 0 or len(shards) not in (0, 1, 3):
                    raise ValueError
            except ValueError:
                raise ValueError("native_experts.txt: a malformed line: " + line)
            for t in (gt, ut, dt):
                if t not in BLOCK:
                    raise ValueError("native_experts.txt: layer %d has type %d, which is not handled" % (l, t))
            made = n_ff * (row_bytes(gt, n_embd) + row_bytes(ut, n_embd)) + n_embd * row_bytes(dt, n_ff)
            if made != blob:
                raise ValueError("native_experts.txt: layer %d blob is %d B but its formats make %d" % (l, blob, made))
            rows[l] = IndexRow(l, gt, ut, dt, off, blob, gguf_off, shards)
    if n_expert is None:
        raise ValueError("native_experts.txt: no expert count in the header and none given")
    # the layers that carry experts run on from the first one listed (leading dense layers have no row)
    at, out = 0, []
    for l in sorted(rows):
        if rows[l].offset != at:
            raise ValueError("native_experts.txt: layer %d is missing or not contiguous" % l)
        at += rows[l].blob_bytes * n_expert
        out.append(rows[l])
    return out, n_expert, at


class LayerStore:
    """One layer's experts resident in HBM, built on the device from the file's three stacked tensors
    (maya_moe_pack_experts): `pool` holds n_expert blobs `stride` bytes apart (256-byte aligned), `table` their
    addresses for the plan kernel, `layout` the blob's layout in the chosen packing."""

    def __init__(self, stacked, layer, packing=None, device="cuda", stream=None):
        import torch
        from . import lib
        packing = lib.PACK_STREAM if packing is None else packing
        gguf_layout, blob = lib.layout(layer.gate_type, layer.down_type, layer.n_embd, layer.n_ff, layer.up_type)
        if blob != layer.blob_bytes:
            raise ValueError("layer %d: the library makes its blob %d B, the file %d" % (layer.layer, blob, layer.blob_bytes))
        self.stride = (blob + 255) & ~255
        self.pool = torch.empty(self.stride * layer.n_expert + 256, dtype=torch.uint8, device=device)
        pad = (-self.pool.data_ptr()) % 256
        dst = self.pool[pad:]
        dev = []
        for s in stacked:   # file pages -> pinned staging -> HBM (the views are read-only maps of the file)
            pinned = torch.empty(int(s.size), dtype=torch.uint8, pin_memory=True)
            np.copyto(pinned.numpy().reshape(s.shape), s)
            dev.append(pinned.to(device))
        lib.pack_experts(gguf_layout, dev[0], dev[1], dev[2], layer.n_expert, packing, dst, self.stride, stream)
        torch.cuda.synchronize()
        base = dst.data_ptr()
        self.addrs = [base + e * self.stride for e in range(layer.n_expert)]
        self.table = torch.tensor(self.addrs, dtype=torch.int64, device=device)
        self.layout = lib.copy_layout(gguf_layout, packing)
        self.bytes = blob * layer.n_expert

    @classmethod
    def from_gguf(cls, g, layer, **kw):
        return cls([g.bytes_of("blk.%d.ffn_%s_exps.weight" % (layer.layer, r)) for r in ROLES], layer, **kw)

    @classmethod
    def from_experts_bin(cls, path, row, n_expert, n_embd, n_ff, **kw):
        """From a pack directory's experts.bin: the layer's blobs are split back into the three stacked tensors (views of
        the memory-mapped file, copied once on their way to the device)."""
        part = (n_ff * row_bytes(row.gate_type, n_embd), n_ff * row_bytes(row.up_type, n_embd), n_embd * row_bytes(row.down_type, n_ff))
        blobs = np.memmap(path, dtype=np.uint8, mode="r", offset=row.offset, shape=(n_expert, row.blob_bytes))
        cuts = (0, part[0], part[0] + part[1], row.blob_bytes)
        layer = ExpertLayer(row.layer, row.gate_type, row.up_type, row.down_type, n_embd, n_ff, n_expert, row.blob_bytes,
                            part, row.gguf_off, None)
        return cls([blobs[:, cuts[i]:cuts[i + 1]] for i in range(3)], layer, **kw)

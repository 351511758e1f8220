"""EXL3 (exllamav3 trellis) routed experts: ctypes bindings of the maya_exl3_* entry points and a generator of
well-formed synthetic expert blobs (any bit pattern is a valid trellis; suh / svh are FP16 sign-and-scale vectors)."""
import ctypes as C

import numpy as np
import torch

from . import lib as L

TYPE_EXL3 = 200
CB_3INST, CB_MCG, CB_MUL1 = 0, 1, 2


class Exl3Layout(C.Structure):
    _fields_ = [("suh", C.c_uint64 * 3), ("svh", C.c_uint64 * 3), ("trellis", C.c_uint64 * 3), ("k2", C.c_int32 * 3),
                ("cb", C.c_int32), ("n_embd", C.c_int32), ("n_ff", C.c_int32)]


class Exl3Args(C.Structure):
    _fields_ = [("layout", Exl3Layout), ("n_tokens", C.c_int32), ("k", C.c_int32), ("plan_ptr", C.c_void_p),
                ("plan_w", C.c_void_p), ("grp_ptr", C.c_void_p), ("grp_start", C.c_void_p), ("grp_ent", C.c_void_p),
                ("n_groups", C.c_void_p), ("skip", C.c_void_p), ("limit", C.c_float), ("x", C.c_void_p),
                ("x_stride", C.c_int64), ("h", C.c_void_p), ("part", C.c_void_p), ("add", C.c_void_p),
                ("add_flag", C.c_void_p), ("add2", C.c_void_p), ("out", C.c_void_p)]


EXPORTS = ["maya_exl3_supported", "maya_exl3_trellis_bytes", "maya_exl3_reconstruct_inner", "maya_exl3_gate_up",
           "maya_exl3_down", "maya_exl3_workspace_bytes", "maya_exl3_layer_decode", "maya_exl3_layout_init",
           "maya_exl3_pack_experts"]
ORDER_SCALES_FIRST, ORDER_TRELLIS_FIRST = 0, 1

_bound = False


def load():
    global _bound
    lib = L.load()
    if not _bound:
        vp, i32, i64, sz, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
        lib.maya_exl3_supported.argtypes = [i32, i32]
        lib.maya_exl3_trellis_bytes.restype = sz
        lib.maya_exl3_trellis_bytes.argtypes = [i64, i64, i32]
        lib.maya_exl3_reconstruct_inner.argtypes = [vp, i64, i64, i32, i32, vp, vp]
        lib.maya_exl3_gate_up.argtypes = [C.POINTER(Exl3Args), vp]
        lib.maya_exl3_down.argtypes = [C.POINTER(Exl3Args), vp]
        lib.maya_exl3_workspace_bytes.restype = sz
        lib.maya_exl3_workspace_bytes.argtypes = [C.POINTER(Exl3Layout), i32, i32]
        lib.maya_exl3_layout_init.restype = sz
        lib.maya_exl3_layout_init.argtypes = [C.POINTER(Exl3Layout), i32, i32, C.POINTER(C.c_int32), i32, i32]
        lib.maya_exl3_pack_experts.argtypes = [C.POINTER(Exl3Layout), vp, i32, vp, sz, vp]
        lib.maya_exl3_layer_decode.argtypes = [C.POINTER(Exl3Layout), vp, i32, i32, vp, vp, i32, f32, vp, vp, vp, vp, vp, sz, vp]
        _bound = True
    return lib


def supported(k2, cb):
    return bool(load().maya_exl3_supported(k2, cb))


def trellis_bytes(k, n, k2):
    return int(load().maya_exl3_trellis_bytes(k, n, k2))


def make_layout(n_embd, n_ff, k2, cb):
    """(Exl3Layout, blob bytes): for gate, up, down in turn [suh | svh | trellis], each part 16-byte aligned."""
    k2 = [k2] * 3 if isinstance(k2, int) else list(k2)
    l = Exl3Layout()
    l.cb, l.n_embd, l.n_ff = cb, n_embd, n_ff
    off = 0
    for r, (k, n) in enumerate(((n_embd, n_ff), (n_embd, n_ff), (n_ff, n_embd))):
        l.k2[r] = k2[r]
        l.suh[r] = off
        off += (2 * k + 15) & ~15
        l.svh[r] = off
        off += (2 * n + 15) & ~15
        l.trellis[r] = off
        off += ((k // 16) * (n // 16) * 16 * k2[r] + 15) & ~15
    return l, off


def layout_init(n_embd, n_ff, k2, cb, order=ORDER_SCALES_FIRST):
    """(Exl3Layout, blob bytes) from the library (maya_exl3_layout_init); order: ORDER_SCALES_FIRST ([suh | svh | trellis], 16-byte
    pieces: what make_layout gives) or ORDER_TRELLIS_FIRST ([trellis | suh | svh], 256-byte pieces: the engine's assembled blob)."""
    k2 = [k2] * 3 if isinstance(k2, int) else list(k2)
    l = Exl3Layout()
    n = int(load().maya_exl3_layout_init(C.byref(l), n_embd, n_ff, (C.c_int32 * 3)(*k2), cb, order))
    if n == 0:
        raise L.MayaError(2, "maya_exl3_layout_init: %d x %d at k2 %s with codebook %d is not covered" % (n_embd, n_ff, k2, cb))
    return l, n


def pack_experts(l, pieces, n_expert, dst, dst_stride, stream=None):
    """pieces: int64 device tensor [n_expert, 9] of addresses (trellis, suh, svh of gate, up, down); dst: uint8 device tensor."""
    assert pieces.dtype == torch.int64 and pieces.numel() == 9 * n_expert and pieces.is_contiguous()
    L.check(load().maya_exl3_pack_experts(C.byref(l), L._p(pieces), n_expert, L._p(dst), dst_stride, L._stream(stream)))


def matrix_of(l, role):
    """(k, n) of gate (0), up (1) or down (2)."""
    return (l.n_ff, l.n_embd) if role == 2 else (l.n_embd, l.n_ff)


def synth_blob(l, nbytes, seed, scale=None):
    """One expert's blob: random trellis bits, suh = random signs, svh = random signs times a scale that keeps the
    outputs near unit size."""
    rng = np.random.default_rng(seed)
    blob = np.zeros(nbytes, dtype=np.uint8)
    for r in range(3):
        k, n = matrix_of(l, r)
        suh = (rng.integers(0, 2, k) * 2 - 1).astype(np.float16)
        sc = (1.0 / np.sqrt(k)) if scale is None else scale
        svh = ((rng.integers(0, 2, n) * 2 - 1) * sc * rng.uniform(0.5, 1.5, n)).astype(np.float16)
        tb = (k // 16) * (n // 16) * 16 * l.k2[r]
        blob[l.suh[r]:l.suh[r] + 2 * k] = suh.view(np.uint8)
        blob[l.svh[r]:l.svh[r] + 2 * n] = svh.view(np.uint8)
        blob[l.trellis[r]:l.trellis[r] + tb] = rng.integers(0, 256, tb, dtype=np.uint8)
    return blob


def parts_of(l, blob, role):
    """(trellis uint32 [k/16 * n/16 * 4 k2], suh uint16 [k], svh uint16 [n]) views of one matrix of a host blob."""
    k, n = matrix_of(l, role)
    tb = (k // 16) * (n // 16) * 16 * l.k2[role]
    tr = blob[l.trellis[role]:l.trellis[role] + tb].view(np.uint32)
    suh = blob[l.suh[role]:l.suh[role] + 2 * k].view(np.uint16)
    svh = blob[l.svh[role]:l.svh[role] + 2 * n].view(np.uint16)
    return tr, suh, svh


def reconstruct_inner(trellis, k, n, k2, cb, stream=None):
    """W' [k][n] as float16 from a device uint32 trellis."""
    dst = torch.empty((k, n), dtype=torch.float16, device=trellis.device)
    L.check(load().maya_exl3_reconstruct_inner(L._p(trellis), k, n, k2, cb, L._p(dst), L._stream(stream)))
    return dst


def make_args(l, n_tokens, k, plan_ptr, plan_w, x, h, part, out, groups=None, limit=0.0, add=None, add_flag=None,
              skip=None, x_stride=0):
    a = Exl3Args()
    a.layout = l
    a.n_tokens, a.k = n_tokens, k
    a.plan_ptr, a.plan_w = plan_ptr.data_ptr(), plan_w.data_ptr()
    if groups is not None:
        a.grp_ptr, a.grp_start, a.grp_ent, a.n_groups = (t.data_ptr() for t in groups)
    a.skip = None if skip is None else skip.data_ptr()
    a.limit = limit
    a.x, a.x_stride = (None if x is None else x.data_ptr()), x_stride
    a.h = None if h is None else h.data_ptr()
    a.part = None if part is None else part.data_ptr()
    a.add = None if add is None else add.data_ptr()
    a.add_flag = None if add_flag is None else add_flag.data_ptr()
    a.out = None if out is None else out.data_ptr()
    return a


def gate_up(a, stream=None):
    L.check(load().maya_exl3_gate_up(C.byref(a), L._stream(stream)))


def down(a, stream=None):
    L.check(load().maya_exl3_down(C.byref(a), L._stream(stream)))


class Exl3Layer:
    """One routed EXL3 layer on the device (maya_exl3_layer_decode); buffers allocated once here."""

    def __init__(self, layout, n_expert, k, max_tokens=1, device="cuda"):
        self.layout, self.n_expert, self.k, self.max_tokens = layout, n_expert, k, max_tokens
        n = int(load().maya_exl3_workspace_bytes(C.byref(layout), max_tokens, k))
        if n == 0:
            raise L.MayaError(2, "maya_exl3_workspace_bytes: bad shape")
        self.ws_bytes = n
        self._ws = torch.empty(n + 256, dtype=torch.uint8, device=device)
        pad = (-self._ws.data_ptr()) % 256
        self.ws = self._ws[pad:pad + n]
        self.ids = torch.empty((max_tokens, k), dtype=torch.int32, device=device)
        self.weights = torch.empty((max_tokens, k), dtype=torch.float32, device=device)
        self.out = torch.empty((max_tokens, layout.n_embd), dtype=torch.float32, device=device)

    def forward(self, expert_table, logits, x, limit=0.0, add=None, stream=None, routed=None):
        """routed = (ids, weights) [nt, k] tensors: the tokens are already routed (logits is then ignored)."""
        nt = x.shape[0]
        assert nt <= self.max_tokens and x.is_contiguous() and x.dtype == torch.float32
        if routed is not None:
            self.ids[:nt].copy_(routed[0])
            self.weights[:nt].copy_(routed[1])
            logits = None
        else:
            assert logits.is_contiguous()
        L.check(load().maya_exl3_layer_decode(C.byref(self.layout), L._p(expert_table), self.n_expert, self.k, L._p(logits),
                                              L._p(x), nt, limit, L._p(add), L._p(self.ids), L._p(self.weights),
                                              L._p(self.out), L._p(self.ws), self.ws_bytes, L._stream(stream)))
        return self.out[:nt]

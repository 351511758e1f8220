"""A prompt chunk's routed experts (the grouped int8 GEMM): ctypes bindings of the maya_moe_prefill_* entry points."""
import ctypes as C

import torch

from . import lib as L


class Plan(C.Structure):
    _fields_ = [("bounds", C.c_void_p), ("row_entry", C.c_void_p), ("entry_row", C.c_void_p), ("tile_expert", C.c_void_p),
                ("tile_row0", C.c_void_p), ("n_tiles", C.c_void_p)]


class PAct(C.Structure):
    _fields_ = [("q", C.c_void_p), ("d", C.c_void_p), ("s", C.c_void_p)]


EXPORTS = ["maya_moe_prefill_tile_rows", "maya_moe_prefill_max_tiles", "maya_moe_prefill_supported", "maya_moe_prefill_plan",
           "maya_moe_prefill_quant", "maya_moe_prefill_gate_up", "maya_moe_prefill_down", "maya_moe_prefill_combine",
           "maya_moe_prefill_workspace_bytes", "maya_moe_prefill_layer"]

_bound = False


def load():
    global _bound
    lib = L.load()
    if not _bound:
        vp, i32, i64, sz, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
        LP, PP = C.POINTER(L.Layout), C.POINTER(Plan)
        lib.maya_moe_prefill_max_tiles.argtypes = [i32, i32]
        lib.maya_moe_prefill_supported.argtypes = [i32]
        lib.maya_moe_prefill_plan.argtypes = [vp, i32, vp, i32, PP, vp]
        lib.maya_moe_prefill_quant.argtypes = [vp, i32, i64, PP, i32, i32, i32, i64, PAct, vp]
        lib.maya_moe_prefill_gate_up.argtypes = [LP, vp, i32, PP, i32, PAct, f32, vp, PAct, vp]
        lib.maya_moe_prefill_down.argtypes = [LP, vp, i32, PP, i32, PAct, vp, vp]
        lib.maya_moe_prefill_combine.argtypes = [PP, vp, vp, i32, i32, i64, vp, vp, i32, vp]
        lib.maya_moe_prefill_workspace_bytes.restype = sz
        lib.maya_moe_prefill_workspace_bytes.argtypes = [LP, i32, i32, i32]
        lib.maya_moe_prefill_layer.argtypes = [LP, vp, i32, i32, vp, vp, i32, i32, f32, vp, vp, vp, vp, i32, vp, sz, vp]
        _bound = True
    return lib


class PlanBuf:
    """The device arrays of one plan."""

    def __init__(self, n_entries, n_expert, device="cuda"):
        lib = load()
        self.n_entries, self.n_expert = n_entries, n_expert
        self.max_tiles = int(lib.maya_moe_prefill_max_tiles(n_entries, n_expert))
        i32 = dict(dtype=torch.int32, device=device)
        self.bounds = torch.zeros(n_expert + 1, **i32)
        self.row_entry = torch.zeros(n_entries, **i32)
        self.entry_row = torch.zeros(n_entries, **i32)
        self.tile_expert = torch.zeros(self.max_tiles, **i32)
        self.tile_row0 = torch.zeros(self.max_tiles, **i32)
        self.n_tiles = torch.zeros(1, **i32)
        self.c = Plan(self.bounds.data_ptr(), self.row_entry.data_ptr(), self.entry_row.data_ptr(), self.tile_expert.data_ptr(),
                      self.tile_row0.data_ptr(), self.n_tiles.data_ptr())


class ActRows:
    def __init__(self, rows, k, device="cuda"):
        self.q = torch.zeros((rows, k), dtype=torch.int8, device=device)
        self.d = torch.zeros((rows, k // 256), dtype=torch.float32, device=device)
        # a block's 8 sub-block code sums as two FP16 digits: [rows][k / 256][the 8 low digits, then the 8 high ones]
        self.s = torch.zeros((rows, k // 256, 16), dtype=torch.float16, device=device)
        self.c = PAct(self.q.data_ptr(), self.d.data_ptr(), self.s.data_ptr())

    def sums(self):
        """The integer sum of every 32 codes [rows][k / 32], from the two digits (lo + 64 hi)."""
        v = self.s.to(torch.float32)
        return (v[:, :, :8] + 64.0 * v[:, :, 8:]).reshape(v.shape[0], -1).to(torch.int32)


def plan(ids, expert_table, stream=None):
    p = PlanBuf(ids.numel(), expert_table.numel(), ids.device)
    L.check(load().maya_moe_prefill_plan(L._p(ids), ids.numel(), L._p(expert_table), expert_table.numel(), C.byref(p.c), L._stream(stream)))
    return p


def quant(x, p, k, stream=None):
    n_embd = x.shape[1]
    a = ActRows(p.n_entries, n_embd, x.device)
    L.check(load().maya_moe_prefill_quant(L._p(x), L.dtype_id(x), x.stride(0), C.byref(p.c), p.n_entries, p.n_expert, k, n_embd,
                                          a.c, L._stream(stream)))
    return a


def gate_up(layout, expert_table, p, xq, limit=0.0, stream=None):
    h = ActRows(p.n_entries, layout.n_ff, xq.q.device)
    h.f32 = torch.zeros((p.n_entries, layout.n_ff), dtype=torch.float32, device=xq.q.device)   # the values before rounding
    L.check(load().maya_moe_prefill_gate_up(C.byref(layout), L._p(expert_table), p.n_expert, C.byref(p.c), p.n_entries, xq.c,
                                            limit, L._p(h.f32), h.c, L._stream(stream)))
    return h


def down(layout, expert_table, p, hq, stream=None):
    part = torch.zeros((p.n_entries, layout.n_embd), dtype=torch.float32, device=hq.q.device)
    L.check(load().maya_moe_prefill_down(C.byref(layout), L._p(expert_table), p.n_expert, C.byref(p.c), p.n_entries, hq.c,
                                         L._p(part), L._stream(stream)))
    return part


def combine(p, weights, part, n_tokens, k, add=None, out_dtype=torch.float32, stream=None):
    n_embd = part.shape[1]
    out = torch.empty((n_tokens, n_embd), dtype=out_dtype, device=part.device)
    L.check(load().maya_moe_prefill_combine(C.byref(p.c), L._p(weights), L._p(part), n_tokens, k, n_embd, L._p(add), L._p(out),
                                            L.dtype_id(out), L._stream(stream)))
    return out


class PrefillLayer:
    """One routed layer over a prompt chunk (maya_moe_prefill_layer); buffers allocated once here."""

    def __init__(self, layout, n_expert, k, max_tokens, out_dtype=torch.bfloat16, device="cuda"):
        self.layout, self.n_expert, self.k, self.max_tokens = layout, n_expert, k, max_tokens
        n = int(load().maya_moe_prefill_workspace_bytes(C.byref(layout), max_tokens, k, n_expert))
        if n == 0:
            raise L.MayaError(2, "maya_moe_prefill_workspace_bytes: bad shape")
        self.ws_bytes = n
        self._ws = torch.empty(n + 256, dtype=torch.uint8, device=device)
        pad = (-self._ws.data_ptr()) % 256
        self.ws = self._ws[pad:pad + n]
        self.ids = torch.empty((max_tokens, k), dtype=torch.int32, device=device)
        self.weights = torch.empty((max_tokens, k), dtype=torch.float32, device=device)
        self.out = torch.empty((max_tokens, layout.n_embd), dtype=out_dtype, device=device)

    def forward(self, expert_table, logits, x, limit=0.0, add=None, stream=None, routed=None):
        """routed = (ids, weights) [nt, k] tensors: the tokens are already routed (logits is then ignored)."""
        nt = x.shape[0]
        assert nt <= self.max_tokens and x.is_contiguous()
        if routed is not None:
            self.ids[:nt].copy_(routed[0])
            self.weights[:nt].copy_(routed[1])
            logits = None
        else:
            assert logits.is_contiguous()
        L.check(load().maya_moe_prefill_layer(C.byref(self.layout), L._p(expert_table), self.n_expert, self.k, L._p(logits),
                                              L._p(x), L.dtype_id(x), nt, limit, L._p(add), L._p(self.ids), L._p(self.weights),
                                              L._p(self.out), L.dtype_id(self.out), L._p(self.ws), self.ws_bytes,
                                              L._stream(stream)))
        return self.out[:nt]

"""ctypes bindings of libmaya_moe.so: one Python function per C entry point of include/maya_moe.h, taking torch tensors
for device memory.  A non-zero status raises MayaError with the library's message."""
import ctypes as C
import os

import torch

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(PKG, "libmaya_moe.so")

Q8_0, Q4_K, IQ2_XXS, IQ1_S, IQ2_S, IQ1_M = 8, 12, 16, 19, 22, 29
DT_F32, DT_BF16, DT_F16 = 0, 1, 2
MAX_TOKENS, MAX_K = 16, 16
PACK_GGUF, PACK_STREAM = 0, 1

EXPORTS = [
    "maya_last_error", "maya_device_info", "maya_init", "maya_moe_supported", "maya_moe_block_bytes",
    "maya_moe_block_values", "maya_moe_row_bytes", "maya_moe_layout_init", "maya_dequant_rows", "maya_quant_act",
    "maya_quant_i8x32", "maya_moe_route_topk", "maya_moe_plan", "maya_moe_group", "maya_moe_gate_up", "maya_moe_down",
    "maya_moe_workspace_bytes", "maya_moe_layer_decode", "maya_moe_repack", "maya_moe_unpack", "maya_moe_pack_experts",
    "maya_moe_route_sigmoid", "maya_moe_layer_decode_routed", "maya_moe_route_plan", "maya_moe_route_tiered", "maya_moe_fetch",
    "maya_moe_tab_update",
    "maya_dequant_rows_packed", "maya_moe_down_rounds_h", "maya_mv_supported", "maya_mv", "maya_moe_layer_decode_static",
    "maya_moe_layer_decode_shared", "maya_moe_route_window_ok", "maya_moe_route_window", "maya_moe_layer_decode_begin",
    "maya_moe_layer_decode_end", "maya_moe_prefetch",
]


ROUTER_SOFTMAX, ROUTER_SIGMOID = 0, 1
NORM_NONE, NORM_CLAMP, NORM_HF = 0, 1, 2


class MayaError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("maya_moe status %d: %s" % (code, msg))
        self.code = code


class Router(C.Structure):
    _fields_ = [("kind", C.c_int32), ("norm", C.c_int32), ("bias", C.c_void_p), ("w_scale", C.c_float)]


class Residency(C.Structure):
    _fields_ = [("tab", C.c_void_p), ("n_keys", C.c_int32), ("n_layers", C.c_int32), ("scratch", C.c_void_p), ("n_scratch", C.c_int32),
                ("reserved", C.c_int32), ("fetch_src", C.c_void_p), ("counts", C.c_void_p), ("seq", C.c_void_p), ("masks", C.c_void_p)]


SPARES = 3


class Layout(C.Structure):
    _fields_ = [("gate_type", C.c_int32), ("up_type", C.c_int32), ("down_type", C.c_int32), ("n_embd", C.c_int32),
                ("n_ff", C.c_int32), ("gate_off", C.c_uint64), ("up_off", C.c_uint64), ("down_off", C.c_uint64),
                ("packing", C.c_int32), ("reserved", C.c_int32)]


class Act(C.Structure):
    _fields_ = [("q", C.c_void_p), ("d", C.c_void_p), ("bsums", C.c_void_p)]


class Args(C.Structure):
    _fields_ = [("layout", Layout), ("n_tokens", C.c_int32), ("k", C.c_int32), ("plan_ptr", C.c_void_p),
                ("plan_w", C.c_void_p), ("grp_ptr", C.c_void_p), ("grp_start", C.c_void_p), ("grp_ent", C.c_void_p),
                ("n_groups", C.c_void_p), ("skip", C.c_void_p), ("limit", C.c_float), ("x", Act), ("h", C.c_void_p),
                ("hq", Act), ("part", C.c_void_p), ("add", C.c_void_p), ("add_flag", C.c_void_p), ("add2", C.c_void_p),
                ("out", C.c_void_p)]


class MvJob(C.Structure):
    """maya_mv_job: y[c] = alpha * W x[c] + bias (glmf::MvJob, include/strata/kernels/glm_fast.hpp:29-43)."""
    _fields_ = [("w", C.c_void_p), ("type", C.c_int32), ("packing", C.c_int32), ("n_in", C.c_int32), ("n_out", C.c_int32),
                ("ncol", C.c_int32), ("alpha", C.c_float), ("x", Act), ("bias", C.c_void_p), ("y", C.c_void_p),
                ("y_stride", C.c_int64)]


_lib = None


def load():
    """The loaded library; raises when it was not built (python -m maya_amd.build, or __graft_entry__.build())."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError("%s is missing: the HIP library was not built; there is no CPU fallback" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, sz, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float
    L.maya_last_error.restype = C.c_char_p
    L.maya_device_info.restype = C.c_char_p
    L.maya_moe_row_bytes.restype = sz
    L.maya_moe_row_bytes.argtypes = [i32, i64]
    L.maya_moe_layout_init.restype = sz
    L.maya_moe_layout_init.argtypes = [C.POINTER(Layout), i32, i32, i32, i32, i32]
    L.maya_dequant_rows.argtypes = [i32, vp, sz, i64, i64, vp, vp]
    L.maya_dequant_rows_packed.argtypes = [i32, i32, vp, sz, i64, i64, vp, vp]
    L.maya_moe_repack.argtypes = [C.POINTER(Layout), vp, vp, vp]
    L.maya_moe_unpack.argtypes = [C.POINTER(Layout), vp, vp, vp]
    L.maya_moe_pack_experts.argtypes = [C.POINTER(Layout), vp, vp, vp, i32, i32, vp, sz, vp]
    L.maya_quant_act.argtypes = [i32, vp, i32, i64, i32, i64, Act, vp]
    L.maya_quant_i8x32.argtypes = [vp, i32, i64, vp, i32, i64, vp, vp, vp]
    L.maya_moe_route_topk.argtypes = [vp, i32, i32, i32, vp, vp, vp]
    L.maya_moe_plan.argtypes = [vp, i32, vp, i32, vp, vp]
    L.maya_moe_route_tiered.argtypes = [vp, vp, i32, i32, i32, i32, C.POINTER(Residency), i32, vp, vp, vp, vp]
    L.maya_moe_fetch.argtypes = [vp, vp, i32, sz, vp]
    L.maya_moe_tab_update.argtypes = [vp, i32, vp, vp, i32, vp]
    L.maya_moe_prefetch.argtypes = [vp, vp, vp, i32, sz, i32, vp]
    L.maya_moe_group.argtypes = [vp, i32, vp, vp, vp, vp, vp]
    L.maya_moe_gate_up.argtypes = [C.POINTER(Args), vp]
    L.maya_moe_down.argtypes = [C.POINTER(Args), vp]
    L.maya_moe_down_rounds_h.argtypes = [C.POINTER(Args)]
    L.maya_mv_supported.argtypes = [i32]
    L.maya_mv.argtypes = [C.POINTER(MvJob), i32, vp]
    L.maya_moe_workspace_bytes.restype = sz
    L.maya_moe_workspace_bytes.argtypes = [C.POINTER(Layout), i32, i32]
    L.maya_moe_layer_decode.argtypes = [C.POINTER(Layout), vp, i32, i32, vp, vp, i32, i32, f32, vp, vp, vp, vp, vp, sz, vp]
    L.maya_moe_layer_decode_routed.argtypes = [C.POINTER(Layout), vp, i32, i32, C.POINTER(Router), vp, vp, i32, i32, f32, vp, vp, vp,
                                               vp, vp, sz, vp]
    L.maya_moe_layer_decode_begin.argtypes = L.maya_moe_layer_decode_routed.argtypes
    L.maya_moe_layer_decode_end.argtypes = L.maya_moe_layer_decode_routed.argtypes
    L.maya_moe_layer_decode_shared.argtypes = [C.POINTER(Layout), vp, i32, i32, C.POINTER(Router), vp, vp, i32, i32, f32,
                                               C.POINTER(Args), vp, vp, vp, vp, sz, vp]
    L.maya_moe_route_sigmoid.argtypes = [vp, vp, i32, i32, i32, f32, i32, vp, vp, vp]
    L.maya_moe_route_plan.argtypes = [C.POINTER(Router), vp, i32, i32, i32, vp, vp, vp, vp, vp]
    L.maya_moe_route_window_ok.argtypes = [C.POINTER(Router), i32, i32, i32]
    L.maya_moe_route_window.argtypes = [C.POINTER(Router), vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise MayaError(rc, load().maya_last_error().decode("utf-8", "replace"))


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(stream=None):
    s = torch.cuda.current_stream() if stream is None else stream
    return C.c_void_p(s.cuda_stream)


def dtype_id(t):
    return {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}[t.dtype]


def layout(gate_type, down_type, n_embd, n_ff, up_type=None):
    """(Layout, blob bytes) of a contiguous [gate | up | down] expert blob."""
    l = Layout()
    n = load().maya_moe_layout_init(C.byref(l), gate_type, gate_type if up_type is None else up_type, down_type, n_embd, n_ff)
    if n == 0:
        raise MayaError(1, load().maya_last_error().decode())
    return l, int(n)


def row_bytes(t, k):
    return int(load().maya_moe_row_bytes(t, k))


class ActBuf:
    """A quantized activation batch on the device (maya_act): codes, per-32 scales, per-16 sums."""

    def __init__(self, rows, k, device="cuda"):
        self.rows, self.k = rows, k
        self.q = torch.empty((rows, k), dtype=torch.int8, device=device)
        self.d = torch.empty((rows, k // 32), dtype=torch.float32, device=device)
        self.bsums = torch.empty((rows, k // 16), dtype=torch.int16, device=device)

    def c(self):
        return Act(self.q.data_ptr(), self.d.data_ptr(), self.bsums.data_ptr())


def dequant_rows(t, w, k, n_rows, stream=None, packing=PACK_GGUF):
    out = torch.empty((n_rows, k), dtype=torch.float32, device=w.device)
    check(load().maya_dequant_rows_packed(t, packing, _p(w), 0, k, n_rows, _p(out), _stream(stream)))
    return out


def copy_layout(l, packing=None):
    c = Layout()
    C.memmove(C.byref(c), C.byref(l), C.sizeof(Layout))
    if packing is not None:
        c.packing = packing
    return c


def repack(l, src, dst, stream=None):
    """src (GGUF blob on the device, layout l) -> dst in the stream packing."""
    check(load().maya_moe_repack(C.byref(l), _p(src), _p(dst), _stream(stream)))


def unpack(l, src, dst, stream=None):
    check(load().maya_moe_unpack(C.byref(l), _p(src), _p(dst), _stream(stream)))


def pack_experts(l, gate_exps, up_exps, down_exps, n_expert, packing, dst, dst_stride, stream=None):
    """The layer's blobs (dst_stride bytes apart in dst) from its three stacked GGUF tensors, in `packing` order."""
    check(load().maya_moe_pack_experts(C.byref(l), _p(gate_exps), _p(up_exps), _p(down_exps), n_expert, packing, _p(dst),
                                       dst_stride, _stream(stream)))


def quant_act(act_type, x, stream=None):
    """x [rows, k] (f32 / bf16 / f16, contiguous) -> ActBuf in the activation format of weight type act_type."""
    assert x.is_contiguous() and x.dim() == 2
    out = ActBuf(x.shape[0], x.shape[1], x.device)
    check(load().maya_quant_act(act_type, _p(x), dtype_id(x), 0, x.shape[0], x.shape[1], out.c(), _stream(stream)))
    return out


def quant_i8x32(x, row_idx=None, rows=None, stream=None):
    assert x.is_contiguous() and x.dim() == 2
    rows = x.shape[0] if rows is None else rows
    q = torch.empty((rows, x.shape[1]), dtype=torch.int8, device=x.device)
    d = torch.empty((rows, x.shape[1] // 32), dtype=torch.float32, device=x.device)
    check(load().maya_quant_i8x32(_p(x), dtype_id(x), 0, _p(row_idx), rows, x.shape[1], _p(q), _p(d), _stream(stream)))
    return q, d


def route_topk(logits, k, stream=None):
    assert logits.is_contiguous() and logits.dtype == torch.float32 and logits.dim() == 2
    nt, ne = logits.shape
    ids = torch.empty((nt, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((nt, k), dtype=torch.float32, device=logits.device)
    check(load().maya_moe_route_topk(_p(logits), nt, ne, k, _p(ids), _p(w), _stream(stream)))
    return ids, w


def route_sigmoid(logits, bias, k, w_scale=1.0, norm=NORM_CLAMP, stream=None):
    assert logits.is_contiguous() and logits.dtype == torch.float32 and logits.dim() == 2
    nt, ne = logits.shape
    ids = torch.empty((nt, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((nt, k), dtype=torch.float32, device=logits.device)
    check(load().maya_moe_route_sigmoid(_p(logits), _p(bias), nt, ne, k, w_scale, norm, _p(ids), _p(w), _stream(stream)))
    return ids, w


def route_plan(logits, k, expert_table, router=None, stream=None):
    """ids, weights and the plan (blob addresses) in one launch."""
    nt, ne = logits.shape
    ids = torch.empty((nt, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((nt, k), dtype=torch.float32, device=logits.device)
    pl = torch.empty(nt * k, dtype=torch.int64, device=logits.device)
    check(load().maya_moe_route_plan(None if router is None else C.byref(router), _p(logits), nt, ne, k, _p(expert_table), _p(ids),
                                     _p(w), _p(pl), _stream(stream)))
    return ids, w, pl


def route_window(logits, k, expert_table, stream=None):
    """A window's ids, weights, plan and groups in one launch (maya_moe_route_window: the softmax router, up to 256
    experts): what route_plan followed by group returns."""
    nt, ne = logits.shape
    dev, n = logits.device, nt * k
    ids = torch.empty((nt, k), dtype=torch.int32, device=dev)
    w = torch.empty((nt, k), dtype=torch.float32, device=dev)
    pl = torch.empty(n, dtype=torch.int64, device=dev)
    grp_ptr = torch.zeros(n, dtype=torch.int64, device=dev)
    grp_start = torch.zeros(n + 1, dtype=torch.int32, device=dev)
    grp_ent = torch.zeros(n, dtype=torch.int32, device=dev)
    n_groups = torch.zeros(1, dtype=torch.int32, device=dev)
    check(load().maya_moe_route_window(None, _p(logits), nt, ne, k, _p(expert_table), _p(ids), _p(w), _p(pl), _p(grp_ptr), _p(grp_start),
                                       _p(grp_ent), _p(n_groups), _stream(stream)))
    return ids, w, pl, (grp_ptr, grp_start, grp_ent, n_groups)


class Tiers:
    """The residency tables of a model's routed experts on the device (glmf::MoeDev's tab, include/strata/kernels/
    glm_fast.hpp:284-296): tab = [n_keys] HBM addresses | [n_keys] second-tier addresses | [n_layers][SPARES] free HBM
    slots, scratch slots for what is fetched but not promoted, and the outputs of a route."""

    def __init__(self, n_layers, n_expert, scratch, max_entries, with_counts=False):
        self.n_layers, self.n_expert = n_layers, n_expert
        self.n_keys = n_layers * n_expert
        self.tab = torch.zeros(2 * self.n_keys + n_layers * SPARES, dtype=torch.int64, device="cuda")
        self.scratch = scratch
        self.fetch_src = torch.zeros(max_entries, dtype=torch.int64, device="cuda")
        self.masks = torch.zeros(4 * max_entries, dtype=torch.int32, device="cuda")
        self.counts = torch.zeros(self.n_keys, dtype=torch.int32, device="cuda") if with_counts else None
        self.seq = torch.zeros(1, dtype=torch.int32, device="cuda") if with_counts else None
        self.c = Residency(self.tab.data_ptr(), self.n_keys, n_layers, scratch.data_ptr() if scratch.numel() else None, scratch.numel(), 0,
                           self.fetch_src.data_ptr(), None if self.counts is None else self.counts.data_ptr(),
                           None if self.seq is None else self.seq.data_ptr(), self.masks.data_ptr())

    def route(self, logits, layer, k, router=None, promote_min=0, stream=None):
        """ids, weights, plan of logits [nt, n_expert] for this layer; fetch_src / masks are left in the object."""
        nt, ne = logits.shape
        assert nt * k <= self.fetch_src.numel()
        ids = torch.empty((nt, k), dtype=torch.int32, device=logits.device)
        w = torch.empty((nt, k), dtype=torch.float32, device=logits.device)
        pl = torch.empty(nt * k, dtype=torch.int64, device=logits.device)
        check(load().maya_moe_route_tiered(None if router is None else C.byref(router), _p(logits), nt, layer, ne, k, C.byref(self.c),
                                           promote_min, _p(ids), _p(w), _p(pl), _stream(stream)))
        return ids, w, pl

    def fetch(self, plan_ptr, blob_bytes, stream=None):
        check(load().maya_moe_fetch(_p(self.fetch_src), _p(plan_ptr), plan_ptr.numel(), blob_bytes, _stream(stream)))

    def update(self, keys, vals, stream=None):
        check(load().maya_moe_tab_update(_p(self.tab), self.tab.numel(), _p(keys), _p(vals), keys.numel(), _stream(stream)))


def prefetch(pf_src, pf_dst, pf_n, blob_bytes, n_workgroups=0, stream=None):
    """Copies the first *pf_n (a device int32) entries of the list: blob_bytes from pf_src[i] to pf_dst[i] (maya_moe_prefetch)."""
    assert pf_src.dtype == torch.int64 and pf_dst.dtype == torch.int64 and pf_n.dtype == torch.int32
    check(load().maya_moe_prefetch(_p(pf_src), _p(pf_dst), _p(pf_n), min(pf_src.numel(), pf_dst.numel()), blob_bytes, n_workgroups,
                                   _stream(stream)))


def plan(ids, expert_table, stream=None):
    out = torch.empty(ids.numel(), dtype=torch.int64, device=ids.device)
    check(load().maya_moe_plan(_p(ids), ids.numel(), _p(expert_table), expert_table.numel(), _p(out), _stream(stream)))
    return out


def group(plan_ptr, stream=None):
    n = plan_ptr.numel()
    dev = plan_ptr.device
    grp_ptr = torch.zeros(n, dtype=torch.int64, device=dev)
    grp_start = torch.zeros(n + 1, dtype=torch.int32, device=dev)
    grp_ent = torch.zeros(n, dtype=torch.int32, device=dev)
    n_groups = torch.zeros(1, dtype=torch.int32, device=dev)
    check(load().maya_moe_group(_p(plan_ptr), n, _p(grp_ptr), _p(grp_start), _p(grp_ent), _p(n_groups), _stream(stream)))
    return grp_ptr, grp_start, grp_ent, n_groups


class ExpertStore:
    """Expert blobs resident in HBM: one contiguous allocation, expert e's [gate | up | down] blob at `offset[e]` (the
    reference keeps VRAM-resident experts in slots of one pool the same way).  `table` is the device array of blob
    addresses the plan kernel reads (0: not resident).  With `pack_layout` (a GGUF Layout) every blob is regrouped into
    the stream packing on its way in (maya_moe_repack), as an engine would do when it uploads an expert."""

    def __init__(self, blobs, device="cuda", misalign=0, pack_layout=None):
        import numpy as np
        self.n = len(blobs)
        sizes = [int(b.size) for b in blobs]
        stride = (max(sizes) + misalign + 255) & ~255
        self.pool = torch.empty(stride * self.n + 256, dtype=torch.uint8, device=device)
        base = self.pool.data_ptr()
        pad = (-base) % 256
        addrs = []
        staging = torch.empty(max(sizes), dtype=torch.uint8, device=device) if pack_layout is not None else None
        for e, b in enumerate(blobs):
            off = pad + e * stride + misalign
            src = torch.from_numpy(np.ascontiguousarray(b))
            if pack_layout is None:
                self.pool[off:off + sizes[e]].copy_(src, non_blocking=False)
            else:
                staging[:sizes[e]].copy_(src, non_blocking=False)
                repack(pack_layout, staging, self.pool[off:off + sizes[e]])
                torch.cuda.synchronize()
            addrs.append(base + off)
        self.addrs = addrs
        self.table = torch.tensor(addrs, dtype=torch.int64, device=device)
        self.bytes = sum(sizes)


class MoeLayer:
    """One routed layer on the device: route -> plan -> group -> quantize -> gate/up -> quantize -> down -> combine
    (maya_moe_layer_decode).  Buffers are allocated once here; a call allocates nothing."""

    def __init__(self, gate_type, down_type, n_embd, n_ff, n_expert, k, max_tokens=1, up_type=None, device="cuda",
                 packing=PACK_GGUF):
        self.gguf_layout, self.blob_bytes = layout(gate_type, down_type, n_embd, n_ff, up_type)
        self.layout = copy_layout(self.gguf_layout, packing)
        self.n_embd, self.n_ff, self.n_expert, self.k, self.max_tokens = n_embd, n_ff, n_expert, k, max_tokens
        n = int(load().maya_moe_workspace_bytes(C.byref(self.layout), max_tokens, k))
        if n == 0:
            raise MayaError(2, load().maya_last_error().decode())
        self.ws_bytes = n
        self._ws = torch.empty(n + 256, dtype=torch.uint8, device=device)
        pad = (-self._ws.data_ptr()) % 256
        self.ws = self._ws[pad:pad + n]
        self.ids = torch.empty((max_tokens, k), dtype=torch.int32, device=device)
        self.weights = torch.empty((max_tokens, k), dtype=torch.float32, device=device)
        self.out = torch.empty((max_tokens, n_embd), dtype=torch.float32, device=device)

    def forward(self, expert_table, logits, x, limit=float("inf"), add=None, stream=None, router=None, routed=None, shared=None,
                shared_limit=float("inf"), half=None):
        """router: None (the softmax router) or a Router (kind, norm, bias pointer, w_scale); routed = (ids, weights)
        [nt, k] tensors: the tokens are already routed (logits is then ignored); shared: a DenseExpert over the same
        tokens that runs beside the routed experts (maya_moe_layer_decode_shared) - out = add + shared(x) + routed(x);
        half: "begin" / "end" = the layer's two halves (maya_moe_layer_decode_begin / _end), same arguments in both."""
        nt = x.shape[0]
        assert nt <= self.max_tokens and x.is_contiguous()
        if routed is not None:
            self.ids[:nt].copy_(routed[0])
            self.weights[:nt].copy_(routed[1])
            logits = None
        else:
            assert logits.is_contiguous()
        if shared is not None:
            assert shared.n == nt and shared.n_embd == self.n_embd
            a = shared.args
            a.limit, a.add = shared_limit, (add.data_ptr() if add is not None else None)
            check(load().maya_moe_layer_decode_shared(C.byref(self.layout), _p(expert_table), self.n_expert, self.k,
                                                      C.byref(router) if router is not None else None, _p(logits), _p(x), dtype_id(x),
                                                      nt, limit, C.byref(a), _p(self.ids), _p(self.weights), _p(self.out), _p(self.ws),
                                                      self.ws_bytes, _stream(stream)))
            a.add = None
            return self.out[:nt]
        if half is not None:
            fn = load().maya_moe_layer_decode_begin if half == "begin" else load().maya_moe_layer_decode_end
            check(fn(C.byref(self.layout), _p(expert_table), self.n_expert, self.k, C.byref(router) if router is not None else None,
                     _p(logits), _p(x), dtype_id(x), nt, limit, _p(add), _p(self.ids), _p(self.weights), _p(self.out), _p(self.ws),
                     self.ws_bytes, _stream(stream)))
            return self.out[:nt]
        if router is not None:
            check(load().maya_moe_layer_decode_routed(C.byref(self.layout), _p(expert_table), self.n_expert, self.k, C.byref(router),
                                                      _p(logits), _p(x), dtype_id(x), nt, limit, _p(add), _p(self.ids),
                                                      _p(self.weights), _p(self.out), _p(self.ws), self.ws_bytes, _stream(stream)))
            return self.out[:nt]
        check(load().maya_moe_layer_decode(C.byref(self.layout), _p(expert_table), self.n_expert, self.k, _p(logits), _p(x),
                                           dtype_id(x), nt, limit, _p(add), _p(self.ids), _p(self.weights), _p(self.out),
                                           _p(self.ws), self.ws_bytes, _stream(stream)))
        return self.out[:nt]


class DenseExpert:
    """The expert every token takes (a shared expert, a dense FFN) through the stage entry points: its plan is static - all
    n tokens on one blob, weight 1, one group - so it is made once here and a step is quantize x -> gate/up -> quantize h
    -> down -> combine, with no routing, plan or grouping launch (the reference runs the shared expert's rows as extra
    blocks of the routed experts' launches, include/strata/kernels/glm_fast.hpp:496-501)."""

    def __init__(self, gate_type, down_type, n_embd, n_ff, n_tokens, blob_addr, packing=PACK_GGUF, device="cuda"):
        self.gguf_layout, self.blob_bytes = layout(gate_type, down_type, n_embd, n_ff)
        self.layout = copy_layout(self.gguf_layout, packing)
        self.n, self.n_embd, self.n_ff = n_tokens, n_embd, n_ff
        n = n_tokens
        self.plan_ptr = torch.full((n,), blob_addr, dtype=torch.int64, device=device)
        self.plan_w = torch.ones(n, dtype=torch.float32, device=device)
        self.grp_ptr, self.grp_start, self.grp_ent, self.n_groups = group(self.plan_ptr)
        self.xq, self.hq = ActBuf(n, n_embd, device), ActBuf(n, n_ff, device)
        self.h = torch.empty((n, n_ff), dtype=torch.float32, device=device)
        self.part = torch.empty((n, n_embd), dtype=torch.float32, device=device)
        self.out = torch.empty((n, n_embd), dtype=torch.float32, device=device)
        a = Args()
        a.layout = self.layout
        a.n_tokens, a.k = n, 1
        a.plan_ptr, a.plan_w = self.plan_ptr.data_ptr(), self.plan_w.data_ptr()
        a.grp_ptr, a.grp_start = self.grp_ptr.data_ptr(), self.grp_start.data_ptr()
        a.grp_ent, a.n_groups = self.grp_ent.data_ptr(), self.n_groups.data_ptr()
        a.x, a.h, a.hq = self.xq.c(), self.h.data_ptr(), self.hq.c()
        a.part, a.out = self.part.data_ptr(), self.out.data_ptr()
        self.args = a

    def forward(self, x, limit=float("inf"), stream=None):
        assert x.shape == (self.n, self.n_embd) and x.is_contiguous()
        L, a, s = load(), self.args, _stream(stream)
        a.limit = limit
        check(L.maya_quant_act(self.layout.gate_type, _p(x), dtype_id(x), 0, self.n, self.n_embd, self.xq.c(), s))
        check(L.maya_moe_gate_up(C.byref(a), s))
        check(L.maya_quant_act(self.layout.down_type, _p(self.h), 0, 0, self.n, self.n_ff, self.hq.c(), s))
        check(L.maya_moe_down(C.byref(a), s))
        return self.out


def mv(jobs, stream=None):
    """jobs: dicts with w (uint8 rows), type, x [ncol, n_in] float activations, n_out and optionally packing, alpha, bias,
    y; quantizes each x to the type's activation format and runs ONE maya_mv call.  Returns the outputs [ncol, n_out]."""
    arr = (MvJob * len(jobs))()
    keep, outs = [], []
    for i, j in enumerate(jobs):
        x = j["x"]
        act = j.get("act") or quant_act(j["type"], x, stream)
        y = j.get("y")
        if y is None:
            y = torch.empty((x.shape[0], j["n_out"]), dtype=torch.float32, device=x.device)
        bias = j.get("bias")
        arr[i] = MvJob(j["w"].data_ptr(), j["type"], j.get("packing", PACK_GGUF), x.shape[1], j["n_out"], x.shape[0],
                       float(j.get("alpha", 1.0)), act.c(), bias.data_ptr() if bias is not None else None, y.data_ptr(),
                       y.stride(0))
        keep.append(act)
        outs.append(y)
    check(load().maya_mv(arr, len(jobs), _stream(stream)))
    return outs

"""ctypes bindings of the CPU checker (oracle/liboracle.so) and, when it was built, of the reference build
(oracle/_ref/libmaya_ref.so).

TEST INFRASTRUCTURE: imported only by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg.  The product
package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
Q8_0, Q4_K, IQ2_XXS, IQ1_S, IQ2_S, IQ1_M = 8, 12, 16, 19, 22, 29

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_vpp = C.POINTER(C.c_void_p)


def _ptr(a, t=C.c_void_p):
    return a.ctypes.data_as(t)


def build(force=False):
    """Compiles liboracle.so (and _ref/libmaya_ref.so when the reference tree is there)."""
    if force or not os.path.exists(os.path.join(HERE, "liboracle.so")):
        subprocess.run(["make", "-C", HERE] + (["-B"] if force else []), check=True, capture_output=True)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(os.path.join(HERE, "liboracle.so"))
        L = _lib
        L.mo_f16_to_f32.restype = C.c_float
        L.mo_f16_to_f32.argtypes = [C.c_uint16]
        L.mo_f32_to_f16.restype = C.c_uint16
        L.mo_f32_to_f16.argtypes = [C.c_float]
        L.mo_f32_to_bf16.restype = C.c_uint16
        L.mo_f32_to_bf16.argtypes = [C.c_float]
        L.mo_bf16_to_f32.restype = C.c_float
        L.mo_bf16_to_f32.argtypes = [C.c_uint16]
        L.mo_iq2s_grid.restype = C.POINTER(C.c_uint64)
        L.mo_iq1s_grid.restype = C.POINTER(C.c_uint64)
        L.mo_iq2xxs_grid.restype = C.POINTER(C.c_uint64)
        L.mo_crc32.restype = C.c_uint32
        L.mo_crc32.argtypes = [C.c_void_p, C.c_size_t]
        L.mo_block_bytes.argtypes = [C.c_int]
        L.mo_block_values.argtypes = [C.c_int]
        L.mo_row_bytes.restype = C.c_size_t
        L.mo_row_bytes.argtypes = [C.c_int, C.c_int64]
        L.mo_dequant_row.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_quant_q8k.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_quant_q80.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_quant_i8x32.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]
        L.mo_act_bytes.restype = C.c_size_t
        L.mo_act_bytes.argtypes = [C.c_int, C.c_int64]
        L.mo_quant_act.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_vec_dot.restype = C.c_float
        L.mo_vec_dot.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_swiglu.restype = C.c_float
        L.mo_swiglu.argtypes = [C.c_float, C.c_float, C.c_float]
        L.mo_expert.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p,
                                C.c_int, C.c_float, C.c_void_p, C.c_int]
        L.mo_router_topk.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.mo_router_topk_f64.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.mo_combine.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_void_p]
        L.mo_moe_layer.argtypes = [C.c_int, C.c_int, _vpp, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_void_p,
                                   C.c_void_p, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.mo_exp_portable.restype = C.c_float
        L.mo_exp_portable.argtypes = [C.c_float]
        L.mo_swiglu_portable.restype = C.c_float
        L.mo_swiglu_portable.argtypes = [C.c_float, C.c_float, C.c_float]
        L.mo_row_lanes.restype = C.c_float
        L.mo_row_lanes.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_int]
        L.mo_exl3_decode.restype = C.c_float
        L.mo_exl3_decode.argtypes = [C.c_uint32, C.c_int]
        L.mo_exl3_tile_states.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.mo_exl3_inner.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
        L.mo_exl3_had128.argtypes = [C.c_void_p, C.c_size_t]
        L.mo_exl3_mv.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.mo_encode_q4k.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_encode_q80.argtypes = [C.c_void_p, C.c_int64, C.c_void_p]
        L.mo_grouped_ref.argtypes = [C.c_int, _vpp, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p,
                                     C.c_void_p, C.c_int]
    return _lib


def ref():
    """The reference build, or None where it was not built (no reference tree in this container)."""
    global _ref
    if _ref is None:
        path = os.path.join(HERE, "_ref", "libmaya_ref.so")
        if not os.path.exists(path):
            return None
        R = C.CDLL(path)
        R.ref_f16_to_f32.restype = C.c_float
        R.ref_f16_to_f32.argtypes = [C.c_uint16]
        R.ref_f32_to_f16.restype = C.c_uint16
        R.ref_f32_to_f16.argtypes = [C.c_float]
        R.ref_dequant_q4_K.argtypes = [C.c_void_p, C.c_void_p]
        R.ref_dequant_q8_0.argtypes = [C.c_void_p, C.c_void_p]
        R.ref_iq256_supported.argtypes = [C.c_int]
        R.ref_iq256_rows.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_int, _vpp, C.c_int, _vpp, C.c_int, C.c_int]
        R.ref_iq256_gu_rows.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, _vpp, C.c_int, _vpp,
                                        C.c_int, C.c_int]
        R.ref_par_act_bytes.restype = C.c_size_t
        R.ref_par_act_bytes.argtypes = [C.c_int]
        R.ref_par_quant.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        R.ref_par_row.restype = C.c_float
        R.ref_par_row.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        R.ref_exp_portable.restype = C.c_float
        R.ref_exp_portable.argtypes = [C.c_float]
        R.ref_swiglu_portable.restype = C.c_float
        R.ref_swiglu_portable.argtypes = [C.c_float, C.c_float, C.c_float]
        R.ref_exl3_decode.restype = C.c_float
        R.ref_exl3_decode.argtypes = [C.c_uint32, C.c_int]
        R.ref_exl3_tile_states.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        R.ref_exl3_inner.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
        R.ref_exl3_had128.argtypes = [C.c_void_p, C.c_size_t]
        R.ref_exl3_mv.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        _ref = R
    return _ref


# ---------------------------------------------------------------------------------------------- numpy-level helpers

def row_bytes(t, k):
    return int(lib().mo_row_bytes(t, k))


def dequant_rows(t, w, k, n):
    """w: uint8 array holding n rows of k values -> float32 [n, k]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    rb = row_bytes(t, k)
    out = np.empty((n, k), dtype=np.float32)
    for r in range(n):
        rc = lib().mo_dequant_row(t, w.ctypes.data + r * rb, k, out[r].ctypes.data)
        assert rc == 0
    return out


def quant_q8k(x):
    """x float32 [k] -> (bytes of k/256 block_q8_K as uint8 array)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros((x.size // 256) * 292, dtype=np.uint8)
    lib().mo_quant_q8k(_ptr(x), x.size, _ptr(out))
    return out


def q8k_fields(blocks):
    """block_q8_K bytes -> (d float32 [nb], qs int8 [nb*256], bsums int16 [nb, 16])."""
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, 292)
    d = b[:, 0:4].copy().view(np.float32).reshape(-1)
    qs = b[:, 4:260].copy().view(np.int8).reshape(-1)
    bs = b[:, 260:292].copy().view(np.int16).reshape(-1, 16)
    return d, qs, bs


def quant_act(t, x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(int(lib().mo_act_bytes(t, x.size)), dtype=np.uint8)
    lib().mo_quant_act(t, _ptr(x), x.size, _ptr(out))
    return out


def quant_i8x32(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.zeros(x.size, dtype=np.int8)
    d = np.zeros(x.size // 32, dtype=np.float32)
    lib().mo_quant_i8x32(_ptr(x), x.size, _ptr(q), _ptr(d))
    return q, d


def vec_dot(t, row, k, act):
    row = np.ascontiguousarray(row, dtype=np.uint8)
    return float(lib().mo_vec_dot(t, _ptr(row), k, _ptr(act)))


def rows(t, w, k, n, act):
    return rows_of(t, w, k, n, act)


def rows_of(t, w, k, n, act):
    """w: n rows of type t; act: quantized activation bytes -> float32 [n]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    rb = row_bytes(t, k)
    out = np.empty(n, dtype=np.float32)
    f = lib().mo_vec_dot
    for r in range(n):
        out[r] = f(t, w.ctypes.data + r * rb, k, _ptr(act))
    return out


def expert(gu_type, d_type, gate, up, down, n_embd, n_ff, x, limit=float("inf"), nthreads=8):
    """x float32 [nt, n_embd] -> out float32 [nt, n_embd]."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_embd)
    out = np.zeros((x.shape[0], n_embd), dtype=np.float32)
    lib().mo_expert(gu_type, d_type, _ptr(gate), _ptr(up), _ptr(down), n_embd, n_ff, _ptr(x), x.shape[0], limit,
                    _ptr(out), nthreads)
    return out


def router_topk(logits, k, f64=False):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    nt, ne = logits.shape
    ids = np.zeros((nt, k), dtype=np.int32)
    w = np.zeros((nt, k), dtype=np.float32)
    (lib().mo_router_topk_f64 if f64 else lib().mo_router_topk)(_ptr(logits), nt, ne, k, _ptr(ids), _ptr(w))
    return ids, w


def router_sigmoid(logits, bias, k, w_scale=1.0, norm=1, f64=False):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    nt, ne = logits.shape
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    ids = np.zeros((nt, k), dtype=np.int32)
    w = np.zeros((nt, k), dtype=np.float32)
    f = lib().mo_router_sigmoid_f64 if f64 else lib().mo_router_sigmoid
    f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p]
    f.restype = None
    f(_ptr(logits), None if b is None else _ptr(b), nt, ne, k, w_scale, norm, _ptr(ids), _ptr(w))
    return ids, w


def plan_tiered(ids, layer, n_expert, tab, scratch, counts=None, seq=None, promote_min=0):
    """The residency plan of routed ids [nt, k] against tab (uint64, edited in place: HBM | second tier | spares); counts
    (uint32 [n_keys]) and seq (uint32 [1]) are edited in place too.  Returns plan, fetch_src (uint64 [nt, k]), masks [nt, 4]."""
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    nt, k = ids.shape
    assert tab.dtype == np.uint64 and tab.flags.c_contiguous
    scratch = np.ascontiguousarray(scratch, dtype=np.uint64)
    plan = np.zeros((nt, k), dtype=np.uint64)
    src = np.zeros((nt, k), dtype=np.uint64)
    masks = np.zeros((nt, 4), dtype=np.uint32)
    f = lib().mo_plan_tiered
    f.restype = None
    f.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                  C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    n_layers = tab.size // (2 * n_expert + 3)
    assert n_layers * (2 * n_expert + 3) == tab.size
    f(_ptr(ids), nt, layer, n_expert, k, _ptr(tab), n_layers * n_expert, _ptr(scratch) if scratch.size else None, scratch.size,
      None if counts is None else _ptr(counts), None if seq is None else _ptr(seq), promote_min, _ptr(plan), _ptr(src), _ptr(masks))
    return plan, src, masks


def combine(parts, w):
    parts = np.ascontiguousarray(parts, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.zeros(parts.shape[1], dtype=np.float32)
    lib().mo_combine(_ptr(parts), _ptr(w), parts.shape[0], parts.shape[1], _ptr(out))
    return out


def moe_layer(gu_type, d_type, blobs, k, n_embd, n_ff, logits, x, limit=float("inf"), nthreads=8):
    """blobs: list of uint8 arrays (one [gate|up|down] blob an expert); logits [nt, ne]; x [nt, n_embd]."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, n_embd)
    nt, ne = logits.shape
    ptrs = (C.c_void_p * ne)(*[b.ctypes.data for b in blobs])
    ids = np.zeros((nt, k), dtype=np.int32)
    w = np.zeros((nt, k), dtype=np.float32)
    out = np.zeros((nt, n_embd), dtype=np.float32)
    lib().mo_moe_layer(gu_type, d_type, ptrs, ne, k, n_embd, n_ff, _ptr(logits), _ptr(x), nt, limit, _ptr(ids), _ptr(w),
                       _ptr(out), nthreads)
    return ids, w, out


def encode_q4k(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros((x.size // 256) * 144, dtype=np.uint8)
    lib().mo_encode_q4k(_ptr(x), x.size, _ptr(out))
    return out


def encode_q80(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros((x.size // 32) * 34, dtype=np.uint8)
    lib().mo_encode_q80(_ptr(x), x.size, _ptr(out))
    return out


def exl3_inner(trellis, k, n, k2, cb):
    trellis = np.ascontiguousarray(trellis, dtype=np.uint32)
    w = np.zeros((k, n), dtype=np.float32)
    lib().mo_exl3_inner(_ptr(trellis), n // 16, k, n, k2, cb, _ptr(w))
    return w


def exl3_mv(w, suh, svh, x):
    k, n = w.shape
    w = np.ascontiguousarray(w, dtype=np.float32)
    suh = np.ascontiguousarray(suh, dtype=np.uint16)
    svh = np.ascontiguousarray(svh, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(n, dtype=np.float32)
    lib().mo_exl3_mv(_ptr(w), _ptr(suh), _ptr(svh), k, n, _ptr(x), _ptr(y))
    return y


def grouped_ref(t, mats, bounds, k, n, xq, xd, nthreads=8):
    """mats: one uint8 array an expert (n rows of k values of type t, or None where the expert has no rows); rows
    bounds[e] .. bounds[e + 1] of xq / xd are expert e's.  Returns float32 [rows, n]: the double products of the
    dequantized weights with the dequantized int8 rows."""
    ne = len(mats)
    bounds = np.ascontiguousarray(bounds, dtype=np.int32)
    xq = np.ascontiguousarray(xq, dtype=np.int8)
    xd = np.ascontiguousarray(xd, dtype=np.float32)
    keep = [None if m is None else np.ascontiguousarray(m, dtype=np.uint8) for m in mats]
    ptrs = (C.c_void_p * ne)(*[None if m is None else m.ctypes.data for m in keep])
    y = np.zeros((int(bounds[ne]), n), dtype=np.float32)
    lib().mo_grouped_ref(t, ptrs, _ptr(bounds), ne, k, n, _ptr(xq), _ptr(xd), _ptr(y), nthreads)
    return y


def prefill_plan(ids, n_expert, resident=None):
    """The stable sort of the entries e = t * k + j by expert: bounds [n_expert + 1], row_entry [rows], entry_row
    [entries] (-1 where the expert is not resident or the id is out of range) (src/kernels/cuda/glm_batch.cu:2102-2133)."""
    flat = np.asarray(ids, dtype=np.int64).reshape(-1)
    ok = (flat >= 0) & (flat < n_expert)
    if resident is not None:
        ok &= np.asarray(resident, dtype=bool)[np.clip(flat, 0, n_expert - 1)]
    ent = np.nonzero(ok)[0]
    order = ent[np.argsort(flat[ent], kind="stable")]
    counts = np.bincount(flat[ent], minlength=n_expert)
    bounds = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    entry_row = np.full(flat.size, -1, dtype=np.int32)
    entry_row[order] = np.arange(order.size, dtype=np.int32)
    return bounds, order.astype(np.int32), entry_row


def swiglu_rows(g, u, limit):
    g = np.asarray(g, dtype=np.float32)
    u = np.asarray(u, dtype=np.float32)
    if limit > 0 and np.isfinite(limit):
        g = np.minimum(g, np.float32(limit))
        u = np.clip(u, -np.float32(limit), np.float32(limit))
    return (g / (np.float32(1) + np.exp(-g)) * u).astype(np.float32)


def prefill_layer(t, blobs, up_off, down_off, n_embd, n_ff, logits, x, k, limit=0.0, resident=None, nthreads=8):
    """A prompt chunk's routed experts as the reference's CPU expert path computes each of them (Q8_K rows of x, the
    gate / up row dots, the clamped SwiGLU, h rounded to Q8_K, the down row dots: src/kernels/cpu/native_expert.cpp:306-442)
    in the plan's row order (src/kernels/cuda/glm_batch.cu:2102-2133), and the weighted sum in slot order.  Returns a dict
    of every stage: xq / xd / xs = the rows' codes, block scales and the integer sum of every 32 codes; h = the SwiGLU values."""
    tg, td = t if isinstance(t, tuple) else (t, t)   # (gate/up type, down type)
    ids, w = router_topk(logits, k)
    ne = len(blobs)
    bounds, row_entry, entry_row = prefill_plan(ids, ne, resident)
    rows = row_entry.size
    lim = float(limit) if limit and limit > 0 else float("inf")
    xq = np.zeros((rows, n_embd), dtype=np.int8)
    xd = np.zeros((rows, n_embd // 256), dtype=np.float32)
    xs = np.zeros((rows, n_embd // 32), dtype=np.int32)
    h = np.zeros((rows, n_ff), dtype=np.float32)
    part = np.zeros((rows, n_embd), dtype=np.float32)
    acts = {}
    sw = lib().mo_swiglu
    for r in range(rows):
        tok, e = int(row_entry[r]) // k, int(ids.reshape(-1)[row_entry[r]])
        if tok not in acts:
            a = quant_act(tg, x[tok])
            d, q, bs = q8k_fields(a)
            acts[tok] = (a, q, d, (bs[:, 0::2].astype(np.int32) + bs[:, 1::2]).reshape(-1))
        a, xq[r], xd[r], xs[r] = acts[tok]
        b = blobs[e]
        g = rows_of(tg, b, n_embd, n_ff, a)
        u = rows_of(tg, b[up_off:], n_embd, n_ff, a)
        h[r] = [sw(float(gv), float(uv), lim) for gv, uv in zip(g, u)]
        part[r] = rows_of(td, b[down_off:], n_ff, n_embd, quant_act(td, h[r]))
    out = np.zeros((x.shape[0], n_embd), dtype=np.float32)
    for tok in range(x.shape[0]):
        sel = [j for j in range(k) if entry_row[tok * k + j] >= 0]
        if sel:
            out[tok] = combine(np.stack([part[entry_row[tok * k + j]] for j in sel]), np.array([w[tok, j] for j in sel]))
    return dict(ids=ids, w=w, bounds=bounds, row_entry=row_entry, entry_row=entry_row, xq=xq, xd=xd, xs=xs, h=h,
                part=part, out=out)

"""Helpers of the GPU parity tests: seeded inputs, the oracle's layer on the host, error metrics."""
import numpy as np
import torch

import synth
from maya_amd import lib


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    want = np.asarray(want, dtype=np.float64).reshape(-1)
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_experts(gate_type, down_type, n_embd, n_ff, n_expert, seed, up_type=None):
    rng = np.random.default_rng(seed)
    return [synth.expert_blob(gate_type, down_type, n_embd, n_ff, rng, up_type) for _ in range(n_expert)]


def oracle_layer(oracle, gate_type, down_type, blobs, k, n_embd, n_ff, logits, x, limit=float("inf"), up_type=None,
                 skip=(), route=None):
    """The reference CPU path on the host: router, each routed expert (ggml contract), weighted sum in slot order.
    `skip`: expert ids whose blob is not resident (their part is left out).  Returns ids, weights, out, h."""
    up_type = gate_type if up_type is None else up_type
    ids, w = route(logits, k) if route else oracle.router_topk(logits, k)
    up_off, down_off, _ = synth.blob_offsets(gate_type, down_type, n_embd, n_ff, up_type)
    nt = x.shape[0]
    out = np.zeros((nt, n_embd), dtype=np.float32)
    L = oracle.lib()
    for t in range(nt):
        parts, ws = [], []
        for i in range(k):
            e = int(ids[t, i])
            if e in skip:
                continue
            b = blobs[e]
            if up_type == gate_type:
                p = oracle.expert(gate_type, down_type, b, b[up_off:], b[down_off:], n_embd, n_ff, x[t:t + 1], limit)[0]
            else:
                act = oracle.quant_act(gate_type, x[t])
                g = oracle.rows(gate_type, b, n_embd, n_ff, act)
                u = oracle.rows(up_type, b[up_off:], n_embd, n_ff, act)
                h = np.array([L.mo_swiglu(float(a), float(c), limit) for a, c in zip(g, u)], dtype=np.float32)
                p = oracle.rows(down_type, b[down_off:], n_ff, n_embd, oracle.quant_act(down_type, h))
            parts.append(p)
            ws.append(w[t, i])
        if parts:
            out[t] = oracle.combine(np.stack(parts), np.array(ws, dtype=np.float32))
    return ids, w, out


# ---- the EXL3 layer on the host (the checker decodes each matrix once an expert)

def swiglu(g, u, limit):
    g = g.astype(np.float32)
    u = u.astype(np.float32)
    if limit > 0 and np.isfinite(limit):
        g = np.minimum(g, np.float32(limit))
        u = np.clip(u, -np.float32(limit), np.float32(limit))
    return (g / (np.float32(1) + np.exp(-g)) * u).astype(np.float32)


class HostExpert:
    def __init__(self, ex, oracle, l, blob):
        self.m = []
        for r in range(3):
            k, n = ex.matrix_of(l, r)
            tr, suh, svh = ex.parts_of(l, blob, r)
            self.m.append((oracle.exl3_inner(tr, k, n, l.k2[r], l.cb), suh, svh))
        self.oracle = oracle

    def h(self, x, limit):
        g = self.oracle.exl3_mv(*self.m[0], x)
        u = self.oracle.exl3_mv(*self.m[1], x)
        return swiglu(g, u, limit)

    def part(self, h):
        return self.oracle.exl3_mv(*self.m[2], h)


def host_layer(oracle, experts, ids, w, x, limit, skip=()):
    nt, k = ids.shape
    hs = np.zeros((nt * k, experts[0].m[0][0].shape[1]), dtype=np.float32)
    out = np.zeros((nt, x.shape[1]), dtype=np.float32)
    for t in range(nt):
        parts, ws = [], []
        for i in range(k):
            e = int(ids[t, i])
            if e in skip:
                continue
            hs[t * k + i] = experts[e].h(x[t], limit)
            parts.append(experts[e].part(hs[t * k + i]))
            ws.append(w[t, i])
        if parts:
            out[t] = oracle.combine(np.stack(parts), np.array(ws, dtype=np.float32))
    return out, hs

#!/usr/bin/env python3
"""bench.py - the routed MoE decode layer on one MI355X (BASELINE.json configs[1]).

A step is one pass of the layer over one token: router top-8 of 256 experts, plan, Q8_K rounding of the bf16 hidden
state, fused dequant gate/up GLU mat-vec over the 8 routed IQ2_S experts, Q8_K rounding of h, down mat-vec, weighted
combine.  All 256 experts (3.6 GB) are resident in HBM; consecutive steps route to disjoint expert sets (32 sets of 8),
so no step re-reads weights that an earlier step left in the on-die caches.  The K timed steps are one HIP graph
(the reference's timing method, tests/hip/expert_kernel_bench.cpp:136-172), bracketed by device synchronisations.

value = algorithmic HBM bytes of a step (weights of the 8 routed experts + logits + x + out) / time per step, GB/s.
roofline = the gate/up kernel alone: its algorithmic bytes / its average duration measured with HIP events.
cpu_baseline = the reference's CPU expert path on this host's cores, same inputs, a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "project-maya_amd"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

N_EMBD, N_FF, N_EXPERT, TOP_K = 7168, 2048, 256, 8
IQ2_S = 22
HBM_PEAK = 8.0e12
# HBM bytes of one gate/up launch on this workload from rocprofv3's FETCH_SIZE and WRITE_SIZE (two runs, each scaled by
# what the counter reads for a plain device copy of known size: 2.000 and 1.000): 73,783.1 KiB read + 64.0 KiB written
# (profiles/decode_iq2s_hbm_traffic_pmc.txt)
GATE_UP_TRAFFIC_BYTES = int((73783.1 + 64.0) * 1024)


def synth_experts_on_device(torch, n_expert, blob_bytes, seed):
    """Constructed IQ2_S blocks made on the device: random bytes, each 82-byte block's FP16 scale drawn from
    [2e-3, 6e-3] (the reference's fixture range, tools/iq_fixture.py:55).  Returns the pool and the address table."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    assert blob_bytes % 82 == 0
    pool = torch.empty(n_expert * blob_bytes, dtype=torch.uint8, device="cuda")
    chunk = 32 * blob_bytes
    for o in range(0, pool.numel(), chunk):
        n = min(chunk, pool.numel() - o)
        pool[o:o + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    blocks = pool.view(-1, 82)
    d = (torch.rand(blocks.shape[0], device="cuda", generator=g) * 4e-3 + 2e-3).to(torch.float16)
    blocks[:, 0:2] = d.view(torch.uint8).view(-1, 2)
    base = pool.data_ptr()
    table = torch.tensor([base + e * blob_bytes for e in range(n_expert)], dtype=torch.int64, device="cuda")
    return pool, table


def rotating_logits(np, n_sets, seed):
    """N(0,1) router logits for n_sets steps whose top-8 sets are the disjoint expert ranges 8 j .. 8 j + 7: each row is
    an i.i.d. N(0,1) sample with its expert axis permuted (still i.i.d. N(0,1))."""
    rng = np.random.default_rng(seed)
    out = np.zeros((n_sets, N_EXPERT), dtype=np.float32)
    for j in range(n_sets):
        v = rng.standard_normal(N_EXPERT).astype(np.float32)
        order = np.argsort(-v, kind="stable")
        want = np.concatenate([np.arange(8 * j, 8 * j + 8), np.setdiff1d(np.arange(N_EXPERT), np.arange(8 * j, 8 * j + 8))])
        row = np.zeros(N_EXPERT, dtype=np.float32)
        row[want] = v[order]
        out[j] = row
    return out


def cpu_baseline(np, torch, oracle_py, pool, blob_bytes, logits_row, x_f32, gpu_out):
    """The reference CPU expert path for one step's 8 routed experts on this host's cores: Q8_K activation, gate/up rows,
    SwiGLU, Q8_K of h, down rows, weighted sum - rows split over the threads as ExpertPool::run_split_multi_native does.
    Uses the reference build (oracle/_ref, the reference's own iq_avx2.cpp) when it travelled here, else the C port."""
    import ctypes as C
    from concurrent.futures import ThreadPoolExecutor
    cores = max(1, min(16, len(os.sched_getaffinity(0))))
    ids, w = oracle_py.router_topk(logits_row[None, :], TOP_K)
    ids, w = ids[0], w[0]
    blobs = [pool[int(e) * blob_bytes:(int(e) + 1) * blob_bytes].cpu().numpy() for e in ids]
    gr, dr = oracle_py.row_bytes(IQ2_S, N_EMBD), oracle_py.row_bytes(IQ2_S, N_FF)
    up_off, down_off = gr * N_FF, 2 * gr * N_FF
    ref = oracle_py.ref()
    kind = "reference" if ref is not None else "port"
    pool_ex = ThreadPoolExecutor(cores)

    def one_layer():
        act = oracle_py.quant_q8k(x_f32)
        actp = (C.c_void_p * 1)(act.ctypes.data)
        parts = np.zeros((TOP_K, N_EMBD), dtype=np.float32)
        for i, b in enumerate(blobs):
            h = np.zeros(N_FF, dtype=np.float32)
            hp = (C.c_void_p * 1)(h.ctypes.data)
            if ref is not None:
                def gu(c):
                    ref.ref_iq256_gu_rows(IQ2_S, b.ctypes.data, gr, up_off, N_EMBD, actp, 1, hp, c[0], c[1])
            else:
                def gu(c):
                    oracle_py.lib().mo_gu_rows(IQ2_S, b.ctypes.data, b.ctypes.data + up_off, gr, N_EMBD, actp, 1, hp, c[0],
                                               c[1], float("inf"))
            step = N_FF // (cores * 4)
            list(pool_ex.map(gu, [(r, min(N_FF, r + step)) for r in range(0, N_FF, step)]))
            hq = oracle_py.quant_q8k(h)
            hqp = (C.c_void_p * 1)(hq.ctypes.data)
            op = (C.c_void_p * 1)(parts[i].ctypes.data)
            if ref is not None:
                def dn(c):
                    ref.ref_iq256_rows(IQ2_S, b.ctypes.data + down_off, dr, N_FF, hqp, 1, op, c[0], c[1])
            else:
                def dn(c):
                    oracle_py.lib().mo_rows(IQ2_S, b.ctypes.data + down_off, dr, N_FF, hqp, 1, op, c[0], c[1])
            step = N_EMBD // (cores * 4)
            list(pool_ex.map(dn, [(r, min(N_EMBD, r + step)) for r in range(0, N_EMBD, step)]))
        return oracle_py.combine(parts, w)

    if ref is None:
        L = oracle_py.lib()
        L.mo_gu_rows.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int64, C.c_void_p, C.c_int, C.c_void_p,
                                 C.c_int, C.c_int, C.c_float]
        L.mo_rows.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_int64, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int]
    out = one_layer()  # warm-up, and the parity check of the GPU result
    err = float(np.linalg.norm(out.astype(np.float64) - gpu_out.astype(np.float64)) / np.linalg.norm(out.astype(np.float64)))
    times = []
    t_end = time.perf_counter() + 12.0
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 40):
        t0 = time.perf_counter()
        one_layer()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    bytes_step = TOP_K * blob_bytes
    return {"value": round(bytes_step / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind,
            "us_per_step": round(med * 1e6, 1),
            "sample": "%d layer calls of the same 8 routed IQ2_S experts (%d MB of weights each call), median" % (
                len(times), bytes_step // 1000000)}, err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-graph", action="store_true", help="launch the timed steps eagerly instead of as one HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--workload", default="decode_iq2s",
                    help="decode_iq2s (configs[1], the default and the headline metric), or one of the other BASELINE "
                         "configurations: single_q4k, batch8_mixed, prefill_q4k, exl3_verify; the prefill chunk on other expert types: "
                         "prefill_iq2s, prefill_mixed")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (nothing here uses a second GPU)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from maya_amd import lib

    L = lib.load()
    lib.check(L.maya_init())
    info = L.maya_device_info().decode()
    torch.cuda.set_device(0)
    if args.calib_copy:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.workload != "decode_iq2s":
        import bench_workloads as workloads
        if args.workload not in workloads.WORKLOADS:
            sys.exit("bench.py: unknown workload %r" % args.workload)
        r = workloads.WORKLOADS[args.workload](args.steps, args.warmup)
        r["config"]["device"] = info
        line = {"metric": r["metric"], "value": r["value"], "unit": r["unit"], "n_gpus": 1, "steps": args.steps,
                "warmup": args.warmup, "ms_per_step": round(r["ms_per_step"], 6), "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic", "config": r["config"], "roofline": r["roofline"],
                "cpu_baseline": None}
        print(json.dumps(line))
        return
    layer = lib.MoeLayer(IQ2_S, IQ2_S, N_EMBD, N_FF, N_EXPERT, TOP_K, max_tokens=1, packing=lib.PACK_STREAM)
    blob_bytes = layer.blob_bytes
    # GGUF blobs are made on the device, then regrouped into the stream packing as an engine's upload would do;
    # the GGUF copy stays for the CPU baseline (it reads the file's own layout)
    gguf_pool, _ = synth_experts_on_device(torch, N_EXPERT, blob_bytes, 20261125)
    pool = torch.empty_like(gguf_pool)
    for e in range(N_EXPERT):
        lib.repack(layer.gguf_layout, gguf_pool[e * blob_bytes:(e + 1) * blob_bytes], pool[e * blob_bytes:(e + 1) * blob_bytes])
    torch.cuda.synchronize()
    base = pool.data_ptr()
    assert base % 16 == 0
    table = torch.tensor([base + e * blob_bytes for e in range(N_EXPERT)], dtype=torch.int64, device="cuda")
    n_sets = N_EXPERT // TOP_K
    logits_np = rotating_logits(np, n_sets, 7)
    logits = torch.from_numpy(logits_np).cuda()
    rng = np.random.default_rng(11)
    x = torch.from_numpy(rng.standard_normal((1, N_EMBD)).astype(np.float32)).to(torch.bfloat16).cuda()
    torch.cuda.synchronize()

    stream = torch.cuda.Stream()
    K, W = args.steps, args.warmup

    def step(i):
        layer.forward(table, logits[i % n_sets:i % n_sets + 1], x)

    with torch.cuda.stream(stream):
        for i in range(W):
            step(i)
        stream.synchronize()
        graph = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(K):
                    step(W + i)
            graph.replay()  # one untimed replay: the graph's first launch uploads it
            stream.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if graph is not None:
            graph.replay()
        else:
            for i in range(K):
                step(W + i)
        stream.synchronize()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0

        # ---- the dominant kernel alone (gate/up: 2/3 of the bytes), HIP events on the launch stream
        import ctypes as C
        ids_all, w_all = lib.route_topk(logits, TOP_K)
        plans = lib.plan(ids_all.view(-1), table).view(n_sets, TOP_K)
        xq = lib.quant_act(IQ2_S, x.to(torch.float32))
        h = torch.empty((TOP_K, N_FF), dtype=torch.float32, device="cuda")
        a = lib.Args()
        a.layout = layer.layout
        a.n_tokens, a.k = 1, TOP_K
        a.limit = float("inf")
        a.x = xq.c()
        a.h = h.data_ptr()
        arg_list = []
        for j in range(n_sets):
            b = lib.Args()
            C.memmove(C.byref(b), C.byref(a), C.sizeof(a))
            b.plan_ptr = plans[j].data_ptr()
            b.plan_w = w_all[j].data_ptr()
            arg_list.append(b)
        sp = C.c_void_p(stream.cuda_stream)
        for j in range(8):
            lib.check(L.maya_moe_gate_up(C.byref(arg_list[j]), sp))
        stream.synchronize()
        reps = max(K, 64)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        kg = torch.cuda.CUDAGraph()
        with torch.cuda.graph(kg, stream=stream):
            for j in range(reps):
                lib.check(L.maya_moe_gate_up(C.byref(arg_list[(8 + j) % n_sets]), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        kg.replay()
        stream.synchronize()
        e0.record(stream)
        kg.replay()
        e1.record(stream)
        stream.synchronize()
        gu_us = e0.elapsed_time(e1) * 1e3 / reps

    step_us = dt / K * 1e6
    w_bytes = TOP_K * blob_bytes
    bytes_step = w_bytes + N_EXPERT * 4 + N_EMBD * 2 + N_EMBD * 4
    value = bytes_step / (dt / K) / 1e9
    gu_bytes = TOP_K * 2 * N_FF * lib.row_bytes(IQ2_S, N_EMBD) + N_EMBD + (N_EMBD // 32) * 4 + TOP_K * N_FF * 4
    gu_rate = gu_bytes / (gu_us * 1e-6) / 1e9

    # ---- parity of the timed configuration + CPU baseline on the same inputs
    with torch.cuda.stream(stream):
        out0 = layer.forward(table, logits[0:1], x).clone()
        ids0 = layer.ids.clone()
        stream.synchronize()
    cpu, err = (None, None)
    if not args.no_cpu:
        import oracle_py
        cpu, err = cpu_baseline(np, torch, oracle_py, gguf_pool, blob_bytes, logits_np[0], x.to(torch.float32).cpu().numpy()[0],
                                out0.cpu().numpy()[0])
        wi, _ = oracle_py.router_topk(logits_np[0:1], TOP_K)
        if not np.array_equal(wi, ids0.cpu().numpy()[:1]):
            err = float("inf")

    line = {
        "metric": "moe_layer_decode_hbm_gbps_1tok",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(step_us / 1e3, 6),
        "us_per_layer": round(step_us, 3),
        "pct_of_hbm_peak": round(100.0 * value * 1e9 / HBM_PEAK, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "configs[1]: routed MoE decode layer, 1 token, hidden 7168 bf16, 256 experts x (gate/up "
                               "[2048x7168] + down [7168x2048]) IQ2_S, softmax top-8 renormalised; 32 disjoint expert sets "
                               "rotate over the steps",
                   "n_embd": N_EMBD, "n_ff": N_FF, "n_expert": N_EXPERT, "top_k": TOP_K, "tokens": 1,
                   "weight_bytes_per_step": w_bytes, "algorithmic_bytes_per_step": bytes_step,
                   "timed_as": "eager launches" if args.no_graph else "one HIP graph of the K steps", "device": info},
        "roofline": {"bound": "hbm", "kernel": "gate_up_iq2s_pos_kernel", "achieved": round(gu_rate, 2), "peak": 8000.0,
                     "unit": "GB/s", "frac": round(gu_rate * 1e9 / HBM_PEAK, 4), "traffic": GATE_UP_TRAFFIC_BYTES,
                     "algorithmic_bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_us, 3)},
        "cpu_baseline": cpu,
        "parity_rel_l2_vs_cpu_path": err,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

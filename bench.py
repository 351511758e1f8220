#!/usr/bin/env python3
"""bench.py - the routed MoE expert block on one MI355X: BASELINE.json's metric on configs[1] (the decode layer), with
configs[3] (the 512-token prompt chunk, the metric's second half) as a sub-object of the same line.

A decode step is one pass of the layer over one token: router top-8 of 256 experts, plan, Q8_K rounding of the bf16 hidden
state, fused dequant gate/up GLU mat-vec over the 8 routed IQ2_S experts, Q8_K rounding of h, down mat-vec, weighted
combine.  All 256 experts (3.6 GB) are resident in HBM; consecutive steps route to disjoint expert sets (32 sets of 8),
so no step re-reads weights that an earlier step left in the on-die caches.  The K steps are one HIP graph (the
reference's timing method, tests/hip/expert_kernel_bench.cpp:136-172): untimed replays until two in a row agree within
1 %, then 7 timed samples - each the graph replayed back to back (at least 256 steps and 10 ms of GPU work) between two
HIP events on the launch stream - the median; the figure does not move with --steps.

value = algorithmic HBM bytes of a step (weights of the 8 routed experts + logits + x + out) / time per step, GB/s.
roofline = the dominant kernel (gate/up: two thirds of the bytes): its algorithmic bytes / its average launch duration
measured with HIP events on the launch stream; roofline.layer = the same for the whole step.
cpu_baseline = the reference's CPU expert path on this host's physical cores (pinned pool, rotating expert sets, median).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "project-maya_amd"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

N_EMBD, N_FF, N_EXPERT, TOP_K = 7168, 2048, 256, 8
IQ2_S = 22
HBM_PEAK = 8.0e12
PARITY_BAR = 1e-3
# HBM bytes of one gate/up launch on this workload from rocprofv3's FETCH_SIZE and WRITE_SIZE (two runs, each scaled by
# what the counter reads for a plain device copy of known size: 2.000 and 1.000): 74,179.7 KiB read + 64.1 KiB written
# (profiles/decode_iq2s_hbm_traffic_pmc.txt)
GATE_UP_TRAFFIC_BYTES = int((74179.7 + 64.1) * 1024)


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


def physical_cores(limit=16):
    """One logical CPU per physical core among those this process may run on (the reference pins one worker per physical
    core, include/strata/kernels/cpu/pool.hpp:66-72), at most `limit`; and the CPU's model string."""
    allowed = sorted(os.sched_getaffinity(0))
    seen, cpus = set(), []
    for c in allowed:
        try:
            sib = open("/sys/devices/system/cpu/cpu%d/topology/thread_siblings_list" % c).read().strip()
        except OSError:
            sib = str(c)
        if sib not in seen:
            seen.add(sib)
            cpus.append(c)
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return cpus[:limit], len(cpus), model


def cpu_baseline(np, oracle_py, gguf_pool, blob_bytes, logits_np, x_f32, n_sets=5, max_seconds=10.0):
    """The reference CPU expert path for one token's 8 routed experts on this host: oracle/cpu_bench.c's pinned spinning
    pool, rows split over the threads as ExpertPool::run_split_multi_native does, n_sets disjoint expert sets (5 x 113 MB)
    rotating so every call streams from DRAM, at least 7 passes over the sets, the median call.  The row kernels are the
    reference's own iq_avx2.cpp (oracle/_ref, kind "reference") when that build travelled here, else the C port.
    Returns the cpu_baseline object and the output of the last call (expert set n_sets - 1)."""
    cpus, n_phys, model = physical_cores()
    ids, w = oracle_py.router_topk(logits_np[:n_sets], TOP_K)
    host = [gguf_pool[int(e) * blob_bytes:(int(e) + 1) * blob_bytes].cpu().numpy() for e in ids.reshape(-1)]
    blobs = (C.c_void_p * len(host))(*[b.ctypes.data for b in host])
    ref = oracle_py.ref()
    L = oracle_py.lib()
    gu = C.cast(ref.ref_iq256_gu_rows, C.c_void_p) if ref is not None else None
    rows = C.cast(ref.ref_iq256_rows, C.c_void_p) if ref is not None else None
    rounds = 600
    times = np.zeros(rounds * n_sets, dtype=np.float64)
    n_done = C.c_int(0)
    out = np.zeros(N_EMBD, dtype=np.float32)
    cpu_arr = (C.c_int * len(cpus))(*cpus)
    wts = np.ascontiguousarray(w, dtype=np.float32)
    x = np.ascontiguousarray(x_f32, dtype=np.float32)
    L.mo_bench_layer.restype = C.c_int
    L.mo_bench_layer.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_double, C.c_void_p, C.c_void_p, C.c_void_p]
    rc = L.mo_bench_layer(IQ2_S, blobs, n_sets, TOP_K, N_EMBD, N_FF, x.ctypes.data, wts.ctypes.data, gu, rows, len(cpus), cpu_arr,
                          rounds, max_seconds, times.ctypes.data, C.byref(n_done), out.ctypes.data)
    if rc != 0 or n_done.value < 1:
        return None, None
    t = np.sort(times[:n_done.value])
    med = float(t[len(t) // 2])
    bytes_step = TOP_K * blob_bytes
    return {"value": round(bytes_step / med / 1e9, 2), "unit": "GB/s", "cores": len(cpus), "kind": "reference" if ref is not None else "port",
            "us_per_step": round(med * 1e6, 1), "cpu_model": model, "physical_cores_available": n_phys,
            "sample": "%d layer calls (%d passes over %d disjoint sets of the 8 routed IQ2_S experts, %d MB of weights a call, "
                      "streamed from DRAM), one pinned thread a physical core, median call" % (
                          n_done.value, n_done.value // n_sets, n_sets, bytes_step // 1000000)}, out


def rel_l2(np, got, want):
    got, want = np.asarray(got, dtype=np.float64).reshape(-1), np.asarray(want, dtype=np.float64).reshape(-1)
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))


def decode_iq2s(args, np, torch, lib, L, info):
    import bench_workloads as bw
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

    if args.no_graph:
        with torch.cuda.stream(stream):
            for i in range(W):
                step(i)
            stream.synchronize()
            times = []
            for _ in range(bw.ROUNDS):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(K):
                    step(W + i)
                stream.synchronize()
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
            dt = sorted(times)[len(times) // 2]
    else:
        dt = bw.timed_graph(step, K, W, stream)

    # ---- the layer's two launches apart, HIP events on the launch stream: its first half (maya_moe_layer_decode_begin:
    # head + gate/up in one launch) and its second (maya_moe_layer_decode_end: the down launch, which rounds h itself), on
    # the same rotating logits - the kernels the layer runs, launched as the layer launches them
    with torch.cuda.stream(stream):
        reps = 64
        gu_s = bw.event_time(lambda i: layer.forward(table, logits[(5 + i) % n_sets:(5 + i) % n_sets + 1], x, half="begin"), reps, stream)
        dn_s = bw.event_time(lambda i: layer.forward(table, logits[(5 + i) % n_sets:(5 + i) % n_sets + 1], x, half="end"), reps, stream)

    sec = dt / K
    w_bytes = TOP_K * blob_bytes
    bytes_step = w_bytes + N_EXPERT * 4 + N_EMBD * 2 + N_EMBD * 4
    value = bytes_step / sec / 1e9
    # (the launch with the head in it reads the logits, the table and x and writes h, ids, weights and the plan)
    gu_bytes = TOP_K * 2 * N_FF * lib.row_bytes(IQ2_S, N_EMBD) + N_EXPERT * 12 + N_EMBD * 2 + TOP_K * N_FF * 4 + TOP_K * 16
    dn_bytes = TOP_K * N_EMBD * lib.row_bytes(IQ2_S, N_FF) + TOP_K * N_FF * 4 + N_EMBD * 4
    gu_rate, dn_rate = gu_bytes / gu_s / 1e9, dn_bytes / dn_s / 1e9

    # ---- parity of the timed configuration + CPU baseline on the same inputs (after the timed regions)
    cpu, err, ids_ok = None, None, None
    if not args.no_cpu:
        import oracle_py
        n_cpu_sets = 5
        with torch.cuda.stream(stream):
            out_g = layer.forward(table, logits[n_cpu_sets - 1:n_cpu_sets], x).clone()
            ids_g = layer.ids.clone()
            stream.synchronize()
        cpu, out_c = cpu_baseline(np, oracle_py, gguf_pool, blob_bytes, logits_np, x.to(torch.float32).cpu().numpy()[0], n_cpu_sets)
        wi, _ = oracle_py.router_topk(logits_np[n_cpu_sets - 1:n_cpu_sets], TOP_K)
        ids_ok = bool(np.array_equal(wi, ids_g.cpu().numpy()[:1]))
        if out_c is not None:
            err = rel_l2(np, out_g.cpu().numpy()[0], out_c)
    del pool, gguf_pool, table
    torch.cuda.empty_cache()

    line = {
        "metric": "moe_layer_decode_hbm_gbps_1tok",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(sec * 1e3, 6),
        "us_per_layer": round(sec * 1e6, 3),
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
                   "timed_as": ("eager launches, median of %d rounds" % bw.ROUNDS if args.no_graph else
                                "one HIP graph of the K steps, replayed back to back (>= 256 steps and >= 10 ms a sample) between "
                                "two HIP events on the launch stream, median of %d samples after the clocks settled" % bw.ROUNDS),
                   "device": info},
        "roofline": {"bound": "hbm", "kernel": "gate_up_iq2s_tiles_kernel (the head in the same launch)", "achieved": round(gu_rate, 2), "peak": 8000.0,
                     "unit": "GB/s", "frac": round(gu_rate * 1e9 / HBM_PEAK, 4), "traffic": GATE_UP_TRAFFIC_BYTES,
                     "algorithmic_bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_s * 1e6, 3),
                     "down_kernel": {"kernel": "down_iq2s_pos_kernel", "achieved": round(dn_rate, 2), "frac": round(dn_rate * 1e9 / HBM_PEAK, 4),
                                     "algorithmic_bytes_per_launch": dn_bytes, "avg_launch_us": round(dn_s * 1e6, 3)},
                     "layer": {"achieved": round(value, 2), "frac": round(value * 1e9 / HBM_PEAK, 4),
                               "algorithmic_bytes_per_step": bytes_step, "us_per_step": round(sec * 1e6, 3),
                               "us_outside_the_two_launches": round((sec - gu_s - dn_s) * 1e6, 3)}},
        "cpu_baseline": cpu,
        "parity_rel_l2_vs_cpu_path": err,
        "parity_ids_exact": ids_ok,
    }
    ok = args.no_cpu or (ids_ok and err is not None and err <= PARITY_BAR)
    return line, ok


def parity_of(np, torch, r):
    """The CPU path on a workload's own bytes (workloads hand back a `_parity` record): one expert, or the rows of the
    sampled tokens of one step - router ids of every token exact, each sampled row's relative L2 against the checker's layer
    on the routed experts' blobs pulled to the host.  Returns (worst relative L2, bar, ids exact or None)."""
    import oracle_py
    p = r.pop("_parity", None)
    if p is None:
        return None, PARITY_BAR, None
    if p["kind"] == "expert":
        blob = p["blob"].cpu().numpy()
        gr = oracle_py.row_bytes(p["type"], p["n_embd"])
        up_off, down_off = gr * p["n_ff"], 2 * gr * p["n_ff"]
        want = oracle_py.expert(p["type"], p["type"], blob, blob[up_off:], blob[down_off:], p["n_embd"], p["n_ff"],
                                p["x"].to(torch.float32).cpu().numpy())
        return rel_l2(np, p["out"].cpu().numpy(), want), PARITY_BAR, None
    tests = os.path.join(ROOT, "tests")   # the parity helpers of the tests: the checker's layer on the host
    if tests not in sys.path:
        sys.path.insert(0, tests)
    import gpu_util
    ids, w = oracle_py.router_topk(p["logits"], p["k"])
    ids_ok = bool(np.array_equal(ids, p["ids"]))
    toks = p["tokens"]

    class Blobs:   # an expert's blob comes to the host when the checker asks for it
        def __init__(self):
            self.have = {}

        def __getitem__(self, e):
            if e not in self.have:
                self.have[e] = p["blob_of"](e)
            return self.have[e]

    blobs = Blobs()
    worst = 0.0
    if p["kind"] == "layer":
        sh = None
        if p.get("shared"):
            st, sblob, sl = p["shared"]
            sh = (st, sblob(), sl)
        for t in toks:
            _, _, want = gpu_util.oracle_layer(oracle_py, p["gate_type"], p["down_type"], blobs, p["k"], p["n_embd"], p["n_ff"],
                                               p["logits"][t:t + 1], p["x"][t:t + 1])
            want = want[0]
            if sh is not None:
                st, sb, sl = sh
                want = want + oracle_py.expert(st, st, sb, sb[sl.up_off:], sb[sl.down_off:], p["n_embd"], p["n_ff"], p["x"][t:t + 1])[0]
            worst = max(worst, rel_l2(np, p["out"][t], want))
    else:
        from maya_amd import exl3
        experts = {}
        for t in toks:
            for e in ids[t]:
                if int(e) not in experts:
                    experts[int(e)] = gpu_util.HostExpert(exl3, oracle_py, p["layout"], blobs[int(e)])
        for t in toks:
            parts = [experts[int(e)].part(experts[int(e)].h(p["x"][t], 0.0)) for e in ids[t]]
            want = oracle_py.combine(np.stack(parts), np.ascontiguousarray(w[t], dtype=np.float32))
            worst = max(worst, rel_l2(np, p["out"][t], want))
    return worst, p.get("tol", PARITY_BAR), ids_ok


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-graph", action="store_true", help="launch the timed steps eagerly instead of as one HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the parity leg")
    ap.add_argument("--no-prefill", action="store_true", help="leave the prompt-chunk sub-object out of the default line")
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
    import bench_workloads as workloads

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
        if args.workload not in workloads.WORKLOADS:
            sys.exit("bench.py: unknown workload %r" % args.workload)
        r = workloads.WORKLOADS[args.workload](args.steps, args.warmup)
        r["config"]["device"] = info
        err, bar, ids_ok = (None, PARITY_BAR, None) if args.no_cpu else parity_of(np, torch, r)
        r.pop("_parity", None)
        line = {"metric": r["metric"], "value": r["value"], "unit": r["unit"], "n_gpus": 1, "steps": args.steps,
                "warmup": args.warmup, "ms_per_step": round(r["ms_per_step"], 6), "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic", "config": r["config"], "roofline": r["roofline"],
                "cpu_baseline": None, "parity_rel_l2_vs_cpu_path": err, "parity_bar": bar, "parity_ids_exact": ids_ok}
        print(json.dumps(line))
        if (err is not None and not err <= bar) or ids_ok is False:
            print("bench.py: parity failed: relative L2 %s against the CPU path (bar %g), ids exact %s" % (err, bar, ids_ok), file=sys.stderr)
            sys.exit(3)
        return

    line, ok = decode_iq2s(args, np, torch, lib, L, info)
    if not args.no_prefill:
        # BASELINE's second metric, the 512-token prompt chunk (configs[3]), in the same line; bench.py --workload prefill_q4k
        # gives the same numbers alone
        ksteps = max(4, min(16, args.steps))
        r = workloads.prefill_q4k(ksteps, 2)
        r.pop("_parity", None)
        line["prefill"] = {"metric": r["metric"], "value": r["value"], "unit": r["unit"], "ms_per_chunk": round(r["ms_per_step"], 4),
                           "steps": ksteps, "pct_of_int8_peak": round(100.0 * r["value"] * 1e12 / workloads.INT8_PEAK, 2),
                           "pct_of_hbm_peak": r["config"]["pct_of_hbm_peak"], "weight_gbps": r["config"]["weight_gbps"],
                           "workload": r["config"]["workload"], "experts_with_rows": r["config"]["experts_with_rows"],
                           "int8_ops_per_chunk": r["config"]["int8_ops_per_step"],
                           "algorithmic_bytes_per_chunk": r["config"]["algorithmic_bytes_per_step"], "roofline": r["roofline"]}
    print(json.dumps(line))
    if not ok:
        print("bench.py: parity failed: ids exact %s, relative L2 %s against the CPU path (bar %g)" % (
            line["parity_ids_exact"], line["parity_rel_l2_vs_cpu_path"], PARITY_BAR), file=sys.stderr)
        sys.exit(3)


if __name__ == "__main__":
    main()

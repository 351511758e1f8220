"""The BASELINE configurations other than the decode layer that bench.py times by default: synthetic inputs made on the
device, K steps captured as one HIP graph, and the algorithmic bytes / operations of a step.  Each function returns the
fields bench.py prints (metric, value, unit, ms_per_step, config, roofline)."""
import ctypes as C
import time

import numpy as np
import torch

from maya_amd import exl3, lib, prefill

HBM_PEAK = 8.0e12
INT8_PEAK = 5.0e15


def zipf_bias(n_expert, s=1.1):
    """The prefill configuration's routing skew: b_e = log(1 / (e + 1)^s), added to N(0, 1) router logits."""
    return (-s * np.log(np.arange(1, n_expert + 1, dtype=np.float64))).astype(np.float32)


def random_blocks(n_bytes, block, fields, seed):
    """Random bytes in `block`-byte blocks whose FP16 fields (byte offset -> (lo, hi)) are drawn uniformly."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    assert n_bytes % block == 0
    pool = torch.empty(n_bytes, dtype=torch.uint8, device="cuda")
    step = 1 << 28
    for o in range(0, n_bytes, step):
        n = min(step, n_bytes - o)
        pool[o:o + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    blocks = pool.view(-1, block)
    for off, (lo, hi) in fields.items():
        d = (torch.rand(blocks.shape[0], device="cuda", generator=g) * (hi - lo) + lo).to(torch.float16)
        blocks[:, off:off + 2] = d.view(torch.uint8).view(-1, 2)
    return pool


ROUNDS = 7


def _settle(replay, stream, tol=0.01, most=24):
    """Replays until two consecutive replays agree within tol (the clocks have risen and stay there)."""
    prev = None
    for _ in range(most):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        replay()
        stream.synchronize()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if prev is not None and abs(dt - prev) <= tol * max(dt, prev):
            return
        prev = dt


MIN_SAMPLE_SECONDS = 0.010


def timed_graph(step, K, W, stream, rounds=ROUNDS):
    """W eager warm-up steps, then the K steps captured as one HIP graph (the reference's timing method,
    tests/hip/expert_kernel_bench.cpp:136-172).  Untimed replays until two in a row agree within 1 %, then `rounds` timed
    samples.  The graph holds the K steps ceil(256 / K) times over; a sample is that graph replayed back to back - at least
    10 ms of GPU work - between two HIP events recorded on the launch stream, so what it holds is the kernels' time: the
    host's launch and synchronisation cost of a sample (tens of microseconds) is spread over its >= 256 steps.  Returns
    the median sample's seconds for K steps."""
    with torch.cuda.stream(stream):
        for i in range(W):
            step(i)
        stream.synchronize()
        inner = -(-256 // K)   # the K steps ceil(256 / K) times over in the one graph: no replay boundary inside 256 steps
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for _ in range(inner):
                for i in range(K):
                    step(W + i)
        g.replay()   # the graph's first launch uploads it
        stream.synchronize()
        _settle(g.replay, stream)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        g.replay()
        e1.record(stream)
        stream.synchronize()
        one = max(e0.elapsed_time(e1) * 1e-3, 1e-7)
        reps = max(1, int(np.ceil(MIN_SAMPLE_SECONDS / one)))
        times = []
        for _ in range(rounds):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                g.replay()
            e1.record(stream)
            stream.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3 / (reps * inner))
        return sorted(times)[len(times) // 2]


def event_time(fn, reps, stream, rounds=ROUNDS):
    """Median over `rounds` graph replays of the average seconds of fn(i) over reps launches in one graph, HIP events on
    the launch stream (the stream the kernels run on)."""
    with torch.cuda.stream(stream):
        fn(0)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(reps):
                fn(i)
        g.replay()
        stream.synchronize()
        _settle(g.replay, stream)
        times = []
        for _ in range(rounds):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            g.replay()
            e1.record(stream)
            stream.synchronize()
            times.append(e0.elapsed_time(e1) * 1e-3 / reps)
        return sorted(times)[len(times) // 2]


# HBM bytes a step (a launch of the named kernel for the prefill chunks) read from rocprofv3's FETCH_SIZE and WRITE_SIZE
# counters, scaled by a plain copy of known size (profiles/other_configs_hbm_traffic_pmc.txt); they belong to the
# synthetic inputs these workloads make (fixed seeds), so they are constants here
TRAFFIC_BYTES = {"single_q4k": 25286343, "batch8_mixed": 1097088000, "exl3_verify": 336937077,
                 "prefill_q4k": 2122985062, "prefill_iq2s": 1253165670, "prefill_mixed": 1253165670}


def hbm_roofline(kernel, bytes_launch, seconds, traffic=None):
    rate = bytes_launch / seconds / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": round(rate, 2), "peak": 8000.0, "unit": "GB/s",
            "frac": round(rate * 1e9 / HBM_PEAK, 4), "traffic": traffic, "algorithmic_bytes_per_launch": int(bytes_launch),
            "avg_launch_us": round(seconds * 1e6, 3)}


def encode_q4k_device(w):
    """F32 weights [n] (n a multiple of 256) -> Q4_K blocks (third_party/ggml/ggml-common.h:327-338) as uint8 [n / 256 * 144],
    on the device.  A plain min/max encoder (the reference never quantizes weights; any valid encoding serves): per 32-value
    sub-block scale (max - min) / 15 and minimum -min (a sub-block with only positive values keeps minimum 0), both rounded
    to 6 bits against the block's FP16 d / dmin, codes q = nearest((x + dmin m) / (d sc)) in 0..15."""
    x = w.reshape(-1, 8, 32).to(torch.float32)
    nb = x.shape[0]
    lo = torch.clamp(x.amin(dim=2), max=0.0)
    hi = torch.maximum(x.amax(dim=2), lo)
    scale = (hi - lo) / 15.0
    mn = -lo
    d = (scale.amax(dim=1) / 63.0).to(torch.float16)
    dmin = (mn.amax(dim=1) / 63.0).to(torch.float16)
    df, dmf = d.to(torch.float32), dmin.to(torch.float32)
    sc = torch.where(df[:, None] > 0, torch.round(scale / df[:, None].clamp_min(1e-30)), torch.zeros_like(scale)).clamp(0, 63).to(torch.int32)
    m = torch.where(dmf[:, None] > 0, torch.round(mn / dmf[:, None].clamp_min(1e-30)), torch.zeros_like(mn)).clamp(0, 63).to(torch.int32)
    step = df[:, None] * sc.to(torch.float32)
    q = torch.where(step[:, :, None] > 0, torch.round((x + (dmf[:, None] * m.to(torch.float32))[:, :, None]) / step[:, :, None].clamp_min(1e-30)),
                    torch.zeros_like(x)).clamp(0, 15).to(torch.uint8)
    blocks = torch.empty((nb, 144), dtype=torch.uint8, device=w.device)
    blocks[:, 0:2] = d.view(torch.uint8).view(nb, 2)
    blocks[:, 2:4] = dmin.view(torch.uint8).view(nb, 2)
    # 6-bit scales / minimums: j < 4: scales[j] = sc_j | (sc_{j+4} >> 4) << 6, scales[j + 4] = m_j | (m_{j+4} >> 4) << 6;
    # scales[j + 8] = (sc_{j+4} & 15) | (m_{j+4} & 15) << 4
    s8 = torch.empty((nb, 12), dtype=torch.int32, device=w.device)
    s8[:, 0:4] = sc[:, 0:4] | ((sc[:, 4:8] >> 4) << 6)
    s8[:, 4:8] = m[:, 0:4] | ((m[:, 4:8] >> 4) << 6)
    s8[:, 8:12] = (sc[:, 4:8] & 15) | ((m[:, 4:8] & 15) << 4)
    blocks[:, 4:16] = s8.to(torch.uint8)
    # sub-blocks 2p and 2p + 1 share qs[32p .. 32p + 31]: low nibbles = 2p, high nibbles = 2p + 1
    qq = q.view(nb, 4, 2, 32)
    blocks[:, 16:144] = (qq[:, :, 0, :] | (qq[:, :, 1, :] << 4)).reshape(nb, 128)
    return blocks.reshape(-1)


def single_q4k(K, W):
    """configs[0]: one Q4_K expert GLU, one token, F32 activation; gate / up [2048 x 7168] and down [7168 x 2048] drawn from
    N(0, 0.02) and quantized to Q4_K; 16 such experts rotate (396 MB > the on-die caches)."""
    E, FF, copies = 7168, 2048, 16
    layer = lib.MoeLayer(lib.Q4_K, lib.Q4_K, E, FF, copies, 1, max_tokens=1, packing=lib.PACK_STREAM)   # (Q4_K: GGUF order, aligned)
    bb = layer.blob_bytes
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    pool = torch.empty(copies * bb, dtype=torch.uint8, device="cuda")
    for e in range(copies):
        pool[e * bb:(e + 1) * bb] = encode_q4k_device(torch.randn(3 * E * FF, device="cuda", generator=g) * 0.02)
    table = torch.tensor([pool.data_ptr() + e * bb for e in range(copies)], dtype=torch.int64, device="cuda")
    logits = torch.full((copies, copies), -30.0, device="cuda")
    logits.fill_diagonal_(0.0)
    x = torch.randn(1, E, device="cuda", generator=g)
    stream = torch.cuda.Stream()
    dt = timed_graph(lambda i: layer.forward(table, logits[i % copies:i % copies + 1], x), K, W, stream)
    with torch.cuda.stream(stream):
        out0 = layer.forward(table, logits[0:1], x).clone()
        stream.synchronize()
    nbytes = bb + E * 4 + E * 4
    sec = dt / K
    return {"metric": "expert_glu_hbm_gbps_1tok", "value": round(nbytes / sec / 1e9, 2), "unit": "GB/s", "ms_per_step": sec * 1e3,
            "dtype": "int8",
            "config": {"workload": "configs[0]: one expert GLU, gate/up [2048x7168] + down [7168x2048] quantized to Q4_K from "
                                   "N(0,0.02), 1 token F32 N(0,1); 16 such experts rotate over the steps",
                       "algorithmic_bytes_per_step": nbytes},
            "roofline": hbm_roofline("layer (gate_up_q4k_pos_kernel with the head in the same launch + down_q4k_pos_kernel)", nbytes, sec, TRAFFIC_BYTES["single_q4k"]),
            # for bench.py's parity leg (the CPU path's expert on the same bytes, after the timed region)
            "_parity": {"kind": "expert", "type": lib.Q4_K, "n_embd": E, "n_ff": FF, "blob": pool[:bb], "x": x, "out": out0}}


def batch8_mixed(K, W):
    """configs[2]: 8 tokens, 256 experts top-8, gate/up IQ2_S + down Q4_K, and a Q8_0 shared expert every token takes."""
    E, FF, NE, TK, T = 7168, 2048, 256, 8, 8
    layer = lib.MoeLayer(lib.IQ2_S, lib.Q4_K, E, FF, NE, TK, max_tokens=T, packing=lib.PACK_STREAM)
    bb = layer.blob_bytes
    l = layer.gguf_layout
    pool = torch.empty(NE * bb, dtype=torch.uint8, device="cuda")
    view = pool.view(NE, bb)
    gu = random_blocks(NE * l.down_off, 82, {0: (2e-3, 6e-3)}, 6).view(NE, l.down_off)
    dn = random_blocks(NE * (bb - l.down_off), 144, {0: (2e-4, 6e-4), 2: (2e-4, 6e-4)}, 7).view(NE, bb - l.down_off)
    view[:, :l.down_off] = gu
    view[:, l.down_off:] = dn
    del gu, dn
    staging = torch.empty(bb, dtype=torch.uint8, device="cuda")
    for e in range(NE):   # the engine's upload: every blob regrouped into the stream packing
        staging.copy_(view[e])
        lib.repack(l, staging, view[e])
    torch.cuda.synchronize()
    table = torch.tensor([pool.data_ptr() + e * bb for e in range(NE)], dtype=torch.int64, device="cuda")
    shared = lib.MoeLayer(lib.Q8_0, lib.Q8_0, E, FF, 1, 1, max_tokens=T, packing=lib.PACK_STREAM)
    n_sh = 4   # copies of the shared expert rotate too (4 x 46.8 MB)
    sh_pool = random_blocks(n_sh * shared.blob_bytes, 34, {0: (1e-4, 4e-4)}, 8)
    staging = torch.empty(shared.blob_bytes, dtype=torch.uint8, device="cuda")
    for c in range(n_sh):
        staging.copy_(sh_pool[c * shared.blob_bytes:(c + 1) * shared.blob_bytes])
        lib.repack(shared.gguf_layout, staging, sh_pool[c * shared.blob_bytes:(c + 1) * shared.blob_bytes])
    torch.cuda.synchronize()
    # (the shared expert's plan is static - every token, weight 1 - so it runs through the stage calls without routing)
    dense = [lib.DenseExpert(lib.Q8_0, lib.Q8_0, E, FF, T, sh_pool.data_ptr() + c * shared.blob_bytes, packing=lib.PACK_STREAM)
             for c in range(n_sh)]
    rng = np.random.default_rng(9)
    n_sets = 8
    logits = torch.from_numpy(rng.standard_normal((n_sets, T, NE)).astype(np.float32)).cuda()
    x = torch.randn(T, E, device="cuda")
    distinct = []
    for s in range(n_sets):
        ids, _ = lib.route_topk(logits[s], TK)
        distinct.append(int(torch.unique(ids).numel()))
    stream = torch.cuda.Stream()

    def step(i):   # (the shared expert's launches run beside the routed experts' on the library's second stream)
        layer.forward(table, logits[i % n_sets], x, shared=dense[i % n_sh])

    dt = timed_graph(step, K, W, stream)
    d_avg = float(np.mean([distinct[(W + i) % n_sets] for i in range(K)]))
    nbytes = d_avg * bb + shared.blob_bytes + T * (E * 4 + E * 4)
    sec = dt / K
    with torch.cuda.stream(stream):   # one step's rows for the parity leg (after the timed region)
        out0 = layer.forward(table, logits[0], x, shared=dense[0]).clone()
        ids0 = layer.ids[:T].clone()
        stream.synchronize()

    def gguf_blob(e):   # expert e as the file holds it (the pool holds the stream packing)
        back = torch.empty(bb, dtype=torch.uint8, device="cuda")
        lib.unpack(l, view[e].contiguous(), back)
        torch.cuda.synchronize()
        return back.cpu().numpy()

    def shared_blob():
        back = torch.empty(shared.blob_bytes, dtype=torch.uint8, device="cuda")
        lib.unpack(shared.gguf_layout, sh_pool[:shared.blob_bytes].contiguous(), back)
        torch.cuda.synchronize()
        return back.cpu().numpy()

    parity = {"kind": "layer", "gate_type": lib.IQ2_S, "down_type": lib.Q4_K, "n_embd": E, "n_ff": FF, "k": TK, "blob_of": gguf_blob,
              "logits": logits[0].cpu().numpy(), "x": x.cpu().numpy(), "out": out0.cpu().numpy(), "ids": ids0.cpu().numpy(),
              "tokens": [0, 5], "shared": (lib.Q8_0, shared_blob, shared.gguf_layout)}
    return {"_parity": parity, "metric": "moe_layer_decode_hbm_gbps_8tok", "value": round(nbytes / sec / 1e9, 2), "unit": "GB/s", "ms_per_step": sec * 1e3,
            "dtype": "int8",
            "config": {"workload": "configs[2]: 8 tokens, 256 experts top-8 (gate/up IQ2_S, down Q4_K) + a Q8_0 shared expert; "
                                   "8 logit sets rotate", "distinct_experts_per_step": d_avg,
                       "algorithmic_bytes_per_step": int(nbytes)},
            "roofline": hbm_roofline("layer (routed gate_up_iq2s_pos_kernel + down_q4k_pos_kernel over 64 entries, shared expert gate_up_q80_pos_kernel + down_q80_pos_kernel)", nbytes, sec, TRAFFIC_BYTES["batch8_mixed"])}


BLOCK_FIELDS = {lib.Q4_K: (144, {0: (2e-4, 6e-4), 2: (2e-4, 6e-4)}), 22: (82, {0: (2e-3, 6e-3)})}


def prefill_q4k(K, W):
    """configs[3]: 512 tokens, 256 Q4_K experts top-8, Zipf(1.1)-skewed routing, int8 (Q8_K) activations, bf16 out."""
    return _prefill(K, W, lib.Q4_K, lib.Q4_K, "configs[3]", "Q4_K")


def prefill_iq2s(K, W):
    """configs[3]'s chunk on the north-star layer's IQ2_S experts (stream packing)."""
    return _prefill(K, W, 22, 22, "configs[3]'s chunk on IQ2_S experts", "IQ2_S")


def prefill_mixed(K, W):
    """configs[3]'s chunk on configs[2]'s experts: IQ2_S gate / up, Q4_K down (stream packing)."""
    return _prefill(K, W, 22, lib.Q4_K, "configs[3]'s chunk on IQ2_S gate/up + Q4_K down experts", "IQ2_S / Q4_K")


def _prefill(K, W, gt, dt, what, types):
    E, FF, NE, TK, T = 7168, 2048, 256, 8, 512
    down_type = dt
    gguf, bb = lib.layout(gt, dt, E, FF)
    stream_packed = gt != lib.Q4_K or dt != lib.Q4_K
    layout = lib.copy_layout(gguf, lib.PACK_STREAM) if stream_packed else gguf
    if stream_packed:
        # the three stacked tensors as a file holds them, then the blobs built on the device in the stream packing
        mats = []
        for i, (t, nbytes) in enumerate(((gt, gguf.up_off), (gt, gguf.down_off - gguf.up_off), (dt, bb - gguf.down_off))):
            block, fields = BLOCK_FIELDS[t]
            mats.append(random_blocks(NE * nbytes, block, fields, 11 + i))
        pool = torch.empty(NE * bb, dtype=torch.uint8, device="cuda")
        lib.pack_experts(gguf, mats[0], mats[1], mats[2], NE, lib.PACK_STREAM, pool, bb)
        torch.cuda.synchronize()
        del mats
    else:
        pool = random_blocks(NE * bb, 144, BLOCK_FIELDS[lib.Q4_K][1], 11)
    table = torch.tensor([pool.data_ptr() + e * bb for e in range(NE)], dtype=torch.int64, device="cuda")
    rng = np.random.default_rng(12)
    logits = torch.from_numpy((rng.standard_normal((T, NE)) + zipf_bias(NE)).astype(np.float32)).cuda()
    x = torch.randn(T, E, device="cuda")
    layer = prefill.PrefillLayer(layout, NE, TK, T, out_dtype=torch.bfloat16)
    stream = torch.cuda.Stream()
    dt = timed_graph(lambda i: layer.forward(table, logits, x), K, W, stream)
    sec = dt / K
    ids, w = lib.route_topk(logits, TK)
    used = int(torch.unique(ids).numel())
    ops = 2 * 3 * E * FF * T * TK
    nbytes = used * bb + T * E * 4 + T * E * 2
    # the dominant kernel alone: the gate/up GEMM (2/3 of the operations)
    with torch.cuda.stream(stream):
        p = prefill.plan(ids.reshape(-1), table)
        xq = prefill.quant(x, p, TK)
        hq = prefill.ActRows(p.n_entries, FF)
        hf = torch.empty((p.n_entries, FF), dtype=torch.float32, device="cuda")
        L = prefill.load()
        # (the call also rounds h: its small kernel rides in the measured time)
        sec_gu = event_time(lambda i: lib.check(L.maya_moe_prefill_gate_up(C.byref(layout), lib._p(table), NE, C.byref(p.c), p.n_entries,
                                                                         xq.c, 0.0, lib._p(hf), hq.c, lib._stream())), 8, stream)
    ops_gu = 2 * 2 * E * FF * T * TK
    tops_gu = ops_gu / sec_gu / 1e12
    parity = None
    if not stream_packed:   # (Q4_K blobs are in the file's order: the CPU path reads them as they are)
        with torch.cuda.stream(stream):
            out0 = layer.forward(table, logits, x).to(torch.float32).clone()
            ids0 = layer.ids[:T].clone()
            stream.synchronize()
        view = pool.view(NE, bb)
        parity = {"kind": "layer", "gate_type": gt, "down_type": down_type, "n_embd": E, "n_ff": FF, "k": TK,
                  "blob_of": lambda e: view[e].cpu().numpy(), "logits": logits.cpu().numpy(), "x": x.cpu().numpy(),
                  "out": out0.cpu().numpy(), "ids": ids0.cpu().numpy(), "tokens": [0, 255, 511], "tol": 5e-3,
                  "note": "bf16 output: the bar of the rounded rows is 5e-3 (2^-8 a value); the F32 rows are held to 1e-3 in tests/"}
    return {"_parity": parity, "metric": "prefill_int8_tops_512tok", "value": round(ops / sec / 1e12, 2), "unit": "TOP/s", "ms_per_step": sec * 1e3,
            "dtype": "int8",
            "config": {"workload": what + ": prefill chunk of 512 tokens, 256 experts " + types + " top-8, logits N(0,1) - 1.1 ln(e+1), "
                                   "int8 activations in the CPU path's Q8_K rounding, bf16 out", "experts_with_rows": used, "int8_ops_per_step": ops,
                       "algorithmic_bytes_per_step": int(nbytes), "weight_gbps": round(nbytes / sec / 1e9, 1),
                       "pct_of_hbm_peak": round(100 * nbytes / sec / HBM_PEAK, 2)},
            "roofline": {"bound": "mfma", "kernel": ("prefill_q4k_kernel" if gt == lib.Q4_K else "prefill_iq2s_kernel") + "<gate_up>",
                         "achieved": round(tops_gu, 2), "peak": 5000.0,
                         "unit": "TOP/s", "frac": round(tops_gu * 1e12 / INT8_PEAK, 4),
                         "traffic": TRAFFIC_BYTES["prefill_q4k" if gt == lib.Q4_K else "prefill_iq2s"],
                         "algorithmic_ops_per_launch": ops_gu, "avg_launch_us": round(sec_gu * 1e6, 1)}}


def exl3_pool(E, FF, NE, k2):
    """NE EXL3 experts (mul1 codebook, k2 / 2 bits a weight) on the device: random trellis words (every pattern is a valid
    encoding, tests/exl3_test.cu:112-116), sign vectors suh and scaled sign vectors svh.  Returns the layout, a blob's bytes,
    the pool, its [NE, stride] view and the address table."""
    l, bb = exl3.make_layout(E, FF, k2, exl3.CB_MUL1)
    stride = (bb + 255) & ~255
    pool = random_blocks(NE * stride, 256, {}, 13)
    view = pool.view(NE, stride)
    g = torch.Generator(device="cuda")
    g.manual_seed(14)
    for r in range(3):
        k, n = exl3.matrix_of(l, r)
        suh = (torch.randint(0, 2, (NE, k), device="cuda", generator=g) * 2 - 1).to(torch.float16)
        svh = ((torch.randint(0, 2, (NE, n), device="cuda", generator=g) * 2 - 1) *
               (torch.rand((NE, n), device="cuda", generator=g) + 0.5) / (k ** 0.5)).to(torch.float16)
        view[:, l.suh[r]:l.suh[r] + 2 * k] = suh.view(torch.uint8).view(NE, -1)
        view[:, l.svh[r]:l.svh[r] + 2 * n] = svh.view(torch.uint8).view(NE, -1)
    table = torch.tensor([pool.data_ptr() + e * stride for e in range(NE)], dtype=torch.int64, device="cuda")
    return l, bb, pool, view, table


def exl3_verify(K, W, k2=6):
    """configs[4]: 160 EXL3 experts (3 bits a weight: k2 = 6, mul1 codebook), top-8, hidden 6144, intermediate 1536, a
    4-token verify window; 8 logit sets rotate.  (k2 = 8, 10: the same layer at 4 and 5 bits a weight.)"""
    E, FF, NE, TK, T = 6144, 1536, 160, 8, 4
    l, bb, pool, view, table = exl3_pool(E, FF, NE, k2)
    layer = exl3.Exl3Layer(l, NE, TK, max_tokens=T)
    rng = np.random.default_rng(15)
    n_sets = 8
    logits = torch.from_numpy(rng.standard_normal((n_sets, T, NE)).astype(np.float32)).cuda()
    x = torch.randn(T, E, device="cuda").to(torch.float16).to(torch.float32)   # FP16 activations, handed over as F32
    distinct = []
    for s in range(n_sets):
        ids, _ = lib.route_topk(logits[s], TK)
        distinct.append(int(torch.unique(ids).numel()))
    stream = torch.cuda.Stream()
    dt = timed_graph(lambda i: layer.forward(table, logits[i % n_sets], x), K, W, stream)
    d_avg = float(np.mean([distinct[(W + i) % n_sets] for i in range(K)]))
    nbytes = d_avg * bb + T * (E * 4 + E * 4)
    sec = dt / K
    with torch.cuda.stream(stream):
        out0 = layer.forward(table, logits[0], x).clone()
        ids0 = layer.ids[:T].clone()
        stream.synchronize()
    parity = {"kind": "exl3_layer", "layout": l, "blob_of": lambda e: view[e, :bb].cpu().numpy(), "k": TK,
              "logits": logits[0].cpu().numpy(), "x": x.cpu().numpy(), "out": out0.cpu().numpy(), "ids": ids0.cpu().numpy(),
              "tokens": [0, 3]}
    return {"_parity": parity, "metric": "exl3_moe_layer_hbm_gbps_4tok", "value": round(nbytes / sec / 1e9, 2), "unit": "GB/s", "ms_per_step": sec * 1e3,
            "dtype": "f16",
            "config": {"workload": ("configs[4]" if k2 == 6 else "configs[4] at another bit rate") +
                                   ": EXL3 %g-bit trellis experts (k2 %d, mul1), 160 experts top-8, hidden 6144, " % (k2 / 2, k2) +
                                   "intermediate 1536, 4-token verify window; 8 logit sets rotate",
                       "distinct_experts_per_step": d_avg, "algorithmic_bytes_per_step": int(nbytes)},
            "roofline": hbm_roofline("layer (exl3_gu_split_kernel + exl3_swiglu_kernel + exl3_down_kernel + exl3_combine_kernel)", nbytes, sec,
                                     TRAFFIC_BYTES["exl3_verify"] if k2 == 6 else None)}


WORKLOADS = {"single_q4k": single_q4k, "batch8_mixed": batch8_mixed, "prefill_q4k": prefill_q4k, "exl3_verify": exl3_verify,
             "prefill_iq2s": prefill_iq2s, "prefill_mixed": prefill_mixed,
             "exl3_verify_4bit": lambda K, W: exl3_verify(K, W, 8), "exl3_verify_5bit": lambda K, W: exl3_verify(K, W, 10)}

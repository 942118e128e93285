#!/usr/bin/env python3
"""Headline benchmark: OIL4 decode GEMV at the Llama-7B up/gate projection shape
(K = 4096 -> N = 11008, M = 1, FP32 activations), one MI355X.

A "step" is one pass of the GEMV over a ring of 40 resident copies of the OIL4
weight matrix (40 launches, 902 MB streamed): one matrix (22.5 MB) fits the
256 MB Infinity Cache, so every launch of a step reads a copy that the cache
no longer holds.  A step is one replay of a HIP graph, so nothing but graph
replays sits inside the timed region; K steps make a round and rounds repeat
until the region is at least 50 ms long.  `ms_per_step` is per step (40
launches); `value` and `roofline` are per launch: payload bytes / time.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
ROWS, COLS = 11008, 4096       # W is [N rows][K cols]: y = W x
RING = 40                      # distinct weight copies: 40 x 22.5 MB = 902 MB > 256 MB cache
# HBM bytes per GEMV launch, cited from the rocprofv3 counter runs summarised in profiles/oil4_gemv_4096x11008_m1.md
# (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB per dispatch, factors from a plain 1 GiB copy); not measured in this run
HBM_TRAFFIC_BYTES_PER_LAUNCH = 22881280


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_weights(rows, cols, seed):
    import numpy as np
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(rows * cols) * 0.02).astype(np.float32)


class Ring:
    """`copies` device-resident uploads of the same quantized matrix."""

    def __init__(self, ia, payload, blocks, rows, cols, copies):
        self.items = [ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) for _ in range(copies)]
        self.payload_bytes = int(payload.size)

    def close(self):
        for d in self.items:
            d.close()


def time_ring(torch, ring, x, y, steps, warmup, settle_s=0.0, min_region_s=0.05):
    """One step = one replay of a HIP graph that holds one GEMV launch per ring copy (`len(ring.items)` launches).
    Nothing but graph replays sits between the two events: `steps` replays make one round, and rounds are repeated
    until the timed region is at least `min_region_s` long.  Returns (seconds per launch, host seconds per launch,
    rounds, seconds of the timed region).  settle_s: untimed replays for that long in front of the timed region, so
    that a device that comes out of idle has reached its steady clocks."""
    n = len(ring.items)
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):                    # untimed warm-up passes, on the stream that is captured below:
        for i in range(max(warmup, 1)):                # first-call set-up, and scratch that belongs to the stream
            for d in ring.items:
                d.gemv(x, out=y)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for d in ring.items:
                d.gemv(x, out=y)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        graph.replay()
        torch.cuda.synchronize()
        t_end = time.perf_counter() + settle_s
        while time.perf_counter() < t_end:
            for _ in range(8):
                graph.replay()
            torch.cuda.synchronize()
        # a short untimed probe sizes the number of rounds
        p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        p0.record(stream)
        for _ in range(4):
            graph.replay()
        p1.record(stream)
        torch.cuda.synchronize()
        est = max(p0.elapsed_time(p1) * 1e-3 / 4, 1e-7)                 # seconds per replay
        rounds = max(1, int(-(-min_region_s // (est * steps))))
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(rounds * steps):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    dev = e0.elapsed_time(e1) * 1e-3
    launches = rounds * steps * n
    return dev / launches, wall / launches, rounds, dev


def cpu_baseline(payload, blocks, rows, cols, x):
    """The oracle's restatement of Qwen35Engine::gemm (per-block bit-stream decode + FP32 dot,
    min(8, cores) threads, qwen35_engine.cpp:47-85) on a row sample sized for ~10-20 s."""
    import numpy as np
    import oracle as O
    ob = np.zeros(blocks.size, dtype=O.BLOCK_DTYPE)
    for k in ("cb_off", "idx_off", "cb_bytes", "idx_bytes", "nw", "fmt"):
        ob[k] = blocks[k]
    bpr = cols // 256
    threads = min(8, os.cpu_count() or 1)
    O.block_gemm(payload, ob, rows, cols, x, wide=False, threads=threads)          # warm-up pass
    passes, t0 = 0, time.perf_counter()
    while True:                                                                     # whole-matrix passes for ~12 s
        O.block_gemm(payload, ob, rows, cols, x, wide=False, threads=threads)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= 12.0 or passes >= 2000:
            break
    nbytes = passes * rows * bpr * 128
    return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{passes} passes over the full {rows} x {cols} matrix, M=1, {dt:.1f} s on {threads} threads; "
                      f"oracle restatement of Qwen35Engine::gemm (per-block bit-stream decode + FP32 dot)"}


def time_calls(torch, fn, min_ms=50.0, warm=3):
    """Seconds per call of fn(): whole batches of calls between two events, the batch doubled until it spans at least
    min_ms of device time (the 3-5 warm-ups and mean-over-iterations convention of bench/bench_oil_quant.cpp:22-31)."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    n = 8
    while True:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        if ms >= min_ms or n >= 1 << 16:
            return ms * 1e-3 / n
        n *= 2


def cpu_flat_oil8(with_reference=True):
    """The flat-codebook CPU leg: kernel::oil8_gemm gather semantics (src/kernel_oil8.cpp:35-68: eight-lane
    accumulators, horizontal add) at config 1's M=1, K=N=4096 on ONE thread, as the reference runs it: 3 warm-ups,
    mean of 100 timed iterations (bench/bench_oil_quant.cpp:22-31).  The oracle's restatement, and beside it the
    compiled reference's own oil8_gemm where oracle/_ref is built."""
    import numpy as np
    import oracle as O
    rng = np.random.default_rng(8)
    N = K = 4096
    idx = rng.integers(0, 256, N * K, dtype=np.uint8)
    cb = np.linspace(-8.0, 8.0, 256, dtype=np.float32)
    act = rng.standard_normal(K).astype(np.float32)
    out = {}

    def timed(fn):
        for _ in range(3):
            fn()
        t0 = time.perf_counter()
        for _ in range(100):
            fn()
        return (time.perf_counter() - t0) / 100

    res = np.zeros(N, dtype=np.float32)
    L = O.lib()
    pi, pc, pa, po = (O._p(idx, O._u8p), O._p(cb, O._f32p), O._p(act, O._f32p), O._p(res, O._f32p))
    t = timed(lambda: L.orc_oil8_gemm(pi, pc, pa, po, 1, N, K, 1))
    out["cpu_flat_oil8_GBps"] = round(N * K / t / 1e9, 3)
    out["cpu_flat_oil8_ms"] = round(t * 1e3, 3)
    out["cpu_flat_oil8_threads"] = 1
    out["cpu_flat_oil8_kind"] = "port (oracle restatement of kernel::oil8_gemm, AVX2 summation order), 100 iterations after 3 warm-ups"
    R = O.ref() if with_reference else None
    if R is not None:
        t = timed(lambda: R.ref_oil8_gemm(pi, pc, pa, po, 1, N, K))
        out["cpu_flat_oil8_reference_GBps"] = round(N * K / t / 1e9, 3)
        out["cpu_flat_oil8_reference_kind"] = "reference (oracle/_ref: the reference's own kernel::oil8_gemm compiled with -mavx2 -mfma), one thread"
    return out


def time_gemvs(torch, items, xs, ys, reps):
    """Seconds per pass over `items` (a list of (DeviceWeights, x index)), graph replay."""
    for d, k in items:
        d.gemv(xs[k], out=ys[k])
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for d, k in items:
                d.gemv(xs[k], out=ys[k])
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / reps


def bench_fused_layer(torch, ia, unfused_s):
    """The same Llama-7B-shaped layer with q/k/v and gate/up stacked into one tensor each, both RMSNorms and the
    SwiGLU product formed inside the GEMVs that consume them: 4 launches per layer instead of 7 GEMVs + glue."""
    import numpy as np
    from innova_amd import layers
    L = _lib_handles(ia)
    copies = 12                                                            # 12 x 101 MB of OIL4 payload per layer > 256 MB cache
    sets = []
    for c in range(copies):
        d = {}
        for name, (r, k) in (("qkv", (12288, 4096)), ("o", (4096, 4096)), ("gate_up", (22016, 4096)), ("down", (4096, 11008))):
            if c == 0:
                w = make_weights(r, k, seed=300 + len(name))
                d[name] = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
            else:
                d[name] = sets[0][name + "_host"]
        sets.append({**{n: ia.DeviceWeights.from_blocks(*d[n], *shape) for n, shape in
                        (("qkv", (12288, 4096)), ("o", (4096, 4096)), ("gate_up", (22016, 4096)), ("down", (4096, 11008)))},
                     **{n + "_host": d[n] for n in d}})
    x = torch.randn(1, 4096, device="cuda")
    wn = torch.randn(4096, device="cuda") * 0.1
    xn = torch.empty_like(x)
    qkv = torch.empty((1, 12288), device="cuda")
    att = torch.randn(1, 4096, device="cuda")
    o = torch.empty((1, 4096), device="cuda")
    y = torch.empty((1, 4096), device="cuda")
    scratch = torch.empty(3 * 11008 + 4096, device="cuda")
    st = lambda: ia._lib.current_stream()  # noqa: E731

    def layer(sx):
        ia._lib.check(L.oilhip_gemv_rmsnorm_f32(sx["qkv"].handle, x.data_ptr(), wn.data_ptr(), qkv.data_ptr(), 1, None, st()))
        sx["o"].gemv(att, out=o)                                         # attention itself is not modelled
        ia._lib.check(L.oilhip_mlp_step_f32(sx["gate_up"].handle, sx["down"].handle, o.data_ptr(), wn.data_ptr(),
                                            y.data_ptr(), 1, scratch.data_ptr(), st()))

    for sx in sets:
        layer(sx)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for sx in sets:
                layer(sx)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(20):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / (20 * copies)
    for sx in sets:
        for n in ("qkv", "o", "gate_up", "down"):
            sx[n].close()
    payload = (12288 + 4096 + 22016) * 4096 // 2 + 4096 * 11008 // 2
    return {"fused_layer_us": round(t * 1e6, 1), "fused_layer_GBps": round(payload / t / 1e9, 1),
            "decode_tok_per_s_7B_fused_layers": round(1.0 / (32 * t), 1),
            "decode_tok_per_s_7B_unfused_gemvs": round(1.0 / unfused_s, 1)}


def bench_tall(torch, ia):
    """The same kernel on taller tensors of the same width (the stacked gate+up rows of a layer, an output head):
    the per-launch set-up is amortised over more rows.  The payload is random index bytes with a fixed FP16 block
    scale (bandwidth does not depend on the values)."""
    import numpy as np
    out = {}
    rng = np.random.default_rng(5)
    for label, rows, copies in (("stacked_gate_up_22016x4096", 22016, 14), ("head_131072x4096", 131072, 3)):
        nb = rows * COLS // 256
        payload = rng.integers(0, 256, nb * 128, dtype=np.uint8)
        payload[0::128], payload[1::128] = 0x1F, 0x25                      # FP16 0x251F = 0.0200
        blocks = np.zeros(nb, dtype=ia._lib.BLOCK_DTYPE)
        blocks["idx_off"] = np.arange(nb, dtype=np.uint64) * 128
        blocks["cb_off"] = blocks["idx_off"]
        blocks["idx_bytes"], blocks["nw"], blocks["fmt"] = 128, 256, int(ia.Format.OIL4)
        ring = Ring(ia, payload, blocks, rows, COLS, copies)
        x = torch.randn(1, COLS, device="cuda")
        y = torch.empty((1, rows), dtype=torch.float32, device="cuda")
        s_t = time_ring(torch, ring, x, y, 4, 1)[0]
        out[f"{label}_M1_us"] = round(s_t * 1e6, 2)
        out[f"{label}_M1_GBps"] = round(ring.payload_bytes / s_t / 1e9, 1)
        ring.close()
    return out


def _lib_handles(ia):
    return ia._lib.lib()


def bench_oil8(torch, ia):
    """OIL8 M=1, K=N=4096: block-codec GEMV and the flat kernel::oil8_gemm form (16.8 MB of codes each)."""
    import numpy as np
    w = make_weights(4096, 4096, seed=11)
    p8, b8 = ia.block_codec.quantize_tensor(w, ia.Format.OIL8)
    ring = Ring(ia, p8, b8, 4096, 4096, 56)
    x = torch.randn(1, 4096, device="cuda")
    y = torch.empty((1, 4096), dtype=torch.float32, device="cuda")
    t = time_ring(torch, ring, x, y, 4, 1)[0]
    ring.close()
    out = {"oil8_block_4096x4096_M1_GBps": round(p8.size / t / 1e9, 1), "oil8_block_4096x4096_M1_us": round(t * 1e6, 2)}
    idx = [torch.randint(0, 256, (4096 * 4096,), dtype=torch.uint8, device="cuda") for _ in range(56)]
    cb = torch.linspace(-8, 8, 256, device="cuda")
    act = torch.randn(4096, device="cuda")
    yo = torch.empty((1, 4096), dtype=torch.float32, device="cuda")
    L = ia._lib.lib()

    def flat(i):
        ia._lib.check(L.oilhip_flat_oil8_gemm(i.data_ptr(), cb.data_ptr(), act.data_ptr(), yo.data_ptr(), 1, 4096, 4096,
                                              ia._lib.current_stream()))

    for i in idx:
        flat(i)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for i in idx:
                flat(i)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(20):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
    tf = e0.elapsed_time(e1) * 1e-3 / (20 * 56)
    out["oil8_flat_4096x4096_M1_us"] = round(tf * 1e6, 2)
    out["oil8_flat_4096x4096_M1_GBps"] = round(4096 * 4096 / tf / 1e9, 1)
    return out


STACK = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
         ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)]


def bench_mixed_stack(torch, ia):
    """The 1.50-bpw stack: 7 matrices of a Llama-7B layer, 1 % of blocks scaled x8, importance = mean |w|
    per block, formats from the planner at target 1.50 (half SPARK_Q0, half OIL1), and a stress plan that is
    NOT reference-derived (importance quartiles -> OIL4 / OIL2 / SPARK_Q0 / OIL1); and the registry's grouped mix
    SPARK_MIX_Q0 (1.925 bpw: OIL8_GRP / OIL4_GRP / OIL2_GRP / OIL1_GRP per block by FormatRegistry::allocate_mix_blocks)."""
    import numpy as np
    from innova_amd.format_planner import FormatPlanner, allocate_mix_blocks
    rng = np.random.default_rng(33)
    plans = {"planner_1p50": [], "stress_quartiles": [], "spark_mix_q0": []}
    for name, rows, cols in STACK:
        w = make_weights(rows, cols, seed=100 + len(name) + rows % 97)
        nb = rows * cols // 256
        hot = rng.choice(nb, nb // 100, replace=False)
        w.reshape(nb, 256)[hot] *= np.float32(8.0)
        pl = FormatPlanner(1.50)
        pl.score_importance(w)
        plan = pl.allocate(nb)
        sc = pl.importance_scores()
        q = np.argsort(np.argsort(-sc, kind="stable"), kind="stable") * 4 // nb          # quartile by descending importance
        stress = np.array([int(ia.Format.OIL4), int(ia.Format.OIL2), int(ia.Format.SPARK_Q0), int(ia.Format.OIL1)], np.uint8)[q]
        mix = allocate_mix_blocks("SPARK_MIX_Q0", w, 256, (rows, cols))[0]
        for key, fm in (("planner_1p50", plan.formats), ("stress_quartiles", stress), ("spark_mix_q0", mix)):
            payload, blocks = ia.block_codec.quantize_tensor(w, fm)
            plans[key].append((rows, cols, payload, blocks))
        del w
    out = {}
    xs = {4096: torch.randn(1, 4096, device="cuda"), 11008: torch.randn(1, 11008, device="cuda")}
    ys = {4096: torch.empty((1, 4096), device="cuda"), 11008: torch.empty((1, 11008), device="cuda")}
    for key, mats in plans.items():
        payload_bytes = sum(int(b["cb_bytes"].astype(np.int64).sum() + b["idx_bytes"].astype(np.int64).sum()) for _, _, _, b in mats)
        copies = max(2, int(600e6 // (payload_bytes + 16 * sum(len(b) for _, _, _, b in mats))) + 1)
        items, keep = [], []
        for _ in range(copies):
            for rows, cols, payload, blocks in mats:
                d = ia.DeviceWeights.from_blocks(payload, blocks, rows, cols)
                keep.append(d)
                items.append((d, (cols, rows)))
        xk = {(m[1], m[0]): xs[m[1]] for m in mats}
        yk = {(m[1], m[0]): ys[m[0]] for m in mats}
        t = time_gemvs(torch, items, xk, yk, 5) / copies
        out[f"stack_{key}_payload_MB"] = round(payload_bytes / 1e6, 2)
        # what the GEMV reads: the window streams (payload + window headers + block tags + padding)
        out[f"stack_{key}_stored_MB"] = round(sum(d.info()["stored_bytes"] for d in keep[:len(mats)]) / 1e6, 2)
        out[f"stack_{key}_us_per_layer"] = round(t * 1e6, 1)
        out[f"stack_{key}_GBps"] = round(payload_bytes / t / 1e9, 1)
        out[f"stack_{key}_tok_per_s_32_layers"] = round(1.0 / (32 * t), 1)
        # the same layer with the projections that share an input stacked at load time: q/k/v and gate/up as one
        # tensor each, four launches instead of seven
        sitems, skeep = [], []
        for c in range(copies):
            q, k, v, o, gate, up, down = keep[7 * c: 7 * c + 7]
            qkv, gu = ia.DeviceWeights.stack_rows([q, k, v]), ia.DeviceWeights.stack_rows([gate, up])
            skeep += [qkv, gu]
            sitems += [(qkv, (4096, 12288)), (o, (4096, 4096)), (gu, (4096, 22016)), (down, (11008, 4096))]
        ysk = dict(yk)
        ysk[(4096, 12288)] = torch.empty((1, 12288), device="cuda")
        ysk[(4096, 22016)] = torch.empty((1, 22016), device="cuda")
        xsk = dict(xk)
        xsk[(4096, 12288)] = xsk[(4096, 22016)] = xs[4096]
        ts = time_gemvs(torch, sitems, xsk, ysk, 5) / copies
        out[f"stack_{key}_stacked_us_per_layer"] = round(ts * 1e6, 1)
        out[f"stack_{key}_stacked_GBps"] = round(payload_bytes / ts / 1e9, 1)
        out[f"stack_{key}_stacked_tok_per_s_32_layers"] = round(1.0 / (32 * ts), 1)
        # ... and as the decode step runs it: both RMSNorms and the SwiGLU product inside the launches that consume them
        L = _lib_handles(ia)
        wn = torch.randn(4096, device="cuda") * 0.1
        scratch = torch.empty(3 * 11008 + 4096, device="cuda")
        cur = lambda: ia._lib.current_stream()  # noqa: E731

        def layer(c):
            qkv, gu = skeep[2 * c], skeep[2 * c + 1]
            o, down = keep[7 * c + 3], keep[7 * c + 6]
            ia._lib.check(L.oilhip_gemv_rmsnorm_f32(qkv.handle, xs[4096].data_ptr(), wn.data_ptr(), ysk[(4096, 12288)].data_ptr(),
                                                    1, None, cur()))
            o.gemv(xs[4096], out=ys[4096])                               # attention itself is not modelled
            ia._lib.check(L.oilhip_mlp_step_f32(gu.handle, down.handle, ys[4096].data_ptr(), wn.data_ptr(),
                                                ysk[(4096, 12288)].data_ptr(), 1, scratch.data_ptr(), cur()))

        for c in range(copies):
            layer(c)
        torch.cuda.synchronize()
        fstream, fgraph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
        with torch.cuda.stream(fstream):
            with torch.cuda.graph(fgraph, stream=fstream):
                for c in range(copies):
                    layer(c)
        torch.cuda.synchronize()
        with torch.cuda.stream(fstream):
            fgraph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(fstream)
            for _ in range(5):
                fgraph.replay()
            e1.record(fstream)
            torch.cuda.synchronize()
        tf = e0.elapsed_time(e1) * 1e-3 / (5 * copies)
        out[f"stack_{key}_fused_layer_us"] = round(tf * 1e6, 1)
        out[f"stack_{key}_fused_layer_tok_per_s_32_layers"] = round(1.0 / (32 * tf), 1)
        for d in keep + skeep:
            d.close()
    return out


def bench_prefill(torch, ia, payload, blocks):
    """OIL4 prefill GEMM (bf16 MFMA, FP32 accumulate): M in {512, 2048}, K=4096, N in {4096, 11008}."""
    out = {}
    wq = make_weights(4096, 4096, seed=9)
    pq, bq = ia.block_codec.quantize_tensor(wq, ia.Format.OIL4)
    for (rows, cols, pay, blk) in ((11008, 4096, payload, blocks), (4096, 4096, pq, bq)):
        with ia.DeviceWeights.from_blocks(pay, blk, rows, cols) as d:
            for M in (512, 2048):
                x = torch.randn(M, cols, device="cuda").to(torch.bfloat16)
                y = torch.empty((M, rows), dtype=torch.float32, device="cuda")
                t = time_calls(torch, lambda: d.gemm_bf16(x, out=y))          # at least 50 ms of launches
                out[f"prefill_M{M}_N{rows}_TFLOPs"] = round(2.0 * M * rows * cols / t / 1e12, 1)
                out[f"prefill_M{M}_N{rows}_us"] = round(t * 1e6, 1)
                if M == 512 and rows == 11008:                                # the reference's own call: FP32 activations
                    xf = x.float()
                    tf = time_calls(torch, lambda: d.gemm_f32(xf, out=y))
                    out["prefill_fp32_in_M512_N11008_us"] = round(tf * 1e6, 1)
                    for Ms in (64, 128, 256):                                 # short prompts: chunks below the reference's cap of 512
                        xs, ys = xf[:Ms].contiguous(), y[:Ms]
                        ts = time_calls(torch, lambda: d.gemm_f32(xs, out=ys), min_ms=20.0)
                        out[f"prefill_fp32_in_M{Ms}_N11008_us"] = round(ts * 1e6, 1)
    # a tensor that is not uniform OIL4 (here SPARK_Q0): decoded to bf16 slab by slab, then the same kernel over a dense operand
    ws = make_weights(11008, 4096, seed=12)
    ps, bs = ia.block_codec.quantize_tensor(ws, ia.Format.SPARK_Q0)
    with ia.DeviceWeights.from_blocks(ps, bs, 11008, 4096) as d:
        x = torch.randn(2048, 4096, device="cuda").to(torch.bfloat16)
        y = torch.empty((2048, 11008), dtype=torch.float32, device="cuda")
        t = time_calls(torch, lambda: d.gemm_bf16(x, out=y))
        out["prefill_spark_q0_M2048_N11008_TFLOPs"] = round(2.0 * 2048 * 11008 * 4096 / t / 1e12, 1)
    # what this box reaches with a plain bf16 GEMM of the largest shape (rocBLAS / hipBLASLt through torch), and with a
    # plain device-to-device copy: the practical ceilings next to the vendor peaks
    a = torch.randn(2048, 4096, device="cuda").to(torch.bfloat16)
    b = torch.randn(11008, 4096, device="cuda").to(torch.bfloat16)
    for _ in range(3):
        torch.matmul(a, b.t())
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        torch.matmul(a, b.t())
    e1.record()
    torch.cuda.synchronize()
    out["plain_bf16_gemm_M2048_N11008_TFLOPs"] = round(2.0 * 2048 * 11008 * 4096 / (e0.elapsed_time(e1) * 1e-3 / 20) / 1e12, 1)
    src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    for _ in range(2):
        dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    out["plain_copy_1GiB_read_plus_write_GBps"] = round(2.0 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3 / 5) / 1e9, 1)
    return out


def bench_read_probe(torch, ia):
    """What a pure reader reaches on this device with the GEMVs' load pattern (liboilhip_probe.so, a measurement tool
    built beside the product library): (a) steady state, one
    launch over a 902 MB buffer, swept over waves per SIMD (2 / 4 / 8) and loads in flight (2 / 4 / 8), plain and
    non-temporal loads; (b) the headline's shape of work, 22.5 MB per launch as a graph of 40 dependent launches over
    40 different slices, which adds the launch gap and the ramp the GEMV pays too."""
    import ctypes
    path = os.path.join(os.path.dirname(ia._lib.LIB_PATH), "liboilhip_probe.so")
    if not os.path.exists(path):
        return {"read_only_probe": "liboilhip_probe.so not built"}
    L = ctypes.CDLL(path)
    L.oilprobe_read.restype = ctypes.c_int
    L.oilprobe_read.argtypes = [ctypes.c_void_p, ctypes.c_uint64] + [ctypes.c_int] * 5 + [ctypes.c_void_p, ctypes.c_void_p]
    L.oilprobe_last_error.restype = ctypes.c_char_p
    one, copies = 22544384, 40
    buf = torch.empty(one * copies, dtype=torch.uint8, device="cuda").fill_(1)
    sink = torch.zeros(1 << 16, dtype=torch.int32, device="cuda")

    def launch(ptr, nbytes, u, nt, pat, wgs, thr):
        if L.oilprobe_read(ptr, nbytes, u, nt, pat, wgs, thr, sink.data_ptr(), ia._lib.current_stream()) != 0:
            raise RuntimeError(L.oilprobe_last_error().decode())

    out, table = {}, {}
    best = 0.0
    for wps, (wgs, thr) in ((2, (256, 512)), (4, (512, 512)), (8, (1024, 512))):
        for u in (2, 4, 8):
            for nt in (0, 1):
                for pat in (0, 1):
                    for _ in range(2):
                        launch(buf.data_ptr(), buf.numel(), u, nt, pat, wgs, thr)
                    torch.cuda.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(4):
                        launch(buf.data_ptr(), buf.numel(), u, nt, pat, wgs, thr)
                    e1.record()
                    e1.synchronize()
                    gbs = buf.numel() / (e0.elapsed_time(e1) * 1e-3 / 4) / 1e9
                    key = f"w{wps}_u{u}_{'nt' if nt else 'ld'}_{'il' if pat else 'ct'}"
                    table[key] = round(gbs)
                    best = max(best, gbs)
    out["read_only_probe_GBps"] = round(best, 1)
    out["read_only_probe_steady_table_GBps"] = table
    # the GEMVs' own launch pattern: dependent launches of one tensor's bytes each over a ring of slices (graph replay),
    # for the payload sizes of the M=1 legs -- what a kernel that did nothing with the data would score per shape
    stream = torch.cuda.Stream()
    per_shape = {}
    for label, nbytes in (("oil4_4096x4096", 4096 * 4096 // 2), ("oil8_4096x4096", 4096 * 4096 + 4096 * 16 * 4),
                          ("oil4_11008x4096", one), ("oil4_22016x4096", 2 * one), ("oil4_131072x4096", 131072 * 4096 // 2)):
        nbytes = (nbytes + 1023) // 1024 * 1024
        ncopies = max(2, min(copies, buf.numel() // nbytes))
        best_us = None
        for (wgs, thr, u) in ((256, 512, 4), (512, 512, 4), (1024, 512, 2), (1024, 512, 4)):
            with torch.cuda.stream(stream):
                for c in range(ncopies):
                    launch(buf.data_ptr() + c * nbytes, nbytes, u, 1, 0, wgs, thr)
                stream.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for c in range(ncopies):
                        launch(buf.data_ptr() + c * nbytes, nbytes, u, 1, 0, wgs, thr)
                reps = max(3, min(50, int(2.0e9 // (nbytes * ncopies))))
                for _ in range(3):
                    g.replay()
                stream.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
                e1.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * ncopies)
            best_us = us if best_us is None else min(best_us, us)
        per_shape[label] = {"bytes": nbytes, "us_per_launch": round(best_us, 2), "GBps": round(nbytes / best_us / 1e3, 1),
                            "frac_of_hbm_peak": round(nbytes / best_us / 1e3 / HBM_PEAK_GBS, 4)}
    out["read_only_probe_per_launch"] = per_shape
    out["read_only_probe_22MB_per_launch_us"] = per_shape["oil4_11008x4096"]["us_per_launch"]
    out["read_only_probe_22MB_per_launch_GBps"] = per_shape["oil4_11008x4096"]["GBps"]
    return out


def bench_dequant_and_engine(torch, ia, payload, blocks):
    """dequantize_block_all over the whole headline tensor (180 MB of FP32 written) and OIL8Engine::quant_gemm at M=1
    (B laid out [K][N], k-ordered FMA chain per output: bit-identical to the reference loop)."""
    L = ia._lib.lib()
    out = {}
    with ia.DeviceWeights.from_blocks(payload, blocks, ROWS, COLS) as d:
        o = torch.empty(ROWS * COLS, dtype=torch.float32, device="cuda")
        for _ in range(3):
            ia._lib.check(L.oilhip_dequant_f32(d.handle, o.data_ptr(), ia._lib.current_stream()))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            ia._lib.check(L.oilhip_dequant_f32(d.handle, o.data_ptr(), ia._lib.current_stream()))
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / 20
        out["dequant_oil4_11008x4096_us"] = round(t * 1e6, 1)
        out["dequant_oil4_11008x4096_written_GBps"] = round(ROWS * COLS * 4 / t / 1e9, 1)
        del o
    N = K = 4096
    b = torch.randint(0, 256, (K * N,), dtype=torch.uint8, device="cuda")
    cb = torch.linspace(-8, 8, 256, device="cuda")
    a = torch.randn(K, device="cuda")
    c = torch.empty(N, device="cuda")
    call = lambda: ia._lib.check(L.oilhip_engine_quant_gemm(8, a.data_ptr(), b.data_ptr(), cb.data_ptr(), c.data_ptr(),  # noqa: E731
                                                             1, N, K, ia._lib.current_stream()))
    call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        call()
    e1.record()
    torch.cuda.synchronize()
    out["engine_oil8_quant_gemm_M1_4096x4096_us"] = round(e0.elapsed_time(e1) * 1e2, 1)
    return out


def bench_kv_cache(torch, ia, with_cpu=False):
    """The OIL4 KV cache of one Llama-7B-shaped layer (32 heads x 128, block 64): get_range over a 4096-token context
    (per value 0.5 B of codes + 0.5 B of centroids read, 4 B of FP32 written, K and V in one launch), a 2048-token
    prefill append and a one-token decode append (Lloyd-Max on the device, one wavefront per 64-value chunk)."""
    heads, dim, ctx = 32, 128, 4096
    pt = heads * dim
    c = ia.OIL4KVCache(1, ctx + 64, heads, dim, 64)
    k = torch.randn((1, heads, 2048, dim), device="cuda")
    v = torch.randn((1, heads, 2048, dim), device="cuda")
    k1, v1 = k.reshape(-1)[:pt].reshape(1, heads, 1, dim).contiguous(), v.reshape(-1)[:pt].reshape(1, heads, 1, dim).contiguous()

    def timed(fn, reps, before=None):
        tot = 0.0
        for r in range(reps + 1):
            if before:
                before()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            if r:
                tot += e0.elapsed_time(e1) * 1e-3
        return tot / reps

    out = {}
    t = timed(lambda: c.append(0, k, v), 5, before=c.clear)
    out["kv_append_prefill_2048tok_us"] = round(t * 1e6, 1)
    out["kv_append_prefill_Mtok_per_s"] = round(2048 / t / 1e6, 3)
    c.clear()
    c.append(0, k, v)
    c.append(0, k, v)
    t = timed(lambda: c.append(0, k1, v1), 20)
    out["kv_append_decode_1tok_us"] = round(t * 1e6, 1)
    L = ia._lib.lib()
    import ctypes as C
    outs = [(torch.empty((ctx, pt), dtype=torch.float32, device="cuda"), torch.empty((ctx, pt), dtype=torch.float32, device="cuda"))
            for _ in range(4)]                         # 4 x 134 MB of outputs in turn: more than the 256 MB Infinity Cache
    got = C.c_int64()

    def ring():
        for r in range(12):
            ko, vo = outs[r % 4]
            ia._lib.check(L.oilhip_kv_get_range(c._h, 0, 0, ctx, ko.data_ptr(), vo.data_ptr(), C.byref(got), ia._lib.current_stream()))

    t = timed(ring, 3) / 12
    assert got.value == ctx
    nbytes = 2 * ctx * pt * (0.5 + 32 / 64 + 4)
    out["kv_get_range_4096tok_us"] = round(t * 1e6, 1)
    out["kv_get_range_4096tok_GBps"] = round(nbytes / t / 1e9, 1)
    if with_cpu:
        # the same cache on one host core through the oracle's restatement of OIL4KVCache (a bounded sample: 32 tokens
        # appended, then read back 8 times)
        import numpy as np
        import oracle as O
        oc = O.KVCache(64, heads, dim, 64)
        kh, vh = k.reshape(-1, pt)[:32].cpu().numpy(), v.reshape(-1, pt)[:32].cpu().numpy()
        t0 = time.perf_counter()
        oc.append(kh, vh)
        t_app = time.perf_counter() - t0
        t0 = time.perf_counter()
        for _ in range(8):
            oc.get_range(0, 32)
        t_get = (time.perf_counter() - t0) / 8
        out["kv_cpu_port_1core_append_us_per_token"] = round(t_app / 32 * 1e6, 1)
        out["kv_cpu_port_1core_get_range_GBps"] = round(2 * 32 * pt * (0.5 + 32 / 64 + 4) / t_get / 1e9, 3)
    return out


def bench_moe(torch, ia):
    """MoE step: 8 OIL4 experts (gate/up 14336x4096, down 4096x14336: 704.6 MB of payload), 64 tokens, top-2.
    One expert is quantized on the host and uploaded 8 times (distinct device copies, same bytes)."""
    import numpy as np
    from innova_amd import moe
    D, F, E, T, K = 4096, 14336, 8, 64, 2
    mats = []
    for seed, (r, c) in enumerate(((F, D), (F, D), (D, F))):
        mats.append(ia.block_codec.quantize_tensor(make_weights(r, c, seed=50 + seed), ia.Format.OIL4))
    experts = [moe.ExpertFFN(ia.DeviceWeights.from_blocks(*mats[0], F, D), ia.DeviceWeights.from_blocks(*mats[1], F, D),
                             ia.DeviceWeights.from_blocks(*mats[2], D, F)) for _ in range(E)]
    rng = np.random.default_rng(2026)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 1.0                                   # an uneven load
    _, idx, w = moe.softmax_with_topk(logits, K)
    hist = np.bincount(idx.ravel(), minlength=E).tolist()
    x = torch.randn(T, D, device="cuda")
    # one step (all its launches, no copy, no host wait) captured once and replayed: the timed region holds graph
    # replays only, as for the headline ring
    ws, out = moe.moe_workspace(x, experts, K), torch.empty(T, D, device="cuda")
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        moe.moe_dispatch_batched(x, experts, idx, w, want_z_loss=False, workspace=ws, out=out)
        st.synchronize()
        eager = out.clone()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            moe.moe_dispatch_batched(x, experts, idx, w, want_z_loss=False, workspace=ws, out=out)
        t = time_calls(torch, g.replay, warm=2)                                    # >= 50 ms of steps
        st.synchronize()
        assert float((out - eager).norm() / eager.norm()) <= 1e-6, "a replayed MoE step differs from the eager one"
    touched = sum(3 * D * F // 2 for h in hist if h > 0)
    for e in experts:
        for d in (e.gate_proj, e.up_proj, e.down_proj):
            d.close()
    return {"moe_tokens_per_expert": hist, "moe_ms_per_step": round(t * 1e3, 3),
            "moe_GBps": round(touched / t / 1e9, 1), "moe_TFLOPs": round(2.0 * 3 * D * F * T * K / t / 1e12, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100, help="timed steps per round (a step = one replay of the 40-launch ring)")
    ap.add_argument("--warmup", type=int, default=5, help="untimed warm-up steps")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--kv-only", action="store_true", help="only run the KV-cache leg (for profiling its kernels)")
    ap.add_argument("--prefill-only", action="store_true", help="only run the prefill GEMM leg (for profiling its kernels)")
    ap.add_argument("--moe-only", action="store_true", help="only run the MoE step leg (for profiling its kernels)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run plain 1 GiB device copies (reference for the FETCH_SIZE/WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path would shard by output rows, with no "
                 "reduction between GPUs); run with --gpus 1")

    import numpy as np
    import torch

    import innova_amd as ia

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    info = ia.probe()
    log(f"device: {info['name']} gfx{info['gfx']} {info['compute_units']} CUs")
    if args.kv_only:
        print(json.dumps({"kv_cache_leg": bench_kv_cache(torch, ia, with_cpu=not args.no_cpu)}), flush=True)
        return
    if args.moe_only:
        print(json.dumps({"moe_leg": bench_moe(torch, ia)}), flush=True)
        return
    if args.prefill_only:
        payload, blocks = ia.block_codec.quantize_tensor(make_weights(ROWS, COLS, seed=20260803), ia.Format.OIL4)
        print(json.dumps({"prefill_leg": bench_prefill(torch, ia, payload, blocks)}), flush=True)
        return
    if args.calibrate_copy:
        a = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()     # 1 GiB
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)                                                              # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy": {"bytes_read": a.numel() * 4, "bytes_written": a.numel() * 4, "copies": 5}}))
        return

    w = make_weights(ROWS, COLS, seed=20260803)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    assert payload.size == ROWS * COLS // 2
    ring = Ring(ia, payload, blocks, ROWS, COLS, RING)
    xh = np.random.default_rng(1).standard_normal((1, COLS)).astype(np.float32)
    x = torch.from_numpy(xh).cuda()
    y = torch.empty((1, ROWS), dtype=torch.float32, device="cuda")

    sec, wall, rounds, region_s = time_ring(torch, ring, x, y, args.steps, args.warmup, settle_s=0.3)
    algo_bytes = ring.payload_bytes + 4 * COLS + 4 * ROWS          # weights + x + y, each once
    value = ring.payload_bytes / sec / 1e9
    achieved = algo_bytes / sec / 1e9

    traffic = HBM_TRAFFIC_BYTES_PER_LAUNCH

    out = {
        "metric": "OIL4 GEMV effective weight GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec * RING * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "OIL4 decode GEMV, Llama-7B up/gate projection K=4096 -> N=11008, M=1, "
                               "FP32 activations ~N(0,1), weights ~N(0,0.02) quantized to OIL4 wire blocks",
                   "rows": ROWS, "cols": COLS, "M": 1, "ring_copies": RING, "launches_per_step": RING,
                   "payload_bytes": ring.payload_bytes, "timed_rounds": rounds, "timed_launches": rounds * args.steps * RING,
                   "timed_region_ms": round(region_s * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": "cited from profiles/oil4_gemv_4096x11008_m1.md (rocprofv3 --pmc), not measured in this run",
                     "us_per_launch": round(sec * 1e6, 3)},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "host_wall_ms_per_step": round(wall * RING * 1e3, 6),
    }

    if not args.no_extra:
        extra = {}
        for M in (4, 16, 32):
            xm = torch.randn(M, COLS, device="cuda")
            ym = torch.empty((M, ROWS), dtype=torch.float32, device="cuda")
            s_m = time_ring(torch, ring, xm, ym, 4, 1)[0]
            extra[f"up_gate_M{M}_GBps"] = round(ring.payload_bytes / s_m / 1e9, 1)
        ring.close()
        # down projection K = 11008 -> N = 4096
        wd = make_weights(COLS, ROWS, seed=7)
        pd, bd = ia.block_codec.quantize_tensor(wd, ia.Format.OIL4)
        ring_d = Ring(ia, pd, bd, COLS, ROWS, RING)
        xd = torch.randn(1, ROWS, device="cuda")
        yd = torch.empty((1, COLS), dtype=torch.float32, device="cuda")
        s_d = time_ring(torch, ring_d, xd, yd, 4, 1)[0]
        extra["down_M1_GBps"] = round(ring_d.payload_bytes / s_d / 1e9, 1)
        for M in (4, 16):
            xm = torch.randn(M, ROWS, device="cuda")
            ym = torch.empty((M, COLS), dtype=torch.float32, device="cuda")
            s_m = time_ring(torch, ring_d, xm, ym, 4, 1)[0]
            extra[f"down_M{M}_GBps"] = round(ring_d.payload_bytes / s_m / 1e9, 1)
        ring_d.close()
        # weights-only decode rate of a Llama-7B-shaped stack: per layer 4 x (4096x4096), 2 x up/gate, 1 x down
        t_qkvo = None
        wq = make_weights(4096, 4096, seed=9)
        pq, bq = ia.block_codec.quantize_tensor(wq, ia.Format.OIL4)
        ring_q = Ring(ia, pq, bq, 4096, 4096, 64)
        xq = torch.randn(1, 4096, device="cuda")
        yq = torch.empty((1, 4096), dtype=torch.float32, device="cuda")
        t_qkvo = time_ring(torch, ring_q, xq, yq, 4, 1)[0]
        ring_q.close()
        per_layer = 4 * t_qkvo + 2 * sec + s_d
        extra["qkvo_4096x4096_M1_GBps"] = round(pq.size / t_qkvo / 1e9, 1)
        extra["decode_tok_per_s_7B_weight_gemvs_only"] = round(1.0 / (32 * per_layer), 1)
        extra.update(bench_fused_layer(torch, ia, 32 * per_layer))
        # the headline shape with the weights resident in the 256 MB Infinity Cache (two copies, 45 MB): NOT the headline,
        # which streams 902 MB; reported for comparison only
        ring_c = Ring(ia, payload, blocks, ROWS, COLS, 2)
        two = ring_c.items
        ring_c.items = two * (RING // 2)               # the same 40 launches per replay, alternating between the two copies
        yc = torch.empty((1, ROWS), dtype=torch.float32, device="cuda")
        s_c = time_ring(torch, ring_c, x, yc, 4, 1)[0]
        ring_c.items = two
        ring_c.close()
        extra["headline_shape_cache_resident_us"] = round(s_c * 1e6, 2)
        extra["headline_shape_cache_resident_GBps"] = round(int(payload.size) / s_c / 1e9, 1)
        extra.update(bench_read_probe(torch, ia))
        extra.update(bench_tall(torch, ia))
        extra.update(bench_oil8(torch, ia))
        extra.update(bench_dequant_and_engine(torch, ia, payload, blocks))
        extra.update(bench_mixed_stack(torch, ia))
        extra.update(bench_prefill(torch, ia, payload, blocks))
        extra.update(bench_moe(torch, ia))
        extra.update(bench_kv_cache(torch, ia, with_cpu=not args.no_cpu))
        # the secondary legs against the same published peaks as the headline's roofline (HBM 8 TB/s, bf16 MFMA 2.5 PFLOP/s):
        # payload GB/s for the memory-bound ones, TFLOP/s for the prefill GEMM
        sec_roof = {}
        for leg, key, bound in (("config1_oil8_block_gemv", "oil8_block_4096x4096_M1_GBps", "hbm"),
                                ("config1_oil8_flat_gemv", "oil8_flat_4096x4096_M1_GBps", "hbm"),
                                ("config2_oil4_gemv_M4", "up_gate_M4_GBps", "hbm"),
                                ("config2_oil4_gemv_M16", "up_gate_M16_GBps", "hbm"),
                                ("config3_planner_1p50_stack", "stack_planner_1p50_GBps", "hbm"),
                                ("config3_planner_1p50_stack_stacked", "stack_planner_1p50_stacked_GBps", "hbm"),
                                ("config3_spark_mix_q0_stack_stacked", "stack_spark_mix_q0_stacked_GBps", "hbm"),
                                ("config4_prefill_M2048_N11008", "prefill_M2048_N11008_TFLOPs", "mfma"),
                                ("config4_prefill_M512_N4096", "prefill_M512_N4096_TFLOPs", "mfma"),
                                ("config5_moe_step", "moe_GBps", "hbm"),
                                ("dequant_oil4_written", "dequant_oil4_11008x4096_written_GBps", "hbm"),
                                ("kv_cache_get_range_4096tok", "kv_get_range_4096tok_GBps", "hbm")):
            if key in extra:
                peak = HBM_PEAK_GBS if bound == "hbm" else 2500.0
                sec_roof[leg] = {"bound": bound, "achieved": extra[key], "peak": peak,
                                 "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "frac": round(extra[key] / peak, 4)}
        extra["roofline_secondary"] = sec_roof
        out["extra"] = extra
    else:
        ring.close()

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(payload, blocks, ROWS, COLS, xh)
        out.setdefault("extra", {}).update(cpu_flat_oil8())      # the second CPU leg: flat-codebook gather, one thread

    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the Blaze sparse CTR inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward pass (Embedding gather/pool -> FC 896-512-256-2 with PReLU -> softmax) over one
synthetic batch of 2048 samples (config 2), inputs already resident in HBM.  A pool of pre-generated
batches is cycled so the id stream is not one cached batch.  The step is Predictor.Forward through the Blaze_* C ABI
(the drop-in path), issued by a few serving threads with one Predictor set and HIP stream each, as the reference is
deployed (blaze/example/cpp/predictor_example.cc:129-140,189).  Prints ONE JSON line:

  value / ms_per_step     exactly K steps after the warm-up (every predictor has run at least twice before the clock
                          starts, whatever W says: W is a floor);
  steady_state            the same loop over a fixed number of steps (>= 2000), so a short K does not hide the rate;
  p50_ms / p99_ms         latency of a request under the load of the steady-state run: every pass of that run, from the
                          start of its launch to the return of its wait on its serving thread (latency_by_load: the
                          throughput / latency pairs at one and two passes queued per thread and at fewer threads; latency_unloaded: one
                          request at a time on one thread, over max(K, 1000) forwards);
  with_host_feed          every step feeds all inputs from host memory and copies the output back (PCIe inclusive);
  roofline                the pooling kernel: algorithmic bytes per launch / average launch duration (HIP events
                          around a replayed graph of back-to-back launches over the pooled batches);
  per_config              configs 1, 3, 4 and 5 of the benchmark definition, each with its own rate and roofline;
  cpu_baseline            the CPU restatement of the reference's path on the box's host cores (a bounded sample).
"""
import argparse
import ctypes
import json
import os
import re
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "x-deeplearning_amd"))
sys.path.insert(1, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16/bf16
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "c2_embed_pool_hbm_traffic.md")


def pool_traffic_from_profile():
    """HBM-side bytes per launch of the pooling kernel on the default workload, as the committed counter profile states
    them (a line `traffic_bytes_per_launch: N` and a line `collected: <date>`); None when the file has no such line."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
    d = re.search(r"collected:\s*([^\n]+)", text)
    if not m:
        return None, None
    return int(m.group(1)), "profiles/%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, collected %s)" % (
        os.path.basename(TRAFFIC_PROFILE), d.group(1).strip() if d else "?")


def graph_timed(torch, fn, n_distinct, reps, rounds=5, warm_ms=0.0):
    """Average duration in us of fn(i): `reps` back-to-back calls recorded into one HIP graph on torch's current stream
    (so host launch cost is not in it), replayed `rounds` times between two events on that stream.  warm_ms: replay for
    about that long first (a 200 us MFMA kernel runs up to 20 % slower at first and keeps getting faster for some 100 ms
    after the device was idle or doing lighter work: whichever of two kernels is timed first would lose)."""
    for i in range(n_distinct):
        fn(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(reps):
            fn(i)
    t0 = time.perf_counter()
    g.replay()
    torch.cuda.synchronize()
    one = max(time.perf_counter() - t0, 1e-5)
    for _ in range(min(200, int(warm_ms * 1e-3 / one))):
        g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(rounds):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * rounds)


def latency_ms(np, step, n):
    lat = np.empty(n)
    for i in range(n):
        a = time.perf_counter()
        step(i)
        lat[i] = (time.perf_counter() - a) * 1e3
    lat.sort()
    return float(lat[n // 2]), float(lat[min(n - 1, int(n * 0.99))]), n


def latency_stats(np, lat_ms):
    """p50 / p99 / mean of a set of per-pass latencies (ms)"""
    lat = np.sort(np.asarray(lat_ms, dtype=np.float64))
    n = len(lat)
    if n == 0:
        return None
    return {"p50_ms": round(float(lat[n // 2]), 4), "p99_ms": round(float(lat[min(n - 1, int(n * 0.99))]), 4),
            "mean_ms": round(float(lat.mean()), 4), "samples": n}


def hbm_roofline(kernel, alg_bytes, us, traffic=None):
    gbs = alg_bytes / us / 1e3
    return {"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 5), "traffic": traffic, "algorithmic_bytes_per_launch": int(alg_bytes),
            "avg_launch_us": round(us, 2)}


def mfma_roofline(kernel, flops, us):
    tf = flops / us / 1e6
    return {"kernel": kernel, "bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tf / MFMA_PEAK_TFLOPS, 5), "traffic": None, "flops_per_launch": int(flops), "avg_launch_us": round(us, 2)}


# ------------------------------------------------------------------------------------------------ counter calibration
def calibration_copy(torch, bz):
    """A plain copy of known size (bz_concat_kernel, one piece of 256 MiB, 5 launches): what rocprofv3's FETCH_SIZE /
    WRITE_SIZE read for it is the scale for the same counters on the other kernels of the run.  Part of --counters-run."""
    rows, width = 65536, 4096
    src = torch.ones(rows * width, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    d = bz.ConcatDesc()
    d.src[0], d.width[0], d.src_pitch[0] = src.data_ptr(), width, width
    d.dst, d.dst_pitch, d.rows, d.n = dst.data_ptr(), width, rows, 1
    for _ in range(5):
        bz.check(bz.lib().bz_concat_cols(ctypes.byref(d), None))
    torch.cuda.synchronize()
    assert bool((dst == 1).all())
    return {"kernel": "bz_concat_kernel", "launches": 5, "bytes_read_per_launch": rows * width,
            "bytes_written_per_launch": rows * width}


# ------------------------------------------------------------------------------------------------ other configurations
def bench_predictor_model(np, torch, pb, predictors, batch, threads, steps, lat_steps):
    """samples/s over `threads` serving threads + single-request latency of a list of fed predictors."""
    T = threads
    pool = pb.ServePool(T, 1)  # a plain synchronous Forward per request on every thread
    pool.run(predictors, 2 * len(predictors))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    pool.run(predictors, steps)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    loaded = latency_stats(np, pool.latencies_ms())  # every pass of that run, launch to the return of its wait
    p50, p99, n = latency_ms(np, lambda i: predictors[i % len(predictors)].forward(), lat_steps)
    return {"samples/s": round(batch * steps / (t1 - t0), 1), "ms_per_step": round((t1 - t0) * 1e3 / steps, 5), "steps": steps,
            "serving_threads": T, "p50_ms": loaded["p50_ms"], "p99_ms": loaded["p99_ms"], "latency_samples": loaded["samples"],
            "unloaded": {"p50_ms": round(p50, 4), "p99_ms": round(p99, 4), "latency_samples": n,
                         "note": "one request at a time on one thread"}}


def count_launches(p):
    """operators of one Forward that ran (the profile observer's trace), as {op type: count}"""
    p.register_observers(["profile"])
    p.forward()
    ev = json.loads(p.dump_observers()["profile"])["traceEvents"]
    out = {}
    for e in ev:
        if e.get("dur", 0) > 0:
            k = e["name"].split(":")[0]
            out[k] = out.get(k, 0) + 1
    return out


def bench_config1(np, torch, bz, pb, threads):
    from ctr_model import build_manager, make_predictor
    from synth import Config1, embedding_bytes
    cfg = Config1()
    tables, mlp = cfg.tables(), cfg.mlp()
    n = 2 * threads
    sparse, dense = cfg.batches(n)
    pm, fgs = build_manager(cfg, tables, mlp, np.float32)
    preds = [make_predictor(pm, fgs, sparse[b], dense[b], np.float32) for b in range(n)]
    res = bench_predictor_model(np, torch, pb, preds, cfg.batch, threads, 4000, 1000)
    # the pooling kernel alone, through the kernel layer
    dts = [bz.DeviceTable(t) for t in tables]
    plans, keep, nnz = [], [], []
    for b in range(n):
        out = torch.zeros((cfg.batch, cfg.slots * cfg.dim), dtype=torch.float32, device="cuda")
        items = []
        for s, (ids, vals, seg) in enumerate(sparse[b]):
            t = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(seg).cuda()]
            keep.append(t)
            items.append(dict(table=dts[s], ids=t[0], values=t[1], segments=t[2], out=out, col=s * cfg.dim, udf=bz.SUM))
        plans.append(bz.EmbeddingPlan(items))
        nnz.append(sum(ids.size for ids, _, _ in sparse[b]))
    us = graph_timed(torch, lambda i: plans[i % n].run(), n, 8 * n, warm_ms=50.0)
    alg = float(np.mean([embedding_bytes(z, cfg.batch, cfg.slots, cfg.dim * 4, 0, cfg.slots * cfg.dim, 4) for z in nnz]))
    res["workload"] = cfg.name
    res["dtype"] = "f32"
    res["roofline"] = hbm_roofline("bz_embed_pool_kernel", alg, us)
    return res


def bench_config3(np, torch, bz, pb, threads):
    import din_model
    cfg = din_model.Config3()
    tables, weights = cfg.tables(), cfg.weights()
    n = 2 * threads
    preds = []
    pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16)
    for b in range(n):
        p = pm.create_predictor(1, 0)
        din_model.feed(p, inputs, cfg.batch_inputs(seed_offset=b), np.float16)
        preds.append(p)
    res = bench_predictor_model(np, torch, pb, preds, cfg.batch, threads, 2000, 1000)
    probe = pm.create_predictor(1, 0)
    din_model.feed(probe, inputs, cfg.batch_inputs(seed_offset=0), np.float16)
    probe.forward()
    ran = count_launches(probe)
    B, T = cfg.batch, cfg.T
    D3 = 3 * cfg.dim
    att = cfg.att_layers
    main = cfg.main_layers
    res["workload"] = cfg.name
    res["dtype"] = "f16"
    res["operators_run_per_forward"] = sum(ran.values())
    res["operators"] = ran
    res["fc_flops"] = int(2 * B * T * sum(att[i] * att[i + 1] for i in range(3)) + 2 * B * sum(main[i] * main[i + 1] for i in range(3)))
    res["attention_bgemm_bytes"] = B * T * D3 * 2 + B * T * 4 + B * D3 * 2
    # the two kernels of the attention block alone, through the kernel layer on operands of the model's shapes (two
    # sets, alternating): the attention MLP [q, k, q-k, q*k] -> 80 -> 40 -> 1 as one launch, and the attention tail
    # (score * mask, weighted sum over the history, plain sum) as one launch
    g = torch.Generator(device="cuda").manual_seed(33)
    rnd = lambda *shape: torch.randn(shape, generator=g, device="cuda")
    sets = []
    for _ in range(2):
        q, k = rnd(B, 1, D3).half(), rnd(B, T, D3).half()
        ws = [bz.pack_weight(rnd(att[i], att[i + 1]).half() / att[i] ** 0.5, False, bz.F16) for i in range(3)]
        bs = [rnd(att[i + 1]) * 0.1 for i in range(3)]
        dice = [(rnd(att[i + 1]) * 0.1, rnd(att[i + 1]) * 0.1, torch.rand(att[i + 1], generator=g, device="cuda") + 0.5) for i in range(2)]
        score = torch.empty((B * T, 1), dtype=torch.float32, device="cuda")
        mlp = bz.AttentionMlp(q, k, ws[0], bs[0], dice[0], ws[1], bs[1], dice[1], ws[2], bs[2], score)
        w16 = rnd(B, T, 1).half()
        mask = (torch.rand((B, T, 1), generator=g, device="cuda") < 0.5).half()
        sets.append((mlp, k, w16, mask))
    mlp_us = graph_timed(torch, lambda i: sets[i % 2][0].run(), 2, 16, warm_ms=20.0)
    tail_us = graph_timed(torch, lambda i: bz.weighted_pool(sets[i % 2][1], sets[i % 2][2], sets[i % 2][3]), 2, 16, warm_ms=20.0)
    res["roofline_attention_mlp"] = mfma_roofline("bz_fc_pieces_kernel (%dx%d: %d->%d->%d->%d)" % (B, T, att[0], att[1], att[2], att[3]),
                                                  sets[0][0].flops, mlp_us)
    res["roofline_attention_tail"] = hbm_roofline("bz_weighted_pool_kernel (history read once; scores and mask in, weighted sum and plain sum out)",
                                                  B * T * D3 * 2 + 2 * B * T * 2 + 2 * B * D3 * 2, tail_us)
    return res


def bench_config4(np, torch, bz):
    from synth import Config4, embedding_bytes
    cfg = Config4()
    free, _ = torch.cuda.mem_get_info()
    need = cfg.slots * cfg.rows * (cfg.dim + 4)
    if free < need * 1.15:
        return {"workload": cfg.name, "skipped": "needs %.0f GB of free HBM, %.0f GB free" % (need * 1.15 / 1e9, free / 1e9)}
    tables = cfg.tables()
    dts = [bz.DeviceTable(q, scale=sc) for q, sc in tables]
    n = 2
    plans, keep, nnz = [], [], []
    for b in range(n):
        out = torch.zeros((cfg.batch, cfg.slots * cfg.dim), dtype=torch.float16, device="cuda")
        items = []
        sp = cfg.batch_inputs(seed_offset=b)
        for s, (ids, vals, seg) in enumerate(sp):
            t = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(seg).cuda()]
            keep.append(t)
            items.append(dict(table=dts[s], ids=t[0], values=t[1], segments=t[2], out=out, col=s * cfg.dim, udf=bz.AVG))
        plans.append(bz.EmbeddingPlan(items))
        nnz.append(sum(ids.size for ids, _, _ in sp))
    us = graph_timed(torch, lambda i: plans[i % n].run(), n, 4 * n, warm_ms=50.0)
    alg = float(np.mean([embedding_bytes(z, cfg.batch, cfg.slots, cfg.dim, 4, cfg.slots * cfg.dim, 2) for z in nnz]))
    res = {"workload": cfg.name, "dtype": "i8 rows x f32 scale -> f32 accumulate -> f16 block", "ids_per_launch": int(np.mean(nnz)),
           "launches_per_step": 1 if plans[0].fused_scan else 2, "samples/s": round(cfg.batch / us * 1e6, 1),
           "roofline": hbm_roofline("bz_embed_pool_kernel", alg, us)}
    del plans, keep, dts, tables
    torch.cuda.empty_cache()
    return res


def bench_config5(np, torch, bz, tables=True):
    """tables=False: the FC tower alone on random activations (no 102 GB of tables), for counter runs of its kernels"""
    from synth import Config5, embedding_bytes
    cfg = Config5()
    mlp = cfg.mlp()
    B, D = cfg.batch, cfg.dim
    n = 2
    plans, keep, nnz, xs = [], [], [], []
    dts = None
    if tables:
        free, _ = torch.cuda.mem_get_info()
        need = cfg.slots * cfg.rows * cfg.dim * 2
        if free < need * 1.3:
            return {"workload": cfg.name, "skipped": "needs %.0f GB of free HBM, %.0f GB free" % (need * 1.3 / 1e9, free / 1e9)}
        dts = [bz.DeviceTable(t) for t in cfg.tables()]
    for b in range(n):
        if not tables:
            g = torch.Generator(device="cuda").manual_seed(5 + b)
            xs.append((torch.randn((B, cfg.slots * D), generator=g, device="cuda") * 0.5).to(torch.bfloat16))
            continue
        x = torch.zeros((B, cfg.slots * D), dtype=torch.bfloat16, device="cuda")
        xs.append(x)
        items = []
        sp = cfg.batch_inputs(seed_offset=b)
        for s, (ids, vals, seg) in enumerate(sp):
            t = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(seg).cuda()]
            keep.append(t)
            items.append(dict(table=dts[s], ids=t[0], values=t[1], segments=t[2], out=x, col=s * D, udf=bz.SUM))
        plans.append(bz.EmbeddingPlan(items))
        nnz.append(sum(ids.size for ids, _, _ in sp))
    pool_us = alg = None
    if tables:
        pool_us = graph_timed(torch, lambda i: plans[i % n].run(), n, 4 * n, warm_ms=50.0)
        alg = float(np.mean([embedding_bytes(z, B, cfg.slots, D * 2, 0, cfg.slots * D, 2) for z in nnz]))
    # the tower: bias + ReLU per layer, sigmoid head riding in the launch of the layer before it
    packed = [bz.pack_weight(w, False, bz.BF16) for w, _ in mlp]
    ys = [torch.empty((B, w.shape[1]), dtype=torch.bfloat16, device="cuda") for w, _ in mlp[:-1]]
    prob = torch.empty((B, 1), dtype=torch.float32, device="cuda")
    L = cfg.layers

    def layer(i, li):
        a = xs[i % n] if li == 0 else ys[li - 1]
        bz.fc_fused(a, packed[li], L[li], bias=mlp[li][1], act=bz.ACT_LEAKY_RELU, act_alpha=0.0, out=ys[li])

    def tail(i):  # layer n-2 with the 1-wide sigmoid layer as its head
        li = len(mlp) - 2
        bz.fc_fused(ys[li - 1], packed[li], L[li], bias=mlp[li][1], act=bz.ACT_LEAKY_RELU, act_alpha=0.0, out=ys[li],
                    head=dict(w=packed[li + 1], bias=mlp[li + 1][1], act=bz.ACT_SIGMOID, out=prob), store_out=False)

    fc_us = [graph_timed(torch, lambda i, li=li: layer(i, li), n, 4 * n, warm_ms=100.0 if li == 0 else 0.0) for li in range(len(mlp) - 2)]
    fc_us.append(graph_timed(torch, tail, n, 4 * n))
    # the vendor library's GEMM on layer 0's operands (no bias, no activation), timed the same way: a yardstick only
    w0 = packed[0][:, :L[0]]
    lib_us = graph_timed(torch, lambda i: torch.nn.functional.linear(xs[i % n], w0), n, 4 * n, warm_ms=100.0)
    flops = [2.0 * B * L[i] * L[i + 1] for i in range(len(L) - 1)]
    kern = {"pool": round(pool_us, 2)} if tables else {}
    for i, u in enumerate(fc_us[:-1]):
        kern["fc[%d]" % i] = round(u, 2)
    kern["fc[%d+%d]" % (len(mlp) - 2, len(mlp) - 1)] = round(fc_us[-1], 2)
    res = {"workload": cfg.name, "dtype": "f16 tables -> bf16 block; bf16 MFMA, f32 accumulate", "kernel_us": kern,
           "roofline_fc": dict(mfma_roofline("bz_fc_stream_kernel (layer 0: %dx%dx%d)" % (B, L[0], L[1]), flops[0], fc_us[0]),
                               library_gemm_us=round(lib_us, 2)),
           "fc_stack": {"TFLOP/s": round(sum(flops) / sum(fc_us) / 1e6, 2),
                        "frac_of_mfma_peak": round(sum(flops) / sum(fc_us) / 1e6 / MFMA_PEAK_TFLOPS, 5),
                        "flops": int(sum(flops)), "us": round(sum(fc_us), 2)}}
    if tables:
        res.update({"ids_per_launch": int(np.mean(nnz)), "pool_launches_per_step": 1 if plans[0].fused_scan else 2,
                    "samples/s_kernels_back_to_back": round(B / (pool_us + sum(fc_us)) * 1e6, 1),
                    "roofline": hbm_roofline("bz_embed_pool_kernel", alg, pool_us)})
    del plans, keep, dts, xs
    torch.cuda.empty_cache()
    return res


# ------------------------------------------------------------------------------------------------ CPU baseline
def cpu_baseline(np, cfg, tables, mlp, sparse, dense):
    """The oracle (a port of the reference's CPU path), one single-threaded predictor per thread: per id a probe of the
    reference's hash index (quick_embedding_dict.h:55-71 -> hashtable.cc:45-64), the ksum loop, then per layer sgemm of
    the BLAS numpy links (as the reference hands the product to MKL's cblas_sgemm, math/gemm.cc:13-27) + a separate
    PReLU pass, softmax.  A bounded sample of the workload: 8 batches per thread."""
    import blaze_oracle as orc
    from model_forward import ctr_forward
    from threadpoolctl import threadpool_info, threadpool_limits
    orc.build()
    rows = tables[0].shape[0]
    keys = np.arange(rows, dtype=np.uint64)
    tabs_hash = [orc.Table(t.cpu().numpy(), keys=keys) for t in tables]   # per-id hash probe, the reference's structure
    tabs_direct = [orc.Table(t.cpu().numpy()) for t in tables]            # id == row, no index
    mlp_np = [(w.cpu().numpy(), b.cpu().numpy(), s.cpu().numpy()) for (w, b, s) in mlp]
    threads = max(1, min(16, len(os.sched_getaffinity(0))))
    per_thread = 8
    blas = next(("%s %s (%s)" % (i.get("internal_api"), i.get("version"), i.get("architecture"))
                 for i in threadpool_info() if i.get("user_api") == "blas"), "numpy's matmul")

    def run_threads(tabs):
        def worker(t):
            for j in range(per_thread):
                b = (t * per_thread + j) % len(sparse)
                ctr_forward(orc, cfg, tabs, mlp_np, sparse[b], dense[b], blas=True)
        ctr_forward(orc, cfg, tabs, mlp_np, sparse[0], dense[0], blas=True)  # warm the page cache of the tables
        c0 = time.perf_counter()
        ths = [threading.Thread(target=worker, args=(t, )) for t in range(threads)]
        for t in ths:
            t.start()
        for t in ths:
            t.join()
        return cfg.batch * threads * per_thread / (time.perf_counter() - c0)

    with threadpool_limits(1, user_api="blas"):
        rate_hash = run_threads(tabs_hash)
        rate_direct = run_threads(tabs_direct)
        s0 = time.perf_counter()  # ... and the hash-probe port on one core alone
        for j in range(per_thread):
            ctr_forward(orc, cfg, tabs_hash, mlp_np, sparse[j % len(sparse)], dense[j % len(sparse)], blas=True)
        s1 = time.perf_counter()
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), "")
    except OSError:
        pass
    return {"value": round(rate_hash, 1), "unit": "samples/s", "cores": threads, "kind": "port",
            "value_without_hash_index": round(rate_direct, 1), "value_1_core": round(cfg.batch * per_thread / (s1 - s0), 1),
            "sgemm": blas, "host_cpus": os.cpu_count(), "cpu_model": model,
            "sample": "%d batches of %d (%d per thread, one single-threaded predictor per core), fp32 oracle: per-id probe of "
                      "the reference's hash index, ksum, sgemm of the BLAS numpy links on one thread + separate PReLU pass, "
                      "softmax" % (threads * per_thread, cfg.batch, per_thread)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--pool", type=int, default=32, help="number of distinct pre-generated batches")
    ap.add_argument("--steady-steps", type=int, default=4000, help="steps of the fixed-length steady-state region (>= 2000)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-config", action="store_true", help="skip configs 1, 3, 4 and 5")
    ap.add_argument("--no-feed", action="store_true", help="skip the PCIe-inclusive leg")
    ap.add_argument("--counters-run", action="store_true",
                    help="for runs under rocprofv3 --pmc, where every dispatch is serialised: skip the steady-state region, take "
                         "the latency from --steps samples only (the line then carries no steady_state), and run a plain "
                         "256 MiB copy of known size first (the scale for FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--only", choices=["c1", "c3", "c4", "c5", "c5_fc"], default=None,
                    help="run one of the other configurations alone and print its record (c5_fc: config 5's FC tower without "
                         "its 102 GB of tables); with --counters-run fewer repetitions, for runs under rocprofv3 --pmc")
    ap.add_argument("--threads", type=int, default=8,
                    help="serving threads, each with its own Predictors and HIP stream (the reference's model: one "
                         "Predictor per thread, blaze/api/cpp_api/predictor.h:90-92)")
    ap.add_argument("--depth", type=int, default=1,
                    help="passes a serving thread keeps queued on its stream (1 = a plain synchronous Forward per request, as "
                         "the reference's serving loop; with 8 threads 2 gives 1 %% more throughput at twice the latency)")
    ap.add_argument("--kernel-api", action="store_true",
                    help="drive the kernel-layer C ABI directly instead of Predictor.Forward (lower host overhead)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (one process, no collectives); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import blaze_hip as bz
    import pyblaze_hip as pb
    from pipeline import CtrForward
    from synth import Config2

    assert torch.cuda.is_available(), "no GPU visible"
    arch = bz.device_check()
    if args.only is not None:
        T = max(1, args.threads)
        fn = {"c1": lambda: bench_config1(np, torch, bz, pb, T), "c3": lambda: bench_config3(np, torch, bz, pb, T),
              "c4": lambda: bench_config4(np, torch, bz), "c5": lambda: bench_config5(np, torch, bz),
              "c5_fc": lambda: bench_config5(np, torch, bz, tables=False)}[args.only]
        print(json.dumps({"only": args.only, "device": arch, "result": fn()}))
        return
    calibration = calibration_copy(torch, bz) if args.counters_run else None
    cfg = Config2()
    tables = cfg.tables()
    mlp = cfg.mlp()
    sparse, dense = cfg.batches(args.pool)
    # kernel-layer harness: per-kernel timing below, and the whole step in --kernel-api mode
    fwd = CtrForward(cfg, tables, mlp, sparse, dense, dtype="f16")
    torch.cuda.synchronize()
    K, W = args.steps, args.warmup
    S = max(2000, args.steady_steps)
    NB = fwd.n_batches
    T = max(1, min(args.threads, NB))
    assert NB % T == 0, "--pool must be a multiple of --threads (a pooled batch always runs on one thread)"
    warm = max(W, 2 * NB)  # W is a floor: every predictor runs at least twice before the clock starts

    predictors = None
    steady = feed_rate = loaded = by_depth = None
    if not args.kernel_api:
        # the drop-in path: one Predictor per pooled batch (inputs fed once = resident in HBM), Forward through
        # the Blaze_* C ABI; consecutive steps go round robin over T serving threads
        from ctr_model import build_manager, make_predictor
        pm, fgs = build_manager(cfg, tables, mlp, np.float16)
        predictors = [make_predictor(pm, fgs, sparse[b], dense[b], np.float16) for b in range(NB)]
        predictors[0].forward()
        ref = fwd.output(0)
        fwd.step(0)
        torch.cuda.synchronize()
        # (the fp16 model's output blob is fp16; the harness keeps the last layer's probabilities in fp32)
        assert np.allclose(predictors[0].output_asnumpy("prob").astype(np.float32), ref.cpu().numpy(), atol=1e-3), \
            "Predictor and kernel-layer harness disagree"

    streams = [torch.cuda.Stream() for _ in range(T)]
    stream_ptrs = [ctypes.c_void_p(st.cuda_stream) for st in streams]

    def run_step(i, t=0):
        if predictors is not None:
            predictors[i % NB].forward()  # launches on the calling thread's stream and waits for it
        else:
            fwd.step(i, stream_ptrs[t])
            streams[t].synchronize()

    # ---- throughput: warm-up, then exactly K steps between two synchronisations.  The Predictor path is
    # driven by the library's own serving threads (Blaze_ServePool*: a C++ loop per thread, as a serving binary
    # would run it); the kernel-layer path by Python threads.
    if predictors is not None:
        pool = pb.ServePool(T, args.depth)
        pool.run(predictors, warm)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pool.run(predictors, K)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        dt = t1 - t0
        s0 = time.perf_counter()
        if not args.counters_run:
            pool.run(predictors, S)
        torch.cuda.synchronize()
        ds = time.perf_counter() - s0
        if not args.counters_run:
            # latency under load: every pass of the steady-state run, from the start of its launch to the return of its
            # wait on its serving thread; then the (throughput, latency) pair at one and at two passes queued per thread
            loaded = latency_stats(np, pool.latencies_ms())
            by_depth = {}
            points = [(t, 1) for t in (1, 2, 4) if t < T and NB % t == 0] + [(T, 1), (T, 2)]
            for threads_, depth in points:
                dp = pb.ServePool(threads_, depth)
                dp.run(predictors, 2 * NB)
                torch.cuda.synchronize()
                d0 = time.perf_counter()
                dp.run(predictors, S // 2)
                torch.cuda.synchronize()
                d1 = time.perf_counter()
                st = latency_stats(np, dp.latencies_ms())
                st["samples/s"] = round(cfg.batch * (S // 2) / (d1 - d0), 1)
                by_depth["threads_%d_depth_%d" % (threads_, depth)] = st
                del dp
    else:
        def run_region(first, count):
            start = threading.Barrier(T + 1)
            errors = []

            def worker(t):
                try:
                    start.wait()
                    for i in range(t, count, T):
                        fwd.step(first + i, stream_ptrs[t])
                    streams[t].synchronize()
                except Exception as e:  # noqa: BLE001
                    errors.append(e)

            threads = [threading.Thread(target=worker, args=(t, )) for t in range(T)]
            for th in threads:
                th.start()
            start.wait()
            a = time.perf_counter()
            for th in threads:
                th.join()
            torch.cuda.synchronize()
            b = time.perf_counter()
            if errors:
                raise errors[0]
            return b - a
        run_region(0, warm)
        dt = run_region(warm, K)
        ds = 0.0 if args.counters_run else run_region(warm + K, S)
    if not args.counters_run:
        steady = {"steps": S, "ms_per_step": round(ds * 1e3 / S, 5), "samples/s": round(cfg.batch * S / ds, 1)}
    ms_per_step = dt * 1e3 / K
    samples_per_s = cfg.batch * K / dt

    # ---- latency: one batch at a time on one thread, each step submitted and waited for on its own
    p50, p99, n_lat = latency_ms(np, run_step, K if args.counters_run else max(K, 1000))

    # ---- PCIe-inclusive rate: every step feeds all 79 inputs from pageable host memory and copies the output back
    if not args.no_feed and predictors is not None:
        fT = T
        n_feed = max(fT, min(max(K, 400), 800) // fT * fT)
        fbar = threading.Barrier(fT + 1)
        # one Blaze_PredictorFeedMany call per step (79 inputs); the argument arrays are built once per batch
        feeds = []
        for b in range(NB):
            items = []
            for (fg, _, _), (ids, vals, seg) in zip(fgs, sparse[b]):
                items += [(fg + ".ids", ids), (fg + ".values", vals), (fg + ".segments", seg)]
            items.append(("dense", dense[b].astype(np.float16)))
            feeds.append(predictors[b].feed_batch(items))

        def feed_worker(t):
            for i in range(t, n_feed + 2 * fT, fT):
                if i == t + 2 * fT:
                    fbar.wait()
                b = i % NB
                predictors[b].feed_many(feeds[b])
                predictors[b].forward()
                predictors[b].output_asnumpy("prob")

        ths = [threading.Thread(target=feed_worker, args=(t, )) for t in range(fT)]
        for th in ths:
            th.start()
        fbar.wait()
        f0 = time.perf_counter()
        for th in ths:
            th.join()
        f1 = time.perf_counter()
        in_bytes = float(np.mean([sum(a.nbytes for trip in sparse[b] for a in trip) + dense[b].size * 2 for b in range(NB)]))
        feed_rate = {"samples/s": round(cfg.batch * n_feed / (f1 - f0), 1), "ms_per_step": round((f1 - f0) * 1e3 / n_feed, 4),
                     "host_bytes_per_step": int(in_bytes), "steps": n_feed, "threads": fT,
                     "note": "Feed of every input from pageable host memory + Forward + Output copy, per step"}

    # ---- per-kernel durations
    R = 8 * NB
    kern_us = {"bz_embed_pool_kernel": graph_timed(torch, fwd.pool, NB, R, warm_ms=50.0)}
    for name, launch in fwd.launches():  # the FC launches one step makes (the skinny head rides in the layer before it)
        kern_us[name] = graph_timed(torch, launch, NB, R)
    emb_bytes = float(np.mean([fwd.embedding_bytes(i) for i in range(NB)]))
    flops = fwd.fc_flops()
    pool_us = kern_us["bz_embed_pool_kernel"]
    pool_gbs = emb_bytes / pool_us / 1e3
    fc_us = sum(v for k, v in kern_us.items() if k != "bz_embed_pool_kernel")
    fc_tflops = sum(flops) / fc_us / 1e6
    dominant = max(kern_us, key=kern_us.get)
    if dominant != "bz_embed_pool_kernel":
        layers = [int(x) for x in dominant[6:-1].split("+")] if dominant.startswith("bz_fc[") else list(range(len(flops)))
        roofline = mfma_roofline("%s (FC layers %s)" % (dominant, layers), sum(flops[li] for li in layers), kern_us[dominant])
    else:
        traffic, source = pool_traffic_from_profile() if args.pool == 32 else (None, None)
        roofline = hbm_roofline("bz_embed_pool_kernel", emb_bytes, pool_us, traffic)
        roofline["traffic_source"] = source

    del fwd
    per_config = None
    if not args.no_per_config:
        per_config = {}
        for key, fn in (("c1", lambda: bench_config1(np, torch, bz, pb, T)), ("c3", lambda: bench_config3(np, torch, bz, pb, T)),
                        ("c4", lambda: bench_config4(np, torch, bz)), ("c5", lambda: bench_config5(np, torch, bz))):
            try:
                per_config[key] = fn()
            except Exception as e:  # noqa: BLE001  (one configuration failing must not lose the headline line)
                per_config[key] = {"error": "%s: %s" % (type(e).__name__, e)}
            torch.cuda.empty_cache()

    cpu = None if args.no_cpu_baseline else cpu_baseline(np, cfg, tables, mlp, sparse, dense)

    out = {
        "metric": "samples/sec @batch 2048 fp16 (sparse CTR forward: embedding pool + FC stack)",
        "value": round(samples_per_s, 1),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "warmup_run": warm,
        "ms_per_step": round(ms_per_step, 5),
        "steady_state": steady,
        # latency of a request under the load that `steady_state` is measured at (every pass of that run); without that
        # run (--counters-run, --kernel-api) the unloaded figure
        "p50_ms": loaded["p50_ms"] if loaded else round(p50, 4),
        "p99_ms": loaded["p99_ms"] if loaded else round(p99, 4),
        "latency_samples": loaded["samples"] if loaded else n_lat,
        "latency_at": ("steady_state: %d serving threads, %d pass(es) queued per thread" % (T, args.depth)) if loaded else "one request at a time",
        "latency_by_load": by_depth,
        "latency_unloaded": {"p50_ms": round(p50, 4), "p99_ms": round(p99, 4), "samples": n_lat,
                             "note": "one request at a time on one thread"},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic (Philox4x32-10 keyed by seed, stream, index; Zipf(1.1) ids, Poisson(8) lengths, N(0,0.01) tables, random-init MLP)",
        "config": {"workload": cfg.name, "batch": cfg.batch, "slots": cfg.slots, "table_rows": cfg.rows, "dim": cfg.dim,
                   "batch_pool": NB,
                   "path": "kernel-layer C ABI (bz_*)" if predictors is None else "Predictor.Forward via Blaze_* C ABI",
                   "serving_threads": T, "passes_queued_per_thread": args.depth,
                   "device": arch},
        "roofline": roofline,
        "embedding_pool": {"GB/s": round(pool_gbs, 1), "frac_of_hbm_peak": round(pool_gbs / HBM_PEAK_GBS, 5),
                           "algorithmic_bytes": int(emb_bytes), "us": round(pool_us, 2)},
        "fc_stack": {"TFLOP/s": round(fc_tflops, 2), "frac_of_mfma_peak": round(fc_tflops / MFMA_PEAK_TFLOPS, 5),
                     "flops": int(sum(flops)), "us": round(fc_us, 2)},
        "kernel_us": {k: round(v, 2) for k, v in kern_us.items()},
        "with_host_feed": feed_rate,
        "per_config": per_config,
        "cpu_baseline": cpu,
    }
    if calibration is not None:
        out["counter_calibration"] = calibration
    print(json.dumps(out))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the Blaze sparse CTR inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward pass (Embedding gather/pool -> FC 896-512-256-2 with PReLU -> softmax) over one
synthetic batch of 2048 samples (config 2), inputs already resident in HBM.  A pool of pre-generated
batches is cycled so the id stream is not one cached batch.  By default the step is Predictor.Forward through
the Blaze_* C ABI (the drop-in path), issued by a few serving threads with one Predictor set and HIP stream
each, as the reference is deployed.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "x-deeplearning_amd"))
sys.path.insert(1, os.path.join(ROOT, "oracle"))

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_PEAK_TFLOPS = 2500.0  # dense fp16/bf16
# HBM-side bytes per launch of the pooling kernel on this exact workload (default seed, pool of 32 batches), from two
# rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE; KiB per dispatch, averaged over 1704 dispatches) scaled by what the same
# counters read for a plain 256 MiB copy (`--calibrate-copy`: FETCH_SIZE reads 0.5 of the bytes, WRITE_SIZE all of them):
# fetch 11961.30 KiB x 2.0 + write 3333.59 KiB.  Below the algorithmic bytes because Zipf-hot rows hit in L2.
POOL_TRAFFIC_BYTES = int((11961.30 * 2.0 + 3333.59) * 1024)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--pool", type=int, default=32, help="number of distinct pre-generated batches")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 256 MiB copy (bz_concat_kernel, one piece) a few times and exit: the known-size "
                         "reference for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    ap.add_argument("--gather-probe", action="store_true",
                    help="only measure what the memory system gives random 64-byte row gathers (a kernel that does nothing else, and "
                         "the pooling kernel on uniform ids with 64-id segments) and exit")
    ap.add_argument("--threads", type=int, default=8,
                    help="serving threads, each with its own Predictors and HIP stream (the reference's model: one "
                         "Predictor per thread, blaze/api/cpp_api/predictor.h:90-92)")
    ap.add_argument("--with-feed", action="store_true",
                    help="also time steps that Feed every input from host memory and copy the output back (the "
                         "PCIe-inclusive rate; reported as an extra key, never as `value`)")
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
    from pipeline import CtrForward
    from synth import Config2

    assert torch.cuda.is_available(), "no GPU visible"
    arch = bz.device_check()
    if args.calibrate_copy:
        import ctypes
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
        print(json.dumps({"calibration": "bz_concat_kernel", "launches": 5, "bytes_read_per_launch": rows * width,
                          "bytes_written_per_launch": rows * width}))
        return
    if args.gather_probe:
        def ev_time(fn, reps=20):
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / reps  # us
        g = torch.Generator(device="cuda").manual_seed(1)
        res = {"probe": "random gathers of 64-byte rows", "device": arch}
        # (o) nothing but the access pattern: four-lane groups read hashed 64-byte rows of a 2 GiB region
        region = torch.ones(2 << 30, dtype=torch.uint8, device="cuda")
        sink = torch.empty((1 << 20) * 64, dtype=torch.uint8, device="cuda")
        pure = {}
        for groups, per in ((1 << 20, 8), (1 << 20, 16), (425984, 1), (106496, 4), (53248, 8)):
            seed = [0]
            def launch():
                seed[0] += 7919
                bz.check(bz.lib().bz_probe_gather64(region.data_ptr(), region.numel(), sink.data_ptr(), groups, per, seed[0], None))
            us = ev_time(launch, 50)
            pure["%d groups x %d rows" % (groups, per)] = {"us": round(us, 2), "row_read_GB/s": round(groups * per * 64 / us / 1e3, 1)}
        res["pure_gather_2GiB_region"] = pure
        del region, sink
        # (i) the pooling kernel where the dependent chain of a launch is amortised and no row is hot:
        # config 2's tables (26 x 64 MB), uniform ids, every segment 64 ids long
        cfg = Config2()
        tables = [bz.DeviceTable(t) for t in cfg.tables()]
        L = 64
        out = torch.zeros((cfg.batch, cfg.slots * cfg.dim), dtype=torch.float16, device="cuda")
        items = []
        for s_ in range(cfg.slots):
            ids = torch.randint(0, cfg.rows, (cfg.batch * L, ), device="cuda", generator=g)
            items.append(dict(table=tables[s_], ids=ids, values=torch.ones(cfg.batch * L, device="cuda"),
                              segments=torch.full((cfg.batch, ), L, dtype=torch.int32, device="cuda"), out=out,
                              col=s_ * cfg.dim, udf=bz.SUM))
        plan = bz.EmbeddingPlan(items, fused_scan=True)
        us = ev_time(plan.pool)
        nnz = cfg.slots * cfg.batch * L
        alg = nnz * (64 + 12) + cfg.slots * cfg.batch * 4 + out.numel() * 2
        res["pool_kernel_uniform_ids_64_per_segment"] = {"ids": nnz, "us": round(us, 1),
                                                         "row_read_GB/s": round(nnz * 64 / us / 1e3, 1),
                                                         "algorithmic_GB/s": round(alg / us / 1e3, 1)}
        print(json.dumps(res))
        return
    cfg = Config2()
    tables = cfg.tables()
    mlp = cfg.mlp()
    sparse, dense = cfg.batches(args.pool)
    # kernel-layer harness: per-kernel timing below, and the whole step in --kernel-api mode
    fwd = CtrForward(cfg, tables, mlp, sparse, dense, dtype="f16", fused_mlp=bool(int(os.environ.get("BZ_FUSED_MLP", "0"))))
    torch.cuda.synchronize()
    K, W = args.steps, args.warmup
    T = max(1, min(args.threads, fwd.n_batches))
    assert fwd.n_batches % T == 0, "--pool must be a multiple of --threads (a pooled batch always runs on one thread)"

    predictors = None
    if not args.kernel_api:
        # the drop-in path: one Predictor per pooled batch (inputs fed once = resident in HBM), Forward through
        # the Blaze_* C ABI; consecutive steps go round robin over T serving threads
        from ctr_model import build_manager, make_predictor
        pm, fgs = build_manager(cfg, tables, mlp, np.float16)
        predictors = [make_predictor(pm, fgs, sparse[b], dense[b], np.float16) for b in range(fwd.n_batches)]
        predictors[0].forward()
        ref = fwd.output(0)
        fwd.step(0)
        torch.cuda.synchronize()
        # (the fp16 model's output blob is fp16; the harness keeps the last layer's probabilities in fp32)
        assert np.allclose(predictors[0].output_asnumpy("prob").astype(np.float32), ref.cpu().numpy(), atol=1e-3), \
            "Predictor and kernel-layer harness disagree"

    import ctypes
    import threading
    streams = [torch.cuda.Stream() for _ in range(T)]
    stream_ptrs = [ctypes.c_void_p(st.cuda_stream) for st in streams]

    def run_step(i, t):
        if predictors is not None:
            predictors[i % fwd.n_batches].forward()  # launches on the calling thread's stream and waits for it
        else:
            fwd.step(i, stream_ptrs[t])

    # ---- throughput: W warm-up steps, then exactly K steps between two synchronisations.  The Predictor path is
    # driven by the library's own serving threads (Blaze_ServePool*: a C++ loop per thread, as a serving binary
    # would run it); the kernel-layer path by Python threads.
    if predictors is not None:
        from pyblaze_hip import ServePool
        pool = ServePool(T)
        pool.run(predictors, W)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        pool.run(predictors, K)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    else:
        start = threading.Barrier(T + 1)
        errors = []

        def worker(t):
            try:
                for i in range(t, W, T):
                    run_step(i, t)
                torch.cuda.synchronize()
                start.wait()
                for i in range(t, K, T):
                    run_step(W - (W % T) + i, t)
            except Exception as e:  # noqa: BLE001
                errors.append(e)
                start.abort()

        threads = [threading.Thread(target=worker, args=(t, )) for t in range(T)]
        for th in threads:
            th.start()
        start.wait()
        t0 = time.perf_counter()
        for th in threads:
            th.join()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        if errors:
            raise errors[0]
    ms_per_step = (t1 - t0) * 1e3 / K
    samples_per_s = cfg.batch * K / (t1 - t0)

    # ---- latency: one batch at a time on one thread, each step submitted and waited for on its own
    lat = []
    for i in range(min(K, 2000)):
        a = time.perf_counter()
        run_step(i, 0)
        if predictors is None:
            torch.cuda.synchronize()
        lat.append((time.perf_counter() - a) * 1e3)
    lat = np.sort(np.array(lat))
    p50, p99 = float(lat[len(lat) // 2]), float(lat[int(len(lat) * 0.99)])

    # ---- PCIe-inclusive rate: every step feeds all 79 inputs from pageable host memory and copies the output back
    feed_rate = None
    if args.with_feed and predictors is not None:
        fT = T
        n_feed = max(fT, min(K, 400) // fT * fT)
        fbar = threading.Barrier(fT + 1)

        # one Blaze_PredictorFeedMany call per step (79 inputs); the argument arrays are built once per batch
        feeds = []
        for b in range(fwd.n_batches):
            items = []
            for (fg, _, _), (ids, vals, seg) in zip(fgs, sparse[b]):
                items += [(fg + ".ids", ids), (fg + ".values", vals), (fg + ".segments", seg)]
            items.append(("dense", dense[b].astype(np.float16)))
            feeds.append(predictors[b].feed_batch(items))

        def feed_worker(t):
            for i in range(t, n_feed + 2 * fT, fT):
                if i == t + 2 * fT:
                    fbar.wait()
                b = i % fwd.n_batches
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
        in_bytes = float(np.mean([sum(a.nbytes for trip in sparse[b] for a in trip) + dense[b].size * 2
                                  for b in range(fwd.n_batches)]))
        feed_rate = {"samples/s": round(cfg.batch * n_feed / (f1 - f0), 1), "ms_per_step": round((f1 - f0) * 1e3 / n_feed, 4),
                     "host_bytes_per_step": int(in_bytes), "steps": n_feed, "threads": fT,
                     "note": "Feed of every input from pageable host memory + Forward + Output copy, per step"}

    # ---- per-kernel durations: HIP events on the launch stream around a replayed HIP graph that holds
    # R back-to-back launches of the one kernel (over the pooled batches), so host launch cost is not in it
    def timed(fn, reps):
        for i in range(fwd.n_batches):
            fn(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(reps):
                fn(i)
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        rounds = 5
        e0.record()
        for _ in range(rounds):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * rounds)  # us

    R = 8 * fwd.n_batches
    kern_us = {"bz_embed_pool_kernel": timed(fwd.pool, R)}
    for name, launch in fwd.launches():  # the FC launches one step makes (the skinny head rides in the layer before it)
        kern_us[name] = timed(launch, R)
    emb_bytes = float(np.mean([fwd.embedding_bytes(i) for i in range(fwd.n_batches)]))
    flops = fwd.fc_flops()
    pool_us = kern_us["bz_embed_pool_kernel"]
    pool_gbs = emb_bytes / pool_us / 1e3
    fc_us = sum(v for k, v in kern_us.items() if k != "bz_embed_pool_kernel")
    fc_tflops = sum(flops) / fc_us / 1e6
    dominant = max(kern_us, key=kern_us.get)
    if dominant != "bz_embed_pool_kernel":
        layers = [int(x) for x in dominant[6:-1].split("+")] if dominant.startswith("bz_fc[") else list(range(len(flops)))
        ach = sum(flops[li] for li in layers) / kern_us[dominant] / 1e6
        roofline = {"kernel": "%s (FC layers %s)" % (dominant, layers), "bound": "mfma", "achieved": round(ach, 2),
                    "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / MFMA_PEAK_TFLOPS, 5), "traffic": None}
    else:
        roofline = {"kernel": "bz_embed_pool_kernel", "bound": "hbm", "achieved": round(pool_gbs, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(pool_gbs / HBM_PEAK_GBS, 5),
                    "traffic": POOL_TRAFFIC_BYTES if args.pool == 32 else None,
                    "algorithmic_bytes_per_launch": int(emb_bytes), "avg_launch_us": round(pool_us, 2)}

    # ---- CPU baseline: the oracle (a port of the reference's CPU path), one single-threaded predictor per thread.
    # The products go to the optimised sgemm numpy links, as the reference's go to MKL's cblas_sgemm.
    cpu = None
    if not args.no_cpu_baseline:
        import blaze_oracle as orc
        from pipeline import oracle_forward
        from threadpoolctl import threadpool_info, threadpool_limits
        orc.build()
        tabs = [orc.Table(t.cpu().numpy()) for t in tables]
        mlp_np = [(w.cpu().numpy(), b.cpu().numpy(), s.cpu().numpy()) for (w, b, s) in mlp]
        threads = max(1, min(16, len(os.sched_getaffinity(0))))
        per_thread = 8
        blas = next(("%s %s (%s)" % (i.get("internal_api"), i.get("version"), i.get("architecture"))
                     for i in threadpool_info() if i.get("user_api") == "blas"), "numpy's matmul")
        def worker(t):
            for j in range(per_thread):
                b = (t * per_thread + j) % len(sparse)
                oracle_forward(orc, cfg, tabs, mlp_np, sparse[b], dense[b], blas=True)
        with threadpool_limits(1, user_api="blas"):
            oracle_forward(orc, cfg, tabs, mlp_np, sparse[0], dense[0], blas=True)  # warm the page cache of the tables
            c0 = time.perf_counter()
            ths = [threading.Thread(target=worker, args=(t, )) for t in range(threads)]
            for t in ths:
                t.start()
            for t in ths:
                t.join()
            c1 = time.perf_counter()
            s0 = time.perf_counter()  # ... and the same port on one core alone
            for j in range(per_thread):
                oracle_forward(orc, cfg, tabs, mlp_np, sparse[j % len(sparse)], dense[j % len(sparse)], blas=True)
            s1 = time.perf_counter()
        t0 = time.perf_counter()  # one batch with the oracle's own k-ascending sgemm, for the record
        oracle_forward(orc, cfg, tabs, mlp_np, sparse[0], dense[0])
        t1 = time.perf_counter()
        model = ""
        try:
            with open("/proc/cpuinfo") as f:
                model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), "")
        except OSError:
            pass
        cpu = {"value": round(cfg.batch * threads * per_thread / (c1 - c0), 1), "unit": "samples/s", "cores": threads,
               "kind": "port", "value_1_core": round(cfg.batch * per_thread / (s1 - s0), 1),
               "value_1_core_textbook_sgemm": round(cfg.batch / (t1 - t0), 1), "sgemm": blas,
               "host_cpus": os.cpu_count(), "cpu_model": model,
               "sample": "%d batches of %d (%d per thread, one single-threaded predictor per core), fp32 oracle: "
                         "hash-free row lookup, ksum, sgemm of the BLAS numpy links on one thread + separate PReLU pass, "
                         "softmax" % (threads * per_thread, cfg.batch, per_thread)}

    out = {
        "metric": "samples/sec @batch 2048 fp16 (sparse CTR forward: embedding pool + FC stack)",
        "value": round(samples_per_s, 1),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 5),
        "p50_ms": round(p50, 4),
        "p99_ms": round(p99, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic (seeded; Zipf(1.1) ids, Poisson(8) lengths, N(0,0.01) tables, random-init MLP)",
        "config": {"workload": cfg.name, "batch": cfg.batch, "slots": cfg.slots, "table_rows": cfg.rows, "dim": cfg.dim,
                   "batch_pool": fwd.n_batches,
                   "path": "kernel-layer C ABI (bz_*)" if predictors is None else "Predictor.Forward via Blaze_* C ABI",
                   "serving_threads": T,
                   "device": arch},
        "roofline": roofline,
        "embedding_pool": {"GB/s": round(pool_gbs, 1), "frac_of_hbm_peak": round(pool_gbs / HBM_PEAK_GBS, 5),
                           "algorithmic_bytes": int(emb_bytes), "us": round(pool_us, 2)},
        "fc_stack": {"TFLOP/s": round(fc_tflops, 2), "frac_of_mfma_peak": round(fc_tflops / MFMA_PEAK_TFLOPS, 5),
                     "flops": int(sum(flops)), "us": round(fc_us, 2)},
        "kernel_us": {k: round(v, 2) for k, v in kern_us.items()},
        "cpu_baseline": cpu,
    }
    if feed_rate is not None:
        out["with_host_feed"] = feed_rate
    print(json.dumps(out))


if __name__ == "__main__":
    main()

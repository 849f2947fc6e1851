"""GPU tests of the drop-in boundary: operators run through Predictor / the Blaze_* C ABI.

The reference's operator tests build a net from a text NetDef whose inputs are ConstantFill ops, run it and compare
outputs with |d| <= 1e-6 (test/operator/operator_test_common.h:20-84).  The same is done here from the same data
(tests/golden/reference_kats.json), through Blaze_PredictorManagerLoadModelFromString / Blaze_PredictorCreate /
Blaze_PredictorForward / Blaze_PredictorOutput on device_type 1.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def pb():
    import torch
    import blaze_hip
    import pyblaze_hip
    assert torch.cuda.is_available(), "no GPU visible"
    blaze_hip.device_check()
    return pyblaze_hip


def _np_dtype(code):
    return {1: np.float32, 2: np.int32, 10: np.int64, 12: np.float16}[code]


def _net_from_kat(pb, case, skip_types=()):
    nb = pb.NetBuilder("kat", device_type=1)
    for name, t in case["tensors"].items():
        nb.constant(name, np.array(t["values"], _np_dtype(t["dtype"])).reshape(t["shape"]), dtype=t["dtype"])
    for op in case["ops"]:
        args = {}
        for k, v in op["args"].items():
            if k in ("store_name", "store_type", "store_url"):
                continue
            if k in ("alpha", "beta"):
                v = float(v)
            args[k] = v
        nb.op(op["type"], op["inputs"], op["outputs"], **args)
    for name, e in case["expected"].items():
        nb.external_output(name, e["dtype"])
    return nb.text()


DENSE = ["gemm_net_v1_cpu", "prelu_net_v1_cpu", "dice_net_v1_cpu", "leaky_relu_net_v1_cpu", "sigmoid_net_v1_cpu",
         "softmax_net_v1_cpu", "matmul_net_v1_cpu", "fused_parallel_gemm_net_v1_cpu", "fused_parallel_gemm_net_v2_cpu",
         "fused_parallel_gemm_net_v3_cpu", "fused_parallel_gemm_net_v4_cpu", "fused_parallel_gemm_net_v5_cpu",
         "fused_parallel_matmul_net_v1_cpu", "fused_parallel_matmul_net_v2_cpu", "fused_parallel_matmul_net_v3_cpu",
         "concat_net_v1_cpu", "concat_net_v2_cpu", "reduce_sum_net_v1_cpu", "fuse_net_v1_cpu", "fuse_net_v2_cpu",
         "reshape_net_v1_cpu", "batch_normalization_net_v1_cpu", "elementwise_add_net_v1_cpu", "elementwise_add_net_v2_cpu",
         "elementwise_sub_net_v1_cpu", "elementwise_sub_net_v2_cpu", "elementwise_mul_net_v1_cpu", "elementwise_mul_net_v2_cpu",
         "elementwise_div_net_v1_cpu", "elementwise_div_net_v2_cpu", "elementwise_broadcast_to_net_v1_cpu",
         "elementwise_broadcast_to_net_v2_cpu", "elementwise_where_net_v1_cpu", "split_net_v1_cpu", "split_net_v2_cpu",
         "gather_net_v1_cpu", "gather_net_v2_cpu", "slice_net_v1_cpu"]


@pytest.mark.parametrize("name", DENSE)
def test_reference_operator_kats_through_predictor(pb, kats, name):
    case = kats[name]
    pm = pb.PredictorManager()
    pm.load_model_from_string(_net_from_kat(pb, case), True)
    p = pm.create_predictor(1, 0)
    print("case", name, flush=True)
    p.register_observers(["profile"])
    p.forward()
    for out_name, e in case["expected"].items():
        got = p.output_asnumpy(out_name)
        assert list(got.shape) == e["shape"]
        np.testing.assert_allclose(got, np.array(e["values"], np.float32).reshape(e["shape"]), rtol=0, atol=1e-6)
    if name.startswith("fused_parallel_gemm"):
        # the parallel_num sibling FCs go out as one launch (the reference: one GemmStridedBatched, fused_parallel_gemm_op.h:115-129)
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["name"].startswith("FusedParallelGemm")]
        assert len(ev) == 1 and ev[0]["args"]["launches"] == 1, ev


def test_reference_embedding_kat_through_predictor(pb, kats):
    """embedding_v1.conf: the reference runs it over its mock puller (every key -> a row of ones); here the device
    store gets tables of ones keyed by every id of the fixture."""
    case = kats["embedding_v1"]
    pm = pb.PredictorManager()
    for fg, table, dim in (("101", "a_01", 4), ("102", "a_02", 8), ("104_7", "a_03", 6)):
        ids = np.unique(np.array(case["tensors"][fg + ".ids"]["values"], np.int64))
        pm.add_table(table, np.ones((ids.size, dim), np.float32), keys=ids)
    pm.load_model_from_string(_net_from_kat(pb, case), True)
    p = pm.create_predictor(1, 0)
    p.forward()
    for out_name, e in case["expected"].items():
        got = p.output_asnumpy(out_name)
        assert list(got.shape) == e["shape"] and got.dtype == np.float32
        np.testing.assert_allclose(got, np.array(e["values"], np.float32).reshape(e["shape"]), rtol=0, atol=1e-6)


def _write_csv(path, keys, rows):
    with open(path, "w") as f:
        for k, r in zip(keys, rows):
            f.write(",".join([str(int(k))] + [repr(float(x)) for x in r]) + "\n")


def _ctr_text(pb, fgs, blocks, dims_in, layers, acts, dtype, fuse, dense_name="dense"):
    """Embedding -> Concat(dense, block) -> [Gemm + activation]* ; returns (text, weights)."""
    code = pb.K_FLOAT16 if dtype == np.float16 else pb.K_FLOAT
    nb = pb.NetBuilder("ctr", device_type=1)
    inputs = []
    for fg, _, _ in fgs:
        nb.external_input(fg + ".ids", pb.K_INT64)
        nb.external_input(fg + ".values", pb.K_FLOAT)
        nb.external_input(fg + ".segments", pb.K_INT32)
        inputs += [fg + ".ids", fg + ".values", fg + ".segments"]
    nb.external_input(dense_name, code)
    nb.external_output("prob", code)
    nb.arg("fuse_gemm_activation", int(fuse))
    rng = np.random.default_rng(77)
    weights = []
    for li in range(len(layers) - 1):
        k, n = layers[li], layers[li + 1]
        w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32)
        b = (rng.standard_normal(n) * 0.1).astype(np.float32)
        extra = ()
        if acts[li] == "PRelu":
            extra = (rng.uniform(0.1, 0.4, n).astype(np.float32), )
        elif acts[li] == "Dice":
            extra = ((rng.standard_normal(n) * 0.1).astype(np.float32), (rng.standard_normal(n) * 0.1).astype(np.float32),
                     rng.uniform(0.5, 1.5, n).astype(np.float32))
        weights.append((w, b, extra))
        nb.constant("w%d" % li, w, dtype=code)
        nb.constant("b%d" % li, b, dtype=code)
        for j, e in enumerate(extra):
            nb.constant("p%d_%d" % (li, j), e, dtype=code)
    nb.op("Embedding", inputs, ["block"], embedding_config=pb.embedding_config_text(fgs, blocks),
          **({"out_dtype": code} if dtype == np.float16 else {}))
    nb.op("Concat", [dense_name, "block"], ["x0"], axis=1)
    for li in range(len(layers) - 1):
        last = li == len(layers) - 2
        nb.op("Gemm", ["x%d" % li, "w%d" % li, "b%d" % li], ["h%d" % li])
        out = "prob" if last else "x%d" % (li + 1)
        if acts[li] == "Softmax":
            nb.op("Softmax", ["h%d" % li], [out], axis=1)
        elif acts[li] == "LeakyRelu":
            nb.op("LeakyRelu", ["h%d" % li], [out], alpha=0.0)
        elif acts[li] == "Sigmoid":
            nb.op("Sigmoid", ["h%d" % li], [out])
        else:
            nb.op(acts[li], ["h%d" % li] + ["p%d_%d" % (li, j) for j in range(len(weights[li][2]))], [out])
    return nb.text(), weights


def _oracle_ctr(oracle, tables, fgs, blocks, inputs, dense, weights, acts, r):
    """The same net on the CPU oracle; r rounds to the model's storage type after every op (identity for fp32)."""
    outs = oracle.embedding_op({fg: (t, d) for fg, t, d in fgs}, blocks, inputs, tables)
    h = np.concatenate([r(dense), r(outs[0])], axis=1)
    for (w, b, extra), act in zip(weights, acts):
        y = r(oracle.gemm_op(h, r(w), r(b)))
        if act == "PRelu":
            y = oracle.prelu(y, r(extra[0]))
        elif act == "Dice":
            y = oracle.dice(y, *[r(e) for e in extra])
        elif act == "LeakyRelu":
            y = oracle.leaky_relu(y, 0.0)
        elif act == "Sigmoid":
            y = oracle.sigmoid(y)
        else:
            y = oracle.softmax(y, 1)
        h = r(y)
    return h


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("acts", [("PRelu", "Dice", "Softmax"), ("LeakyRelu", "Sigmoid", "Softmax")])
def test_ctr_model_from_qed_file_fused_and_unfused(pb, oracle, tmp_path, dtype, acts):
    """Text tables -> Blaze_QuickEmbeddingBuild* -> Blaze_LoadSparseModelWeight -> Embedding + Concat + FC stack.
    With and without folding the activations into the Gemm epilogue; both against the oracle."""
    rng = np.random.default_rng(5)
    fgs = [("101", "t_a", 8), ("102", "t_b", 16), ("103", "t_c", 8)]
    blocks = [[dict(fg="101", udf=0), dict(fg="102", udf=1), dict(fg="103", udf=0)]]
    tabs, oracle_tabs = {}, {}
    for _, tname, dim in fgs:
        n = int(rng.integers(30, 120))
        keys = np.unique(rng.integers(-2**40, 2**40, n * 2, dtype=np.int64))[:n]
        rows = (rng.standard_normal((n, dim)) * 0.5).astype(np.float32)
        _write_csv(tmp_path / tname, keys, rows)
        tabs[tname] = (keys, rows)
    open(tmp_path / "meta", "w").write("".join(t + "\n" for _, t, _ in fgs))
    qed = str(tmp_path / "model.qed")
    pb.build_qed(str(tmp_path), "meta", qed, fp16=(dtype == np.float16))
    for tname, (keys, rows) in tabs.items():
        # what the builder parsed back from text (repr round-trips fp32 exactly), narrowed for the fp16 file
        oracle_tabs[tname] = oracle.Table(rows.astype(np.float16) if dtype == np.float16 else rows, keys=keys)
    batch, dense_dim = 37, 5
    layers = (dense_dim + 32, 24, 16, 2)
    inputs = {}
    for fg, tname, _ in fgs:
        seg = rng.integers(0, 6, batch).astype(np.int32)
        pool = np.concatenate([tabs[tname][0], rng.integers(-2**40, 2**40, 10, dtype=np.int64)])
        ids = rng.choice(pool, int(seg.sum()))
        inputs[fg] = (ids.astype(np.int64), rng.standard_normal(ids.size).astype(np.float32), seg)
    dense = rng.standard_normal((batch, dense_dim)).astype(np.float32)
    r = (lambda x: np.asarray(x, np.float32).astype(np.float16).astype(np.float32)) if dtype == np.float16 else (lambda x: x)
    results = []
    for fuse in (True, False):
        text, weights = _ctr_text(pb, fgs, blocks, dense_dim, layers, acts, dtype, fuse)
        pm = pb.PredictorManager()
        pm.load_sparse_model_weight(qed)
        pm.load_model_from_string(text, True)
        p = pm.create_predictor(1, 0)
        assert p.list_input_names() == [n for fg, _, _ in fgs for n in (fg + ".ids", fg + ".values", fg + ".segments")] + ["dense"]
        assert p.list_output_names() == ["prob"]
        for fg, (ids, vals, seg) in inputs.items():
            p.feed(fg + ".ids", ids)
            p.feed(fg + ".values", vals)
            p.feed(fg + ".segments", seg)
        p.feed("dense", dense.astype(dtype))
        print("case dtype=%s acts=%s fuse=%s" % (dtype.__name__, acts, fuse), flush=True)
        p.forward()
        got = p.output_asnumpy("prob")
        assert got.shape == (batch, 2) and got.dtype == dtype
        results.append(got.astype(np.float32))
        p.forward()  # a second run reuses cached descriptors and packed weights
        assert np.array_equal(p.output_asnumpy("prob").astype(np.float32), results[-1])
    want = _oracle_ctr(oracle, oracle_tabs, fgs, blocks, inputs, dense, weights, acts, r)
    tol = 2e-3 if dtype == np.float16 else 1e-5
    for got in results:
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol)
    np.testing.assert_allclose(results[0], results[1], rtol=tol, atol=tol)
    names = p.list_internal_names()
    assert "w0" in names and p.internal_shape("w0") == (layers[0], layers[1])
    np.testing.assert_array_equal(p.internal_asnumpy("w0"), weights[0][0].astype(dtype))


def test_feed_and_forward_error_conventions(pb):
    pm = pb.PredictorManager()
    nb = pb.NetBuilder("err", device_type=1)
    nb.external_input("x", pb.K_FLOAT)
    nb.external_output("y")
    nb.constant("w", np.ones((4, 3), np.float32))
    nb.op("Gemm", ["x", "w"], ["y"])
    pm.load_model_from_string(nb.text(), True)
    p = pm.create_predictor(1, 0)
    x = np.ones((2, 4), np.float32)
    p.reshape_input("x", x.shape)
    with pytest.raises(pb.BlazeError, match="Feed x failed"):
        p.feed_raw("x", x, x.nbytes - 4)  # len must equal size * sizeof(dtype)
    with pytest.raises(pb.BlazeError, match="Feed nope failed"):
        p.feed_raw("nope", x, x.nbytes)
    p.feed("x", x)
    p.forward()
    np.testing.assert_array_equal(p.output_asnumpy("y"), np.full((2, 3), 4, np.float32))
    p.feed("x", np.ones((2, 5), np.float32))  # inner dimension no longer matches the weight
    with pytest.raises(pb.BlazeError, match="Forward failed.*a_k=5 b_k=4"):
        p.forward()
    p.feed("x", x)  # the predictor stays usable after a failed run
    p.forward()
    np.testing.assert_array_equal(p.output_asnumpy("y"), np.full((2, 3), 4, np.float32))
    p.register_observers(["profile"])
    p.forward()
    trace = json.loads(p.dump_observers()["profile"])
    assert [e["name"].split(":")[0] for e in trace["traceEvents"]] == ["ConstantFill", "Gemm"]


def test_embedding_operator_errors(pb):
    cfg = pb.embedding_config_text([("101", "t", 4)], [[dict(fg="101", udf=0)]])

    def build(cfg_text, store=True, inputs=("101.ids", "101.values", "101.segments")):
        pm = pb.PredictorManager()
        if store:
            pm.add_table("t", np.ones((3, 4), np.float32))
        nb = pb.NetBuilder("e", device_type=1)
        for n, dt in zip(inputs, (pb.K_INT64, pb.K_FLOAT, pb.K_INT32)):
            nb.external_input(n, dt)
        nb.external_output("block")
        nb.op("Embedding", list(inputs), ["block"], embedding_config=cfg_text)
        pm.load_model_from_string(nb.text(), True)
        return pm

    with pytest.raises(pb.BlazeError, match="Parse embedding config failed"):
        build("feature_group_config { feature_group : ").create_predictor(1, 0)
    with pytest.raises(pb.BlazeError, match="feature group config not exist"):
        build(pb.embedding_config_text([("101", "t", 4)], [[dict(fg="999", udf=0)]])).create_predictor(1, 0)
    with pytest.raises(pb.BlazeError, match="id input name"):
        build(cfg, inputs=("101.ids", "102.values", "101.segments")).create_predictor(1, 0)
    p = build(cfg, store=False).create_predictor(1, 0)
    p.feed("101.ids", np.array([0, 1], np.int64))
    p.feed("101.values", np.ones(2, np.float32))
    p.feed("101.segments", np.array([2], np.int32))
    with pytest.raises(pb.BlazeError, match="no sparse puller"):
        p.forward()
    p = build(cfg).create_predictor(1, 0)
    p.feed("101.ids", np.array([0, 1], np.int64))
    p.feed("101.values", np.ones(3, np.float32))  # ids / values disagree
    p.feed("101.segments", np.array([2], np.int32))
    with pytest.raises(pb.BlazeError, match="id_blob->size"):
        p.forward()
    p.feed("101.values", np.array([2.0, 3.0], np.float32))
    p.forward()
    np.testing.assert_array_equal(p.output_asnumpy("block"), np.full((1, 4), 5.0, np.float32))
    # unknown table name: the block stays zero
    p = build(pb.embedding_config_text([("101", "unknown_table", 4)], [[dict(fg="101", udf=0)]])).create_predictor(1, 0)
    p.feed("101.ids", np.array([0, 1], np.int64))
    p.feed("101.values", np.ones(2, np.float32))
    p.feed("101.segments", np.array([2], np.int32))
    p.forward()
    assert not p.output_asnumpy("block").any()


def test_concat_inputs_written_in_place_give_identical_results(pb):
    """Concat(dense, block) whose inputs are an external input and an Embedding block read by nothing else: both
    live inside the Concat's output (the Feed copies rows at that tensor's pitch, the pooling kernel writes at it)
    and nothing is copied.  Bit-identical to the net with the aliasing switched off, also after the batch size and
    the fed data change."""
    import torch
    from ctr_model import build_manager, feed_inputs
    from synth import Config2
    cfg = Config2(batch=257, rows=3000, slots=26)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(2)
    small = Config2(batch=64, rows=3000, slots=26)
    sparse_s, dense_s = small.batches(1, seed_offset=9)
    outs = {}
    for alias in (1, 0):
        pm, fgs = build_manager(cfg, tables, mlp, np.float16, net_args={"alias_concat_inputs": alias})
        p = pm.create_predictor(1, 0)
        got = []
        for sp, dn in ((sparse[0], dense[0]), (sparse_s[0], dense_s[0]), (sparse[1], dense[1])):  # batch 257 -> 64 -> 257
            feed_inputs(p, fgs, sp, dn, np.float16)
            p.forward()
            got.append(p.output_asnumpy("prob").copy())
        outs[alias] = got
        if alias:
            with pytest.raises(pb.BlazeError):
                p.input_device_ptr("dense")  # a strided input has no plain buffer to hand out
        else:
            assert p.input_device_ptr("dense")
    torch.cuda.synchronize()
    for a, b in zip(outs[1], outs[0]):
        assert a.shape == b.shape and np.array_equal(a.view(np.uint16), b.view(np.uint16))
    assert outs[1][0].shape == (257, 2) and outs[1][1].shape == (64, 2)


def test_forward_in_two_halves_and_serve_pool_match_plain_forward(pb):
    """ForwardLaunch / ForwardWait keep two predictors of one thread queued at once, and the serving pool does the
    same inside the library (depth 2) or calls plain Forward (depth 1): every predictor ends with bit-identical
    probabilities to its own synchronous Forward.  ForwardWait without a launch is an error, not a hang."""
    import torch
    from ctr_model import build_manager, make_predictor
    from synth import Config2
    cfg = Config2(batch=200, rows=3000, slots=26)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(4)
    pm, fgs = build_manager(cfg, tables, mlp, np.float16)
    preds = [make_predictor(pm, fgs, sparse[b], dense[b], np.float16) for b in range(4)]
    want = []
    for p in preds:
        p.forward()
        want.append(p.output_asnumpy("prob").copy())
    assert not np.array_equal(want[0], want[1])  # different batches: a mixed-up predictor would show

    with pytest.raises(pb.BlazeError, match="ForwardWait without a ForwardLaunch"):
        preds[0].forward_wait()
    preds[0].forward_launch()
    preds[1].forward_launch()
    preds[0].forward_wait()
    preds[1].forward_wait()
    preds[2].forward_launch()
    preds[2].forward()  # a launch nobody waited for is waited for by the next Forward
    for b in range(3):
        np.testing.assert_array_equal(preds[b].output_asnumpy("prob"), want[b])

    for threads, depth, steps in ((2, 1, 13), (2, 2, 13), (1, 4, 9), (4, 2, 6), (2, 2, 1), (2, 2, 0)):
        print("serve pool threads=%d depth=%d steps=%d" % (threads, depth, steps), flush=True)
        pool = pb.ServePool(threads, depth)
        pool.run(preds, steps)
        torch.cuda.synchronize()
        for b in range(4):
            np.testing.assert_array_equal(preds[b].output_asnumpy("prob"), want[b])
        # one latency per pass of the job (launch to the return of its wait), positive and well under a second
        lat = pool.latencies_ms()
        assert lat.shape == (steps, ) and (steps == 0 or (lat.min() > 0 and lat.max() < 1000.0)), lat
        del pool
    with pytest.raises(pb.BlazeError, match="multiple of the pool's threads"):
        pb.ServePool(3).run(preds, 4)
    # the serving threads (and their streams) are gone; destroying predictors whose last passes ran on those streams
    # must not leave a runtime error behind for the caller's next GPU call
    import gc
    preds[0].forward_launch()  # one pass still in flight at destruction, on this thread's stream
    del preds, p
    gc.collect()
    assert float(torch.ones(4, device="cuda").sum()) == 4.0
    torch.cuda.synchronize()


def test_serve_pool_spreads_its_streams_evenly_over_the_hardware_queues(pb):
    """The pool creates its threads' streams and measures which of them share a hardware queue: every queue it saw
    serves as many threads as any other, give or take one, whatever streams the process holds besides (some idle ones
    are created first), and neighbouring threads sit on different queues.  Results are the plain Forward's."""
    import collections
    import torch
    from ctr_model import build_manager, make_predictor
    from synth import Config2
    cfg = Config2(batch=64, rows=500, slots=26)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(8)
    pm, fgs = build_manager(cfg, tables, mlp, np.float16)
    preds = [make_predictor(pm, fgs, sparse[b], dense[b], np.float16) for b in range(8)]
    want = []
    for p in preds:
        p.forward()
        want.append(p.output_asnumpy("prob").copy())
    idle = [torch.cuda.Stream() for _ in range(3)]  # streams of the process that serve nothing
    for st in idle:
        with torch.cuda.stream(st):
            torch.zeros(1, device="cuda")
    torch.cuda.synchronize()
    for threads in (8, 4, 2, 1):
        pool = pb.ServePool(threads, 1)
        assert pool.stream_queues() == []
        pool.run(preds, 16)
        q = pool.stream_queues()
        print("threads", threads, "queues", q, flush=True)
        assert len(q) == threads
        per_queue = collections.Counter(q)
        assert max(per_queue.values()) - min(per_queue.values()) <= 1, q
        assert len(per_queue) >= min(threads, 2), q  # (the runtime's default is 4 queues)
        if threads > 1 and len(per_queue) > 1:
            assert all(q[t] != q[t + 1] for t in range(threads - 1)), q
        pool.run(preds, 8)
        assert pool.stream_queues() == q  # measured once
        for b in range(8):
            np.testing.assert_array_equal(preds[b].output_asnumpy("prob"), want[b])
        del pool


def test_skinny_last_layer_rides_in_the_launch_before_it(pb, oracle):
    """Gemm+PRelu (512 -> 256) followed by Gemm+Softmax (256 -> 2): by default the second runs inside the first one's
    launch (bz_fc_desc.head_*) and the 256-wide tensor between them is never stored; fuse_fc_head: 0 runs them one by
    one.  Same probabilities to 2e-3 (the fused tile sums in another order), also after the batch size changes."""
    import torch
    from ctr_model import build_manager, feed_inputs
    from synth import Config2
    cfg = Config2(batch=300, rows=4000, slots=26)
    small = Config2(batch=33, rows=4000, slots=26)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(2)
    sparse_s, dense_s = small.batches(1, seed_offset=4)
    probs = {}
    for fuse in (1, 0):
        pm, fgs = build_manager(cfg, tables, mlp, np.float16, net_args={"fuse_fc_head": fuse})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for sp, dn in ((sparse[0], dense[0]), (sparse_s[0], dense_s[0]), (sparse[1], dense[1])):
            feed_inputs(p, fgs, sp, dn, np.float16)
            p.forward()
            got.append(p.output_asnumpy("prob").astype(np.float32))
        ran = [e["name"].split(":")[0] for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        assert ran.count("Gemm") == (2 if fuse else 3), ran
        probs[fuse] = got
    torch.cuda.synchronize()
    for a, b, n in zip(probs[1], probs[0], (300, 33, 300)):
        assert a.shape == (n, 2)
        np.testing.assert_allclose(a, b, rtol=2e-3, atol=2e-3)
        np.testing.assert_allclose(a.sum(1), 1.0, rtol=2e-3)
    assert not np.array_equal(probs[1][0], probs[1][2])


def test_embedding_operator_scans_first_when_the_batch_is_large(pb):
    """A batch so large that every workgroup of the pooling kernel would re-read tens of thousands of counts: the
    puller follows the planner's advice, scans the segments in a launch of their own and pools from the offsets.
    Bit-identical block to the one-launch form of the kernel layer."""
    import torch
    import blaze_hip as bz
    from ctr_model import build_manager, make_predictor
    from synth import Config2
    cfg = Config2(batch=70000, rows=5000, slots=2)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(1)
    pm, fgs = build_manager(cfg, tables, mlp, np.float16, expose_block=True)
    p = make_predictor(pm, fgs, sparse[0], dense[0], np.float16)
    p.forward()
    got = p.output_asnumpy("block")
    out = torch.zeros((cfg.batch, cfg.slots * cfg.dim), dtype=torch.float16, device="cuda")
    items, keep = [], []
    for s, (ids, vals, seg) in enumerate(sparse[0]):
        t = [torch.from_numpy(x).cuda() for x in (ids, vals, seg)]
        keep.append(t)
        items.append(dict(table=bz.DeviceTable(tables[s]), ids=t[0], values=t[1], segments=t[2], out=out, col=s * cfg.dim, udf=bz.SUM))
    auto = bz.EmbeddingPlan(items)
    assert auto.launch.fused_scan == 0  # the same advice the puller received
    bz.EmbeddingPlan(items, fused_scan=True).run()
    torch.cuda.synchronize()
    assert got.shape == (cfg.batch, cfg.slots * cfg.dim) and got.any()
    assert np.array_equal(got.view(np.uint16), out.cpu().numpy().view(np.uint16))
    assert p.output_asnumpy("prob").shape == (cfg.batch, 2)


def test_feed_many_equals_feeding_one_by_one(pb):
    """Blaze_PredictorFeedMany: all inputs in one call, the plain device inputs in one transfer through an arena the
    input tensors then view.  Same probabilities as feeding one by one -- after the first call, after the batch grows
    (the arena is outgrown), after it shrinks, and when single Feed calls follow on the re-viewed tensors; a wrong
    length is refused with the reference's message."""
    from ctr_model import build_manager, feed_inputs
    from synth import Config2

    def items_of(fgs, sp, dn):
        items = []
        for (fg, _, _), (ids, vals, seg) in zip(fgs, sp):
            items += [(fg + ".ids", ids), (fg + ".values", vals), (fg + ".segments", seg)]
        return items + [("dense", dn.astype(np.float16))]

    base = Config2(batch=64, rows=3000, slots=26)
    tables, mlp = base.tables(), base.mlp()
    pm, fgs = build_manager(base, tables, mlp, np.float16)
    one, many = pm.create_predictor(1, 0), pm.create_predictor(1, 0)
    for batch, seed in ((64, 0), (300, 3), (17, 5), (300, 7)):
        cfg = Config2(batch=batch, rows=3000, slots=26)
        sparse, dense = cfg.batches(1, seed_offset=seed)
        feed_inputs(one, fgs, sparse[0], dense[0], np.float16)
        one.forward()
        want = one.output_asnumpy("prob").copy()
        items = items_of(fgs, sparse[0], dense[0])
        for name, a in items:
            many.reshape_input(name, a.shape)
        fb = many.feed_batch(items)
        for _ in range(2):  # the second call finds the tensors already viewing the arena
            many.feed_many(fb)
            many.forward()
            np.testing.assert_array_equal(many.output_asnumpy("prob"), want)
    # single feeds on tensors that view the arena
    sparse, dense = Config2(batch=300, rows=3000, slots=26).batches(1, seed_offset=11)
    feed_inputs(one, fgs, sparse[0], dense[0], np.float16)
    one.forward()
    many.feed("fg00.values", sparse[0][0][1])          # same shape as before: reshape + Feed
    for name, a in items_of(fgs, sparse[0], dense[0]):
        many.feed(name, a)
    many.forward()
    np.testing.assert_array_equal(many.output_asnumpy("prob"), one.output_asnumpy("prob"))
    bad = many.feed_batch([("fg00.segments", np.zeros(7, np.int32))])
    with pytest.raises(pb.BlazeError, match="FeedMany failed"):
        many.feed_many(bad)


def test_threads_feeding_alternating_requests_get_their_own_results(pb):
    """Four serving threads, a predictor each, every step another request (two request sizes alternate, so the feed
    arena's layout, the tensors' addresses and the pooling kernel's slot records change every step) through
    FeedMany + Forward + Output: every result equals the one computed for that request alone."""
    import threading
    from ctr_model import build_manager, feed_inputs
    from synth import Config2
    base = Config2(batch=128, rows=3000, slots=26)
    tables, mlp = base.tables(), base.mlp()
    pm, fgs = build_manager(base, tables, mlp, np.float16)
    requests = []
    ref = pm.create_predictor(1, 0)
    for batch, seed in ((128, 1), (61, 2), (128, 3), (200, 4)):
        cfg = Config2(batch=batch, rows=3000, slots=26)
        sparse, dense = cfg.batches(1, seed_offset=seed)
        feed_inputs(ref, fgs, sparse[0], dense[0], np.float16)
        ref.forward()
        items = []
        for (fg, _, _), (ids, vals, seg) in zip(fgs, sparse[0]):
            items += [(fg + ".ids", ids), (fg + ".values", vals), (fg + ".segments", seg)]
        items.append(("dense", dense[0].astype(np.float16)))
        requests.append((items, ref.output_asnumpy("prob").copy()))
    errors = []

    def worker(t):
        try:
            p = pm.create_predictor(1, 0)
            batches = [p.feed_batch(items) for items, _ in requests]
            for i in range(60):
                r = (i + t) % len(requests)
                for name, a in requests[r][0]:
                    p.reshape_input(name, a.shape)
                p.feed_many(batches[r])
                p.forward()
                got = p.output_asnumpy("prob")
                if not np.array_equal(got, requests[r][1]):
                    errors.append("thread %d step %d request %d: max diff %g" % (t, i, r, np.abs(got.astype(np.float32) - requests[r][1].astype(np.float32)).max()))
                    return
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=worker, args=(t, )) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_optimized_model_file_gives_the_same_outputs(pb, oracle, tmp_path):
    """NetDef -> NetDef: Blaze_OptimizeBlaze rewrites three sibling Gemms (constant weights and biases of one shape)
    into FusedParallelGemm + Split; the optimized model file, loaded through Blaze_PredcitorManagerLoadModel, gives the
    outputs of the original one and of the oracle, with one FC launch and a Split that copies nothing.  Also the
    reference's own fixture (tests/golden/pattern/parallel_gemm_fusion.blaze, moved to the device)."""
    import json
    rng = np.random.default_rng(11)
    M, K, N, P = 37, 24, 16, 3
    x = rng.standard_normal((M, K)).astype(np.float32)
    ws = [(rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32) for _ in range(P)]
    bs = [(rng.standard_normal(N) * 0.1).astype(np.float32) for _ in range(P)]
    nb = pb.NetBuilder("siblings", device_type=1)
    nb.external_input("x", pb.K_FLOAT)
    nb.arg("pack_sibling_gemms", 0)  # keep the in-net packing out of it: this test is about the offline pass
    for p in range(P):
        nb.constant("w%d" % p, ws[p])
        nb.constant("b%d" % p, bs[p])
    for p in range(P):
        nb.op("Gemm", ["x", "w%d" % p, "b%d" % p], ["y%d" % p])
    nb.op("Concat", ["y%d" % p for p in range(P)], ["out"], axis=1)
    nb.external_output("out", pb.K_FLOAT)
    raw, opt = str(tmp_path / "raw.blaze"), str(tmp_path / "opt.blaze")
    open(raw, "wb").write(pb.convert_netdef(nb.text().encode(), True, False))
    pb.optimize_blaze(raw, opt, True)
    outs = {}
    for path in (raw, opt):
        pm = pb.PredictorManager()
        pm.load_model(path)
        p = pm.create_predictor(1, 0)
        p.reshape_input("x", [M, K])
        p.feed("x", x)
        p.register_observers(["profile"])
        p.forward()
        outs[path] = p.output_asnumpy("out").copy()
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        kinds = [e["name"].split(":")[0] for e in ev if not e["name"].startswith("ConstantFill")]
        if path == opt:
            assert kinds == ["FusedParallelGemm", "Split", "Concat"], kinds
            assert [e["args"]["launches"] for e in ev if e["name"].split(":")[0] in ("FusedParallelGemm", "Split")] == [1, 0]
        else:
            assert kinds == ["Gemm"] * P + ["Concat"], kinds
    want = np.concatenate([oracle.gemm_op(x, ws[p], bs[p], False, False, 1.0, 1.0) for p in range(P)], axis=1)
    np.testing.assert_allclose(outs[raw], want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(outs[opt], want, rtol=1e-5, atol=1e-6)
    # the reference's fixture: constants only, placed on the device
    text = open(os.path.join(ROOT, "tests", "golden", "pattern", "parallel_gemm_fusion.blaze")).read().replace("device_type: 0", "device_type: 1")
    raw2, opt2 = str(tmp_path / "raw2.blaze"), str(tmp_path / "opt2.blaze")
    open(raw2, "w").write(text)
    pb.optimize_blaze(raw2, opt2, False)
    got = []
    for path in (raw2, opt2):
        pm = pb.PredictorManager()
        pm.load_model(path)
        p = pm.create_predictor(1, 0)
        p.forward()
        got.append(p.output_asnumpy("output").copy())
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    w = np.arange(6, dtype=np.float32).reshape(3, 2)
    assert np.array_equal(got[0], np.concatenate([a @ w, a @ w], axis=1)) and np.array_equal(got[0], got[1])


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_sibling_gemms_run_as_one_launch(pb, oracle, dtype):
    """Three towers read the same input: Gemm + PRelu each with weights of one shape (what the reference's ParallelGemm
    fusion rewrites into FusedParallelGemm + Split, parallel_gemm_fusion_pattern_impl.cc:20-98), plus a fourth Gemm of
    another width that must stay on its own.  By default the three run as one launch and their outputs are views of
    one buffer; with pack_sibling_gemms: 0 each runs by itself.  Both against the oracle; a second request with another
    batch size reuses the stacked weights."""
    rng = np.random.default_rng(41)
    code = pb.K_FLOAT16 if dtype == np.float16 else pb.K_FLOAT
    K, N, N4 = 48, 24, 40
    r = (lambda x: np.asarray(x, np.float32).astype(np.float16).astype(np.float32)) if dtype == np.float16 else (lambda x: np.asarray(x, np.float32))
    ws = [(rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32) for _ in range(3)]
    bs = [(rng.standard_normal(N) * 0.1).astype(np.float32) for _ in range(3)]
    slopes = [rng.uniform(0.1, 0.4, N).astype(np.float32) for _ in range(3)]
    w4 = (rng.standard_normal((K, N4)) / np.sqrt(K)).astype(np.float32)
    outs = {}
    for pack in (1, 0):
        nb = pb.NetBuilder("towers", device_type=1)
        nb.external_input("x", code)
        nb.external_output("y", code)
        nb.arg("pack_sibling_gemms", pack)
        for t in range(3):
            nb.constant("w%d" % t, ws[t], dtype=code)
            nb.constant("b%d" % t, bs[t], dtype=code)
            nb.constant("s%d" % t, slopes[t], dtype=code)
        nb.constant("w4", w4, dtype=code)
        for t in range(3):
            nb.op("Gemm", ["x", "w%d" % t, "b%d" % t], ["h%d" % t])
            nb.op("PRelu", ["h%d" % t, "s%d" % t], ["t%d" % t])
        nb.op("Gemm", ["x", "w4"], ["t3"])
        nb.op("Concat", ["t0", "t1", "t2", "t3"], ["y"], axis=1)
        pm = pb.PredictorManager()
        pm.load_model_from_string(nb.text(), True)
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for batch in (70, 33, 70):
            x = rng.standard_normal((batch, K)).astype(np.float32) if pack == 1 or True else None
            x = np.random.default_rng(batch).standard_normal((batch, K)).astype(np.float32)
            p.reshape_input("x", x.shape)
            p.feed("x", x.astype(dtype))
            print("sibling case dtype=%s pack=%d batch=%d" % (dtype.__name__, pack, batch), flush=True)
            p.forward()
            got.append((x, p.output_asnumpy("y").astype(np.float32)))
        ev = json.loads(p.dump_observers()["profile"])["traceEvents"]
        gemms = [e for e in ev if e["name"].startswith("Gemm") and e["dur"] > 0]
        if pack:
            assert len(gemms) == 2 and sorted(e["args"]["launches"] for e in gemms) == [1, 1], gemms
        else:
            assert len(gemms) == 4
        outs[pack] = got
    tol = 2e-3 if dtype == np.float16 else 1e-5
    for pack in (1, 0):
        for x, y in outs[pack]:
            xr = r(x)
            want = [oracle.prelu(r(oracle.gemm_op(xr, r(ws[t]), r(bs[t]))), r(slopes[t])) for t in range(3)]
            want.append(oracle.gemm_op(xr, r(w4), None))
            want = r(np.concatenate([r(w_) for w_ in want], axis=1))
            assert y.shape == want.shape
            np.testing.assert_allclose(y, want, rtol=tol, atol=tol)
    for (x1, y1), (x0, y0) in zip(outs[1], outs[0]):
        np.testing.assert_allclose(y1, y0, rtol=tol, atol=tol)


def test_folded_gemm_chain_gives_the_same_outputs(pb, oracle, tmp_path):
    """Blaze_OptimizeBlaze folds Gemm(transB, alpha, beta, bias) -> Gemm(bias) with nothing between them into one Gemm on
    the product of the weights; the folded model gives the original's outputs (to the reassociation of fp32 sums) with one
    FC launch instead of two.  Also the reference's four fixtures (tests/golden/pattern/in_order_gemm_gemm_fusion*.blaze,
    constants only, moved to the device): the folded nets' outputs are those of the unfolded ones."""
    import json
    rng = np.random.default_rng(12)
    M, K, H, N = 41, 24, 32, 16
    x = rng.standard_normal((M, K)).astype(np.float32)
    w0 = (rng.standard_normal((H, K)) / np.sqrt(K)).astype(np.float32)   # used transposed
    w1 = (rng.standard_normal((H, N)) / np.sqrt(H)).astype(np.float32)
    b0, b1 = (rng.standard_normal(H) * 0.1).astype(np.float32), (rng.standard_normal(N) * 0.1).astype(np.float32)
    nb = pb.NetBuilder("chain", device_type=1)
    nb.external_input("x", pb.K_FLOAT)
    for name, v in (("w0", w0), ("b0", b0), ("w1", w1), ("b1", b1)):
        nb.constant(name, v)
    nb.op("Gemm", ["x", "w0", "b0"], ["h"], transB=1, alpha=0.5, beta=2.0)
    nb.op("Gemm", ["h", "w1", "b1"], ["out"])
    nb.external_output("out", pb.K_FLOAT)
    raw, opt = str(tmp_path / "raw.blaze"), str(tmp_path / "opt.blaze")
    open(raw, "wb").write(pb.convert_netdef(nb.text().encode(), True, False))
    pb.optimize_blaze(raw, opt, True)
    outs = {}
    for path in (raw, opt):
        pm = pb.PredictorManager()
        pm.load_model(path)
        p = pm.create_predictor(1, 0)
        p.reshape_input("x", [M, K])
        p.feed("x", x)
        p.register_observers(["profile"])
        p.forward()
        outs[path] = p.output_asnumpy("out").copy()
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        kinds = [e["name"].split(":")[0] for e in ev if not e["name"].startswith("ConstantFill")]
        assert kinds == (["Gemm"] if path == opt else ["Gemm", "Gemm"]), kinds
    want = oracle.gemm_op(oracle.gemm_op(x, w0, b0, False, True, 0.5, 2.0), w1, b1, False, False, 1.0, 1.0)
    np.testing.assert_allclose(outs[raw], want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(outs[opt], want, rtol=1e-5, atol=1e-5)
    for case in ("", "2", "3", "4"):
        text = open(os.path.join(ROOT, "tests", "golden", "pattern", "in_order_gemm_gemm_fusion%s.blaze" % case)).read()
        raw2, opt2 = str(tmp_path / ("raw%s.blaze" % case)), str(tmp_path / ("opt%s.blaze" % case))
        open(raw2, "w").write(text.replace("device_type: 0", "device_type: 1"))
        pb.optimize_blaze(raw2, opt2, False)
        got = []
        for path in (raw2, opt2):
            pm = pb.PredictorManager()
            pm.load_model(path)
            p = pm.create_predictor(1, 0)
            p.forward()
            got.append(p.output_asnumpy("output").copy())
        assert got[0].shape == (2, 3) and got[0].any()
        np.testing.assert_allclose(got[1], got[0], rtol=1e-6, atol=0)


@pytest.mark.parametrize("out_dtype", [np.float32, np.float16])
@pytest.mark.parametrize("with_keys", [False, True])
def test_store_get_with_host_pointers(pb, oracle, out_dtype, with_keys):
    """SparsePuller::Get in the reference's own form (blaze/store/sparse_puller.h:77-83: every pointer host memory), as
    its host Embedding operator calls it (embedding_op.cc:87): bit-identical to the oracle's QuickEmbeddingDict::Get on
    the same block; columns of no item and the columns of an unknown table keep the caller's contents; two calls in a
    row on one thread (the second smaller) reuse the staging state; calls from other threads are served too."""
    import threading
    rng = np.random.default_rng(77)
    rows, dim = 500, 12
    data = rng.standard_normal((rows, dim)).astype(np.float32)
    keys = rng.choice(1 << 40, rows, replace=False).astype(np.int64) if with_keys else None
    pm = pb.PredictorManager()
    pm.add_table("t", data, keys=keys)
    table = oracle.Table(data, keys=None if keys is None else keys.astype(np.uint64))

    def case(batch, seed):
        r = np.random.default_rng(seed)
        seg = r.integers(0, 7, batch).astype(np.int32)
        seg[r.integers(0, batch)] = 0
        nnz = int(seg.sum())
        pick = r.integers(0, rows, nnz)
        ids = (keys[pick] if with_keys else pick).astype(np.int64)
        ids[r.random(nnz) < 0.1] = (1 << 41) + 5  # unknown keys are skipped
        vals = r.standard_normal(nnz).astype(np.float32)
        return ids, seg, vals

    def run(batch, seed):
        ids, seg, vals = case(batch, seed)
        stride = 3 + dim + dim + 4 * dim + 2
        layout = [(oracle.SUM, oracle.REVERSE, 0, 3), (oracle.AVG, oracle.ORDER, 3, 3 + dim),
                  (oracle.ASSIGN, oracle.REVERSE, 4, 3 + 2 * dim)]
        sentinel = r0 = np.random.default_rng(seed + 1).standard_normal((batch, stride)).astype(np.float32)
        want = sentinel.copy()
        oracle.embed_get(table, ids, vals, seg, [(u, d, n, want, c) for u, d, n, c in layout])
        got = sentinel.astype(out_dtype)
        pm.store_get("t", ids, seg, vals, dim, [(u, d, n, got, c) for u, d, n, c in layout])
        if out_dtype == np.float32:
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        else:
            # item columns: the fp32 result narrowed once (round to nearest even); the rest: the caller's halves
            item = np.zeros(stride, bool)
            item[3:3 + 6 * dim] = True
            expect = np.where(item[None, :], want, r0.astype(np.float16).astype(np.float32)).astype(np.float16)
            assert np.array_equal(got.view(np.uint16), expect.view(np.uint16))
        # unknown table: nothing is written
        keep = sentinel.astype(out_dtype)
        before = keep.copy()
        pm.store_get("no_such_table", ids, seg, vals, dim, [(u, d, n, keep, c) for u, d, n, c in layout])
        assert np.array_equal(keep.view(np.uint8), before.view(np.uint8))

    run(300, 1)
    run(37, 2)
    run(1, 3)
    errors = []

    def worker(seed):
        try:
            run(120, seed)
        except BaseException as e:  # noqa: BLE001 -- reported by the main thread
            errors.append(e)

    ts = [threading.Thread(target=worker, args=(10 + i,)) for i in range(3)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors, errors
    # the counts must add up to the ids handed over
    ids, seg, vals = case(20, 5)
    with pytest.raises(pb.BlazeError):
        pm.store_get("t", ids, seg, vals, dim, [(oracle.SUM, 0, 0, np.zeros((20, 4), np.float32), 0)])  # stride < dim

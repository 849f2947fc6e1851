"""GPU tests of what lies either side of the hot path: model files, table files, request-sized inputs (all through the
Blaze_* C ABI).

* a binary NetDef file read by Blaze_PredcitorManagerLoadModel (predictor_manager_impl.cc:31-116), fp16 ConstantFill
  values narrowed as blaze/common/proto_helper.cc:174 does;
* the reference's own text tables (utest_data/store/quick_embedding) through the QED builder and the device reader;
* config 2 at full size through Predictor.Forward against the oracle;
* counts that disagree with the ids array (a malformed request) leave every read inside the arrays;
* requests of changing sizes (ReshapeInput + FeedMany + Forward) allocate nothing once warmed up.
"""
import os

import numpy as np
import pytest

from test_predictor_gpu import _ctr_text, _oracle_ctr

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


def _r16(x):
    return np.asarray(x, np.float32).astype(np.float16).astype(np.float32)


def _small_ctr_case(rng, n_tables=3, batch=41):
    fgs = [("10%d" % i, "t_%d" % i, (8, 16, 4)[i % 3]) for i in range(n_tables)]
    blocks = [[dict(fg=fg, udf=i % 2) for i, (fg, _, _) in enumerate(fgs)]]
    tables = {}
    for _, tname, dim in fgs:
        n = int(rng.integers(40, 90))
        keys = np.unique(rng.integers(-2**40, 2**40, n * 2, dtype=np.int64))[:n]
        tables[tname] = (keys, (rng.standard_normal((n, dim)) * 0.5).astype(np.float32))
    inputs = {}
    for fg, tname, _ in fgs:
        seg = rng.integers(0, 7, batch).astype(np.int32)
        pool = np.concatenate([tables[tname][0], rng.integers(-2**40, 2**40, 5, dtype=np.int64)])
        ids = rng.choice(pool, int(seg.sum())).astype(np.int64)
        inputs[fg] = (ids, rng.standard_normal(ids.size).astype(np.float32), seg)
    return fgs, blocks, tables, inputs


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_binary_model_file_through_load_model(pb, oracle, tmp_path, dtype):
    """text NetDef -> Blaze_ConvertNetDef -> file -> Blaze_PredcitorManagerLoadModel(path) -> Forward, against the
    oracle; the text form of the same net loaded from a file gives the same bits."""
    rng = np.random.default_rng(21)
    fgs, blocks, tables, inputs = _small_ctr_case(rng)
    batch, dense_dim = 41, 6
    width = sum(d for _, _, d in fgs)
    layers = (dense_dim + width, 24, 16, 2)
    acts = ("PRelu", "Dice", "Softmax")
    text, weights = _ctr_text(pb, fgs, blocks, dense_dim, layers, acts, dtype, True)
    wire = pb.convert_netdef(text, True, False)
    assert wire[:1] != b"n" and len(wire) > 1000
    bin_path, txt_path = str(tmp_path / "model_blaze"), str(tmp_path / "model_blaze.txt")
    open(bin_path, "wb").write(wire)
    open(txt_path, "w").write(text)
    dense = rng.standard_normal((batch, dense_dim)).astype(np.float32)
    r = _r16 if dtype == np.float16 else (lambda x: x)
    got = []
    for path, spelling in ((bin_path, "Blaze_PredcitorManagerLoadModel"), (bin_path, "Blaze_PredictorManagerLoadModel"),
                           (txt_path, "Blaze_PredcitorManagerLoadModel")):
        pm = pb.PredictorManager()
        for tname, (keys, rows) in tables.items():
            pm.add_table(tname, rows.astype(dtype), keys=keys)
        rc = getattr(pb.lib(), spelling)(pm.handle, path.encode(), 0)
        assert rc == 0, pb.last_error()
        p = pm.create_predictor(1, 0)
        for fg, (ids, vals, seg) in inputs.items():
            p.feed(fg + ".ids", ids)
            p.feed(fg + ".values", vals)
            p.feed(fg + ".segments", seg)
        p.feed("dense", dense.astype(dtype))
        print("binary model case dtype=%s file=%s via %s" % (dtype.__name__, os.path.basename(path), spelling), flush=True)
        p.forward()
        out = p.output_asnumpy("prob")
        assert out.shape == (batch, 2) and out.dtype == dtype
        got.append(out.astype(np.float32))
        # the weights the predictor holds are the file's fp32 values narrowed to the blob type, nearest even
        np.testing.assert_array_equal(p.internal_asnumpy("w0"), weights[0][0].astype(dtype))
    assert np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[2])
    otabs = {t: oracle.Table(rows.astype(dtype), keys=keys) for t, (keys, rows) in tables.items()}
    want = _oracle_ctr(oracle, otabs, fgs, blocks, inputs, dense, weights, acts, r)
    tol = 2e-3 if dtype == np.float16 else 1e-5
    np.testing.assert_allclose(got[0], want, rtol=tol, atol=tol)


def test_reference_text_tables_through_builder_and_device_reader(pb, oracle, tmp_path):
    """The reference's utest_data/store/quick_embedding text tables (embedding_builder_test.cc:13-23) -> QED file ->
    Blaze_LoadSparseModelWeight -> Embedding on the device; every key of the tables plus absent keys, ksum / kavg /
    kassign, against the oracle's dictionary walk: bit-exact."""
    from test_host_cpu import _reference_text_tables
    d, tables = _reference_text_tables()
    qed = str(tmp_path / "ref.qed")
    pb.build_qed(d, "meta", qed)
    fgs = [("f1", "a_01", 9), ("f2", "a_02", 9), ("f3", "a_03", 9)]  # a_03 is not in the file: meta's last line has no newline
    blocks = [[dict(fg="f1", udf=0), dict(fg="f2", udf=1), dict(fg="f3", udf=0)],
              [dict(fg="f2", udf=2, trunc_dir=0, trunc_num=3)]]
    rng = np.random.default_rng(8)
    batch = 23
    inputs = {}
    for fg, tname, _ in fgs:
        keys = tables[tname][0]
        seg = rng.integers(0, 5, batch).astype(np.int32)
        seg[0] = len(keys)  # one sample walks the whole table
        pool = np.concatenate([keys, np.array([0, 2424123, -1], np.int64)])
        ids = np.concatenate([keys, rng.choice(pool, int(seg[1:].sum()))]).astype(np.int64)
        inputs[fg] = (ids, rng.uniform(0.5, 1.5, ids.size).astype(np.float32), seg)
    nb = pb.NetBuilder("lookup", device_type=1)
    names = []
    for fg, _, _ in fgs:
        nb.external_input(fg + ".ids", pb.K_INT64)
        nb.external_input(fg + ".values", pb.K_FLOAT)
        nb.external_input(fg + ".segments", pb.K_INT32)
        names += [fg + ".ids", fg + ".values", fg + ".segments"]
    nb.external_output("b0", pb.K_FLOAT)
    nb.external_output("b1", pb.K_FLOAT)
    nb.op("Embedding", names, ["b0", "b1"], embedding_config=pb.embedding_config_text(fgs, blocks))
    pm = pb.PredictorManager()
    pm.load_sparse_model_weight(qed)
    pm.load_model_from_string(nb.text(), True)
    p = pm.create_predictor(1, 0)
    for fg, (ids, vals, seg) in inputs.items():
        p.feed(fg + ".ids", ids)
        p.feed(fg + ".values", vals)
        p.feed(fg + ".segments", seg)
    print("reference text tables: a_01 %d rows, a_02 %d rows, dim 9" % (len(tables["a_01"][0]), len(tables["a_02"][0])), flush=True)
    p.forward()
    otabs = {"a_01": oracle.Table(tables["a_01"][1], keys=tables["a_01"][0]),
             "a_02": oracle.Table(tables["a_02"][1], keys=tables["a_02"][0])}
    want = oracle.embedding_op({fg: (t, dim) for fg, t, dim in fgs}, blocks, inputs, otabs)
    for i, name in enumerate(("b0", "b1")):
        got = p.output_asnumpy(name)
        assert got.shape == want[i].shape and got.dtype == np.float32
        assert np.array_equal(got.view(np.uint32), want[i].view(np.uint32)), name
    b0 = p.output_asnumpy("b0")
    assert b0[:, :18].any() and not b0[:, 18:].any()  # the table missing from the file leaves its columns zero


@pytest.mark.timeout(300)
def test_config2_full_size_through_predictor_against_oracle(pb, oracle):
    """Batch 2048, 26 x [1M, 32] fp16 tables, MLP 896-512-256-2: one Predictor.Forward end to end.  The pooled block
    equals the oracle's fp32 block rounded to fp16 (bit for bit), the probabilities agree within 2e-3."""
    import torch
    from ctr_model import build_manager, make_predictor
    from model_forward import ctr_forward
    from synth import Config2
    torch.cuda.empty_cache()
    cfg = Config2()
    print("config2 full size: batch %d, %d x [%d,%d] fp16" % (cfg.batch, cfg.slots, cfg.rows, cfg.dim), flush=True)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(1)
    pm, fgs = build_manager(cfg, tables, mlp, np.float16, expose_block=True)
    p = make_predictor(pm, fgs, sparse[0], dense[0], np.float16)
    p.forward()
    prob = p.output_asnumpy("prob").astype(np.float32)
    block = p.output_asnumpy("block")
    assert prob.shape == (cfg.batch, 2) and block.shape == (cfg.batch, cfg.slots * cfg.dim) and block.dtype == np.float16
    tabs = [oracle.Table(t.cpu().numpy()) for t in tables]
    mlp_np = [(_r16(w.cpu().numpy()), _r16(b.cpu().numpy()), _r16(s.cpu().numpy())) for (w, b, s) in mlp]
    want_pooled, want = ctr_forward(oracle, cfg, tabs, mlp_np, sparse[0], dense[0], in_round=_r16)
    assert np.array_equal(block.view(np.uint16), want_pooled[:, cfg.dense:].astype(np.float16).view(np.uint16))
    np.testing.assert_allclose(prob, want, rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(prob.sum(1), 1.0, atol=2e-3)


def test_counts_that_disagree_with_the_ids_are_kept_inside_the_arrays(pb, oracle):
    """A request whose per-sample counts sum past the ids array, or hold a negative count, must not read outside ids /
    values: negative counts count as zero and offsets stop at the array length, so the call returns normally and the
    result is that of the clamped counts."""
    import blaze_hip as bz
    import torch
    rng = np.random.default_rng(3)
    rows, dim, batch = 500, 32, 300
    table = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float16)
    seg = rng.integers(1, 9, batch).astype(np.int32)
    nnz = int(seg.sum()) - 400  # the array ends well before the counts do
    ids = rng.integers(0, rows, nnz).astype(np.int64)
    vals = rng.uniform(0.5, 1.5, nnz).astype(np.float32)
    bad = seg.copy()
    bad[5] = -7
    bad[17] = -(2**31)
    bad[-1] = 2**31 - 1
    # what the kernel is specified to use: max(count, 0), running offsets capped at nnz
    off = np.minimum(np.concatenate([[0], np.cumsum(np.maximum(bad, 0).astype(np.int64))]), nnz)
    eff = np.diff(off).astype(np.int32)
    assert eff.sum() == nnz and eff[5] == 0
    dt = bz.DeviceTable(torch.from_numpy(table).cuda())
    for udf in (bz.SUM, bz.AVG, bz.ASSIGN):
        for fused in (True, False):
            trunc = 4 if udf == bz.ASSIGN else 0
            width = dim * max(trunc, 1)
            out = torch.full((batch, width), float("nan"), dtype=torch.float32, device="cuda")
            # ids / values sit at the very end of their allocations
            d_ids, d_vals = torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda()
            item = dict(table=dt, ids=d_ids, values=d_vals, segments=torch.from_numpy(bad).cuda(), out=out, udf=udf,
                        trunc_num=trunc, trunc_dir=bz.ORDER)
            print("clamp case udf=%d fused_scan=%s nnz=%d sum(counts)=%d" % (udf, fused, nnz, int(np.maximum(bad, 0).sum())), flush=True)
            bz.EmbeddingPlan([item], fused_scan=fused).run()
            torch.cuda.synchronize()
            want = np.zeros((batch, width), np.float32)
            # kavg divides by the clamped count: the kernel never learns of ids it does not have
            oracle.embed_get(oracle.Table(table), ids, vals, eff, [(udf, 0, trunc, want, 0)])
            assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_requests_of_changing_size_allocate_nothing_in_steady_state(pb, oracle):
    """ReshapeInput + FeedMany + Forward with nnz changing from request to request: after the largest request has been
    seen once, no request allocates (device, pinned or operator scratch), and every result still matches the oracle."""
    rng = np.random.default_rng(31)
    fgs, blocks, tables, _ = _small_ctr_case(rng, n_tables=3)
    dense_dim = 6
    width = sum(d for _, _, d in fgs)
    layers = (dense_dim + width, 16, 2)
    acts = ("PRelu", "Softmax")
    text, weights = _ctr_text(pb, fgs, blocks, dense_dim, layers, acts, np.float32, True)
    pm = pb.PredictorManager()
    for tname, (keys, rows) in tables.items():
        pm.add_table(tname, rows, keys=keys)
    pm.load_model_from_string(text, True)
    p = pm.create_predictor(1, 0)
    otabs = {t: oracle.Table(rows, keys=keys) for t, (keys, rows) in tables.items()}

    def request(batch, max_len):
        inputs = {}
        for fg, tname, _ in fgs:
            seg = rng.integers(0, max_len + 1, batch).astype(np.int32)
            ids = rng.choice(tables[tname][0], int(seg.sum())).astype(np.int64)
            inputs[fg] = (ids, rng.standard_normal(ids.size).astype(np.float32), seg)
        return inputs, rng.standard_normal((batch, dense_dim)).astype(np.float32)

    def serve(inputs, dense):
        items = []
        for fg, (ids, vals, seg) in inputs.items():
            items += [(fg + ".ids", ids), (fg + ".values", vals), (fg + ".segments", seg)]
        items.append(("dense", dense))
        for name, a in items:
            p.reshape_input(name, a.shape)
        p.feed_many(p.feed_batch(items))
        p.forward()
        got = p.output_asnumpy("prob")
        want = _oracle_ctr(oracle, otabs, fgs, blocks, inputs, dense, weights, acts, lambda x: x)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)

    serve(*request(64, 12))       # the largest request first: arena, blobs and scratch reach their final sizes
    serve(*request(64, 12))
    before = pb.allocation_count()
    for i in range(12):
        batch = int(rng.integers(1, 65))
        print("request %d: batch %d" % (i, batch), flush=True)
        serve(*request(batch, int(rng.integers(1, 13))))
    assert pb.allocation_count() == before, "a steady-state request allocated memory"
    # a request that outgrows everything is still served (and may allocate)
    serve(*request(200, 20))
    # reshaping an input beyond what was fed and running without feeding it is refused, not run on stale memory
    p.reshape_input(fgs[0][0] + ".ids", (100000, ))
    with pytest.raises(pb.BlazeError, match="reshaped"):
        p.forward()


def test_the_reference_shipped_model_file_end_to_end(pb, oracle):
    """blaze/example/tdm_data/model_blaze_optimized, the one binary model the reference ships (committed byte for byte as
    tests/golden/model_blaze_optimized.bin: 70 Embedding, 69 Gather, 10 Slice, ReduceSum, Div, Concat, Reshape, Gemm,
    BatchNormalization, PRelu, Softmax; exported for the CPU, run_mode hybrid), loaded unmodified through
    Blaze_PredcitorManagerLoadModel, fed synthetic inputs (69 user-level feature groups over 9 users, expanded to 70 ads by
    indicator.0; one ad-level group) and a synthetic `item_emb` table, against the oracle's operator-by-operator forward
    of the same file.  fp32: pooled and gathered blocks bit-exact, probabilities to 1e-5.  The reference ships no
    expected output for this model: parity rests on the operators' own known answers."""
    from blaze_proto import NetDef
    import model_forward
    path = os.path.join(ROOT, "tests", "golden", "model_blaze_optimized.bin")
    net = NetDef()
    net.ParseFromString(open(path, "rb").read())
    rng = np.random.default_rng(2024)
    rows, dim, users, ads = 4000, 24, 9, 70
    table = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float32)
    keys = np.unique(rng.integers(1, 2**40, rows * 2, dtype=np.int64))[:rows]
    feeds = {"indicator.0": rng.integers(0, users, ads).astype(np.int32)}
    groups = sorted({v.name.rsplit(".", 1)[0] for v in net.external_input if v.name != "indicator.0"})
    assert len(groups) == 70 and len(net.external_input) == 211
    for fg in groups:
        batch = ads if fg == "unit_id_expand" else users
        seg = rng.integers(0, 5, batch).astype(np.int32)
        seg[rng.integers(0, batch)] = 0
        nnz = int(seg.sum())
        ids = rng.choice(np.concatenate([keys, np.array([-5, 2**41], np.int64)]), nnz).astype(np.int64)  # two keys the table lacks
        feeds[fg + ".ids"], feeds[fg + ".values"], feeds[fg + ".segments"] = ids, rng.uniform(0.5, 1.5, nnz).astype(np.float32), seg
    want = model_forward.run_netdef(oracle, net, feeds, {"item_emb": oracle.Table(table, keys=keys)})
    assert want["softmaxoutput0"].shape == (ads, 2) and want["concat10"].shape == (ads, 264)

    pm = pb.PredictorManager()
    pm.add_table("item_emb", table, keys=keys)
    pm.load_model(path)
    p = pm.create_predictor(1, 0)
    assert sorted(p.list_input_names()) == sorted(feeds)
    for name, arr in feeds.items():
        p.feed(name, arr)
    p.forward()
    got = p.output_asnumpy("softmaxoutput0")
    assert got.shape == (ads, 2)
    np.testing.assert_allclose(got, want["softmaxoutput0"], rtol=1e-5, atol=1e-6)
    assert np.abs(got.sum(1) - 1).max() < 1e-5 and got.std() > 1e-3
    # a second request of another size through the same predictor
    feeds2 = dict(feeds)
    feeds2["indicator.0"] = feeds["indicator.0"][:33]
    seg = feeds["unit_id_expand.segments"][:33]
    n = int(seg.sum())
    feeds2["unit_id_expand.segments"], feeds2["unit_id_expand.ids"], feeds2["unit_id_expand.values"] = \
        seg, feeds["unit_id_expand.ids"][:n], feeds["unit_id_expand.values"][:n]
    want2 = model_forward.run_netdef(oracle, net, feeds2, {"item_emb": oracle.Table(table, keys=keys)})
    for name in ("indicator.0", "unit_id_expand.segments", "unit_id_expand.ids", "unit_id_expand.values"):
        p.feed(name, feeds2[name])
    p.forward()
    np.testing.assert_allclose(p.output_asnumpy("softmaxoutput0"), want2["softmaxoutput0"], rtol=1e-5, atol=1e-6)

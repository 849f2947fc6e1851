"""The benchmark configurations at their full sizes, as parity cases (GPU).

config 1 (fp32, batch 128) runs through Predictor.Forward and is compared with the CPU oracle end to end:
pooled block bit-exact, probabilities rel 1e-5.  config 4 (int8 + per-row scale, 34 GB of tables) and
config 5 (fp16 tables, 102 GB; bf16 MLP whose first layer is 215 GFLOP) are generated on the device; the
oracle sees only the rows a batch touches (copied back and indexed by key).  Tolerance for the fp16 / bf16 /
int8 paths: 2e-3 against the fp32 oracle fed the same rounded inputs.  Size-independent properties checked at
full size: scaling all values by 2 doubles every pooled element exactly; an empty segment gives a zero row.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def bz():
    import torch
    import blaze_hip
    assert torch.cuda.is_available(), "no GPU visible"
    blaze_hip.device_check()
    return blaze_hip


def _touched_table(oracle, dev_rows, ids, dev_scale=None, regen=None):
    """Oracle table holding only the rows `ids` name, keyed by id (the device indexes the full table by row).
    regen(unique rows) -> rows [, scale]: the generator's own values for those rows, computed on the host; the oracle is
    then fed these, and the device's copy of the same rows must hold the same bits (the fill kernel against numpy)."""
    import torch
    uniq = np.unique(ids)
    idx = torch.from_numpy(uniq).cuda()
    rows = dev_rows[idx].cpu().numpy()
    scale = None if dev_scale is None else dev_scale[idx].cpu().numpy()
    if regen is not None:
        host = regen(uniq)
        host_rows, host_scale = host if isinstance(host, tuple) else (host, None)
        assert host_rows.dtype == rows.dtype and np.array_equal(host_rows.view(np.uint8), rows.view(np.uint8)), "table rows differ from the generator's"
        assert (scale is None) == (host_scale is None)
        if scale is not None:
            assert np.array_equal(host_scale.view(np.uint32), scale.view(np.uint32)), "row scales differ from the generator's"
        rows, scale = host_rows, host_scale
    return oracle.Table(rows, scale=scale, keys=uniq.astype(np.uint64))


def _bf16_round(x):
    """fp32 -> nearest-even bf16, back to fp32 (numpy)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def test_config1_fp32_end_to_end_through_predictor(oracle):
    import torch
    from ctr_model import build_manager, make_predictor
    from model_forward import ctr_forward as oracle_forward
    from synth import Config1
    cfg = Config1()
    print("config1 full size: batch %d, %d x [%d,%d] fp32" % (cfg.batch, cfg.slots, cfg.rows, cfg.dim), flush=True)
    tables, mlp = cfg.tables(), cfg.mlp()
    sparse, dense = cfg.batches(2)
    pm, fgs = build_manager(cfg, tables, mlp, np.float32, expose_block=True)
    tabs = [oracle.Table(t.cpu().numpy()) for t in tables]
    mlp_np = [(w.cpu().numpy(), b.cpu().numpy(), s.cpu().numpy()) for (w, b, s) in mlp]
    for b in range(2):
        p = make_predictor(pm, fgs, sparse[b], dense[b], np.float32)
        p.forward()
        prob = p.output_asnumpy("prob")
        block = p.output_asnumpy("block")
        want_pooled, want_prob = oracle_forward(oracle, cfg, tabs, mlp_np, sparse[b], dense[b])
        # pooled block: bit-exact (same summation order, unfused multiply/add)
        assert np.array_equal(block.view(np.uint32), want_pooled[:, cfg.dense:].view(np.uint32))
        assert prob.shape == (cfg.batch, 2)
        np.testing.assert_allclose(prob, want_prob, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(prob.sum(1), 1.0, rtol=1e-5)
    torch.cuda.synchronize()


@pytest.mark.timeout(400)
def test_config4_int8_kavg_full_size(bz, oracle):
    import torch
    torch.cuda.empty_cache()
    from synth import Config4
    cfg = Config4()
    free, _ = torch.cuda.mem_get_info()
    need = cfg.slots * cfg.rows * (cfg.dim + 4)
    if free < need * 1.1:
        pytest.skip("needs %.0f GB of free HBM" % (need / 1e9))
    print("config4 full size: batch %d, %d x [%d,%d] int8 + scale" % (cfg.batch, cfg.slots, cfg.rows, cfg.dim), flush=True)
    tables = cfg.tables()
    # Poisson(20) practically never draws 0: empty every 97th segment so that the zero-row case is in
    rng = np.random.default_rng(44)
    sparse = []
    for ids, vals, seg in cfg.batch_inputs():
        off = np.concatenate([[0], np.cumsum(seg)])
        drop = np.zeros(ids.size, bool)
        for b in range(int(rng.integers(0, 97)), cfg.batch, 97):
            drop[off[b]:off[b + 1]] = True
            seg[b] = 0
        sparse.append((ids[~drop], vals[~drop], seg))
    dts = [bz.DeviceTable(q, scale=sc) for q, sc in tables]
    B, D = cfg.batch, cfg.dim

    def run(scale_values, out_dtype):
        out = torch.full((B, cfg.slots * D), float("nan"), dtype=out_dtype, device="cuda")
        items, keep = [], []
        for s, (ids, vals, seg) in enumerate(sparse):
            t = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals * np.float32(scale_values)).cuda(), torch.from_numpy(seg).cuda()]
            keep.append(t)
            items.append(dict(table=dts[s], ids=t[0], values=t[1], segments=t[2], out=out, col=s * D, udf=bz.AVG))
        bz.EmbeddingPlan(items).run()
        torch.cuda.synchronize()
        return out.cpu().numpy()

    got32 = run(1.0, torch.float32)
    got16 = run(1.0, torch.float16)
    want = np.zeros((B, cfg.slots * D), np.float32)
    for s, (ids, vals, seg) in enumerate(sparse):
        tab = _touched_table(oracle, tables[s][0], ids, tables[s][1], regen=lambda u, s=s: cfg.table_rows(s, u))
        oracle.embed_get(tab, ids, vals, seg, [(1, 0, 0, want, s * D)])
    # fp32 block: the int8 extension is defined as w = scale*(float)q, then the reference's kavg: bit-exact
    assert np.array_equal(got32.view(np.uint32), want.view(np.uint32))
    # fp16 block = that result rounded to nearest even (contract 2e-3)
    assert np.array_equal(got16.view(np.uint16), want.astype(np.float16).view(np.uint16))
    np.testing.assert_allclose(got16.astype(np.float32), want, rtol=2e-3, atol=2e-3 * np.abs(want).max())
    # empty segments are zero rows
    for s, (_, _, seg) in enumerate(sparse[:5]):
        empty = np.nonzero(seg == 0)[0]
        assert empty.size and not got32[empty, s * D:(s + 1) * D].any()
    # linearity in the values (a power of two is exact): pool(2*v) == 2*pool(v)
    got2 = run(2.0, torch.float32)
    assert np.array_equal(got2.view(np.uint32), (got32 * np.float32(2.0)).view(np.uint32))


@pytest.mark.timeout(400)
def test_config5_fp16_tables_bf16_tower_full_size(bz, oracle):
    import torch
    torch.cuda.empty_cache()
    from synth import Config5
    cfg = Config5()
    free, _ = torch.cuda.mem_get_info()
    need = cfg.slots * cfg.rows * cfg.dim * 2
    if free < need * 1.6:  # generation goes through an fp32 temporary of one table
        pytest.skip("needs %.0f GB of free HBM" % (need * 1.6 / 1e9))
    print("config5 full size: batch %d, %d x [%d,%d] fp16, MLP %s bf16" % (cfg.batch, cfg.slots, cfg.rows, cfg.dim, cfg.layers),
          flush=True)
    tables = cfg.tables()
    sparse = cfg.batch_inputs()
    mlp = cfg.mlp()
    dts = [bz.DeviceTable(t) for t in tables]
    B, D = cfg.batch, cfg.dim
    pooled32 = torch.full((B, cfg.slots * D), float("nan"), dtype=torch.float32, device="cuda")
    pooled = torch.full((B, cfg.slots * D), float("nan"), dtype=torch.bfloat16, device="cuda")
    keep = []
    for out in (pooled32, pooled):
        items = []
        for s, (ids, vals, seg) in enumerate(sparse):
            t = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(seg).cuda()]
            keep.append(t)
            items.append(dict(table=dts[s], ids=t[0], values=t[1], segments=t[2], out=out, col=s * D, udf=bz.SUM))
        plan = bz.EmbeddingPlan(items)
        # 128 workgroups per slot would each re-read up to 8192 counts: the planner asks for the separate scan launch
        assert plan.launch.fused_scan == 0 and not plan.fused_scan and plan.total_wg == cfg.slots * 128
        plan.run()
    torch.cuda.synchronize()
    rng = np.random.default_rng(5)
    rows = np.sort(rng.choice(B, 64, replace=False))
    # oracle pooling of every sample for 8 slots, of the 64 sampled rows for all slots
    want_rows = np.zeros((64, cfg.slots * D), np.float32)
    got32 = pooled32.cpu().numpy()
    for s, (ids, vals, seg) in enumerate(sparse):
        off = np.concatenate([[0], np.cumsum(seg)])
        if s % 25 == 0:
            full = np.zeros((B, D), np.float32)
            oracle.embed_get(_touched_table(oracle, tables[s], ids, regen=lambda u, s=s: cfg.table_rows(s, u)), ids, vals, seg, [(0, 0, 0, full, 0)])
            assert np.array_equal(got32[:, s * D:(s + 1) * D].view(np.uint32), full.view(np.uint32))
        sel = np.concatenate([np.arange(off[r], off[r + 1]) for r in rows])
        sub = np.zeros((64, D), np.float32)
        oracle.embed_get(_touched_table(oracle, tables[s], ids[sel], regen=lambda u, s=s: cfg.table_rows(s, u)), ids[sel], vals[sel], seg[rows], [(0, 0, 0, sub, 0)])
        want_rows[:, s * D:(s + 1) * D] = sub
    assert np.array_equal(got32[rows].view(np.uint32), want_rows.view(np.uint32))  # fp32 block: bit-exact
    x0 = _bf16_round(want_rows)
    assert np.array_equal(pooled[torch.from_numpy(rows).cuda()].float().cpu().numpy().view(np.uint32), x0.view(np.uint32))

    # MLP in bf16 (fp32 accumulate); oracle: fp32 path fed the same bf16-rounded inputs, first layer also in fp64
    x = pooled
    h = x0
    n_layers = len(mlp)
    for li, (w, b) in enumerate(mlp):
        last = li == n_layers - 1
        wp = bz.pack_weight(w, False, bz.BF16)
        y = torch.empty((B, w.shape[1]), dtype=torch.float32 if last else torch.bfloat16, device="cuda")
        print("fc layer %d: %dx%d . %dx%d" % (li, B, w.shape[0], w.shape[0], w.shape[1]), flush=True)
        bz.fc_fused(x, wp, w.shape[0], bias=b, act=bz.ACT_SIGMOID if last else bz.ACT_LEAKY_RELU, act_alpha=0.0, out=y)
        torch.cuda.synchronize()
        w_r = _bf16_round(w.cpu().numpy())
        got = y[torch.from_numpy(rows).cuda()].float().cpu().numpy()
        if li == 0:
            ref64 = h.astype(np.float64) @ w_r.astype(np.float64) + b.cpu().numpy().astype(np.float64)
            ref64 = np.where(ref64 >= 0, ref64, 0.0)
            np.testing.assert_allclose(got, ref64, rtol=2e-3, atol=2e-3 * np.abs(ref64).max())
        want = oracle.fc(h, w_r, b.cpu().numpy(), act="sigmoid" if last else "relu")
        np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3 * max(1e-3, float(np.abs(want).max())))
        h = want if last else _bf16_round(want)
        x = y
    assert got.shape == (64, 1) and np.all((got > 0) & (got < 1))


@pytest.mark.timeout(400)
def test_config3_din_attention_end_to_end_through_predictor(oracle):
    """config 3 at full size through Predictor.Forward: two Embedding ops (ksum target, kassign history), the
    attention unit built from Reshape / Concat / Sub / Mul / BroadcastTo / 3-D Gemm + Dice / Mul(mask) / MatMul /
    ReduceSum, the main MLP with Dice, softmax.  fp16 model against the fp32 oracle fed the same fp16-rounded
    tables, weights and intermediate tensors: 2e-3."""
    import torch
    import din_model
    import model_forward
    torch.cuda.empty_cache()
    cfg = din_model.Config3()
    print("config3 full size: batch %d, history %d, 3 x [%d,%d] fp16" % (cfg.batch, cfg.T, cfg.rows, cfg.dim), flush=True)
    tables = cfg.tables()
    weights = cfg.weights()
    batch = cfg.batch_inputs()
    expose = ("q", "his", "score", "att", "hsum")
    pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=expose)
    p = pm.create_predictor(1, 0)
    din_model.feed(p, inputs, batch, np.float16)
    p.forward()
    got = {name: p.output_asnumpy(name).astype(np.float32) for name in expose + ("prob", )}
    # seven kernel launches a forward: 2 Embedding (the history one writes its three blocks straight into the history
    # Concat's output; that Concat does not run), 1 Concat (main input), 3 Gemm (the whole attention MLP 216 -> 80 -> 40 -> 1
    # with its input [q, k, q-k, q*k] computed on the fly; the two launches of the main MLP, each with its Dice / skinny
    # layer / softmax folded in), 1 MatMul (with the Mul and the ReduceSum)
    import json
    p.register_observers(["profile"])
    p.forward()
    ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
    launching = [e for e in ev if e["name"].split(":")[0] not in ("ConstantFill", "Reshape")]
    kinds = sorted(e["name"].split(":")[0] for e in launching)
    assert kinds == ["Concat"] + ["Embedding"] + ["Gemm"] * 3 + ["MatMul"], kinds
    assert [e["args"]["launches"] for e in launching if e["name"].split(":")[0] == "Embedding"] == [1]
    assert all(e["args"]["launches"] == 1 for e in launching if e["name"].split(":")[0] in ("Gemm", "MatMul")), launching
    tabs = {}
    for ki, (k, t) in enumerate(zip(din_model.KINDS, tables)):
        ids = np.concatenate([batch[k + ".ids"], batch[k + "_his.ids"]])
        tabs[k] = _touched_table(oracle, t, ids, regen=lambda u, ki=ki: cfg.table_rows(ki, u))
    rnd = lambda a: np.asarray(a, np.float32).astype(np.float16).astype(np.float32)
    want = model_forward.din_forward(oracle, cfg, tabs, weights, batch, rnd)
    B, T, D3 = cfg.batch, cfg.T, 3 * cfg.dim
    # pooled blocks: exactly the oracle's fp32 result rounded to fp16
    assert np.array_equal(got["q"], want["q"])
    assert got["his"].shape == (B, T, D3) and np.array_equal(got["his"], want["his"])
    # positions past a sample's history are zero rows
    seg = batch["item_his.segments"]
    pad = np.arange(T)[None, :] >= seg[:, None]
    assert not got["his"][pad].any()
    np.testing.assert_allclose(got["hsum"], want["hsum"], rtol=2e-3, atol=2e-3 * np.abs(want["hsum"]).max())
    assert got["score"].shape == (B, T, 1)
    np.testing.assert_allclose(got["score"], want["score"], rtol=2e-3, atol=2e-3 * np.abs(want["score"]).max())
    assert got["att"].shape == (B, D3)
    np.testing.assert_allclose(got["att"], want["att"], rtol=2e-3, atol=2e-3 * np.abs(want["att"]).max())
    assert got["prob"].shape == (B, 2)
    np.testing.assert_allclose(got["prob"], want["prob"], rtol=2e-3, atol=2e-3)
    # the same model with Gemm+Dice folding switched off gives the same probabilities at that tolerance
    import os
    os.environ["BLAZE_NO_FUSION"] = "1"
    try:
        pm2, _ = din_model.build_manager(cfg, tables, weights, np.float16)
        p2 = pm2.create_predictor(1, 0)
        din_model.feed(p2, inputs, batch, np.float16)
        p2.forward()
        np.testing.assert_allclose(p2.output_asnumpy("prob").astype(np.float32), want["prob"], rtol=2e-3, atol=2e-3)
    finally:
        del os.environ["BLAZE_NO_FUSION"]


def test_attention_unit_assembled_by_the_concat_equals_the_separate_operators():
    """The DIN graph's BroadcastTo / Sub / Mul feeding Concat(axis 2): by default the Concat computes those pieces
    itself in one launch and the three operators never run; with fuse_concat_pieces: 0 each runs and the Concat copies.
    Same bits in the assembled tensor and in the probabilities, also after the batch shrinks and grows again."""
    import json
    import torch
    import din_model
    cfg = din_model.Config3(batch=96, rows=5000, T=20)
    small = din_model.Config3(batch=17, rows=5000, T=20)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=5), cfg.batch_inputs(seed_offset=9)]
    outs = {}
    for fuse in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("att_in", ),
                                             net_args={"fuse_concat_pieces": fuse, "fuse_weighted_pool": 0})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append((p.output_asnumpy("att_in").copy(), p.output_asnumpy("prob").copy()))
        ran = {e["name"].split(":")[0] for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0}
        assert ("BroadcastTo" in ran) == (fuse == 0) and ("Sub" in ran) == (fuse == 0), ran
        assert "Mul" in ran  # Mul(score, mask) is nobody's concat piece
        outs[fuse] = got
    torch.cuda.synchronize()
    D3 = 3 * cfg.dim
    for (a1, p1), (a0, p0), b in zip(outs[1], outs[0], (96, 17, 96)):
        assert a1.shape == (b, cfg.T, 4 * D3) and a1.any()
        assert np.array_equal(a1.view(np.uint16), a0.view(np.uint16))
        assert np.array_equal(p1, p0)
        q, k = a1[:, :, :D3].astype(np.float32), a1[:, :, D3:2 * D3].astype(np.float32)
        assert np.array_equal(a1[:, :, 2 * D3:3 * D3], (q - k).astype(np.float16))
        assert np.array_equal(a1[:, :, 3 * D3:], (q * k).astype(np.float16))


def test_attention_tail_in_one_launch_equals_the_separate_operators():
    """Mul(score, mask) -> MatMul(transA) and ReduceSum(his, axis 1): by default the MatMul runs all three as one launch
    (bz_weighted_pool) and the Mul and the ReduceSum never run; with fuse_weighted_pool: 0 each runs.  Same bits in the
    attention vector, the history sum and the probabilities, also after the batch shrinks and grows again."""
    import json
    import torch
    import din_model
    cfg = din_model.Config3(batch=96, rows=5000, T=20)
    small = din_model.Config3(batch=17, rows=5000, T=20)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=5), cfg.batch_inputs(seed_offset=9)]
    outs = {}
    for fuse in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("att", "hsum"),
                                             net_args={"fuse_weighted_pool": fuse})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append(tuple(p.output_asnumpy(n).copy() for n in ("att", "hsum", "prob")))
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        ran = {e["name"].split(":")[0] for e in ev}
        assert ("ReduceSum" in ran) == (fuse == 0) and ("Mul" in ran) == (fuse == 0), ran
        assert [e["args"]["launches"] for e in ev if e["name"].startswith("MatMul:")] == [1]
        outs[fuse] = got
    torch.cuda.synchronize()
    for one, sep, b in zip(outs[1], outs[0], (96, 17, 96)):
        assert one[0].shape == (b, 3 * cfg.dim) and one[0].any() and one[1].any()
        for x1, x0 in zip(one, sep):
            assert np.array_equal(x1.view(np.uint16 if x1.dtype == np.float16 else np.uint32),
                                  x0.view(np.uint16 if x0.dtype == np.float16 else np.uint32))


def test_attention_input_computed_by_its_first_layer_equals_the_separate_operators():
    """Concat([q, k, q-k, q*k]) -> Gemm + Dice: by default the Gemm computes the Concat's rows while it loads them
    (bz_fc_desc.a_pieces) and the Concat never runs; with fuse_concat_into_fc: 0 the tensor is stored and read back.  The
    first attention layer's output agrees to a rounding of the tensor type (another order of the K sum), the
    probabilities to 2e-3, also after the batch shrinks and grows again."""
    import json
    import torch
    import din_model
    cfg = din_model.Config3(batch=96, rows=5000, T=20)
    small = din_model.Config3(batch=17, rows=5000, T=20)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=5), cfg.batch_inputs(seed_offset=9)]
    outs = {}
    for fuse in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("att0_y", ),
                                             net_args={"fuse_concat_into_fc": fuse})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append((p.output_asnumpy("att0_y").astype(np.float32), p.output_asnumpy("prob").copy()))
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        ran = [e["name"] for e in ev]
        assert ("Concat:concat_att_in" in ran) == (fuse == 0), ran
        assert [e["args"]["launches"] for e in ev if e["name"] == "Gemm:gemm_att0_g"] == [1]
        outs[fuse] = got
    torch.cuda.synchronize()
    for (y1, p1), (y0, p0), b in zip(outs[1], outs[0], (96, 17, 96)):
        assert y1.shape == (b, cfg.T, 80) and y1.any()
        np.testing.assert_allclose(y1, y0, rtol=2e-3, atol=2e-3 * np.abs(y0).max())
        np.testing.assert_allclose(p1, p0, rtol=2e-3, atol=2e-3)


def test_attention_mlp_in_one_launch_equals_layer_by_layer():
    """Gemm+Dice (on the Concat it computes itself) -> Gemm+Dice -> Gemm: by default one launch (bz_fc_desc.next + head); with
    chain_narrow_fcs: 0 the second Gemm runs on its own (hosting the third).  Scores agree to the roundings of the tensor
    type, probabilities to 2e-3, also after the batch shrinks and grows again."""
    import json
    import torch
    import din_model
    cfg = din_model.Config3(batch=96, rows=5000, T=20)
    small = din_model.Config3(batch=17, rows=5000, T=20)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=5), cfg.batch_inputs(seed_offset=9)]
    outs = {}
    for chain in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("score", ), net_args={"chain_narrow_fcs": chain})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append((p.output_asnumpy("score").astype(np.float32), p.output_asnumpy("prob").copy()))
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        ran = [e["name"] for e in ev]
        assert ("Gemm:gemm_att1_g" in ran) == (chain == 0), ran
        assert [e["args"]["launches"] for e in ev if e["name"] == "Gemm:gemm_att0_g"] == [1]
        outs[chain] = got
    torch.cuda.synchronize()
    for (s1, p1), (s0, p0), b in zip(outs[1], outs[0], (96, 17, 96)):
        assert s1.shape == (b, cfg.T, 1) and s1.any()
        np.testing.assert_allclose(s1, s0, rtol=0, atol=4e-3 * max(1.0, float(np.abs(s0).max())))
        np.testing.assert_allclose(p1, p0, rtol=2e-3, atol=2e-3)


def test_history_blocks_written_into_their_concat_equal_the_copy():
    """Embedding kAssign blocks [batch, T * D] -> Reshape [batch, T, D] -> Concat(axis 2): the Embedding writes each block at
    its columns of the Concat's output (interleave_assign_blocks, on by default) and neither the Reshapes nor the Concat
    run; with the switch off the Concat copies.  Same bits either way, also when the batch changes between forwards."""
    import json
    import din_model
    cfg = din_model.Config3(batch=64, rows=3000, T=12)
    small = din_model.Config3(batch=9, rows=3000, T=12)
    big = din_model.Config3(batch=130, rows=3000, T=12)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=1), big.batch_inputs(seed_offset=2), cfg.batch_inputs(seed_offset=3)]
    outs = {}
    for alias in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("his", "hsum", "att"), net_args={"interleave_assign_blocks": alias})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append({k: p.output_asnumpy(k).copy() for k in ("his", "hsum", "att", "prob")})
        ran = [e["name"] for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        assert ("Concat:concat_his" in ran) == (alias == 0), ran
        outs[alias] = got
    for g1, g0, b in zip(outs[1], outs[0], (64, 9, 130, 64)):
        assert g1["his"].shape == (b, cfg.T, 3 * cfg.dim) and g1["his"].any()
        for k in g1:
            np.testing.assert_array_equal(g1[k], g0[k], err_msg=k)
    # a reshaped block that is also an output of the net keeps its own memory: the rewrite does not apply
    mid = "his3_" + din_model.KINDS[0]
    pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("his", mid))
    p = pm.create_predictor(1, 0)
    p.register_observers(["profile"])
    din_model.feed(p, inputs, batches[0], np.float16)
    p.forward()
    ran = [e["name"] for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
    assert "Concat:concat_his" in ran, ran
    np.testing.assert_array_equal(p.output_asnumpy("his"), outs[1][0]["his"])
    np.testing.assert_array_equal(p.output_asnumpy(mid), outs[1][0]["his"][:, :, :cfg.dim])


def test_main_input_concat_written_by_the_attention_tail():
    """Mul -> MatMul(transA) -> Reshape, ReduceSum, Concat(axis 1)[q, hsum, att]: the attention tail's one launch also
    writes the Concat's output - its own two results at their columns, the target block copied alongside
    (fuse_concat_into_weighted_pool, on by default) - and neither the Reshape nor the Concat runs; with the switch off the
    Concat copies.  Same bits either way, also when the batch changes between forwards; a tail result that is an output
    of the net keeps its own memory and the Concat runs."""
    import json
    import din_model
    cfg = din_model.Config3(batch=64, rows=3000, T=12)
    small = din_model.Config3(batch=9, rows=3000, T=12)
    big = din_model.Config3(batch=130, rows=3000, T=12)
    tables, weights = cfg.tables(), cfg.weights()
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=1), big.batch_inputs(seed_offset=2), cfg.batch_inputs(seed_offset=3)]
    outs = {}
    for fuse in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("main_in", "q"),
                                             net_args={"fuse_concat_into_weighted_pool": fuse})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for b in batches:
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            got.append({k: p.output_asnumpy(k).copy() for k in ("main_in", "q", "prob")})
        ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
        ran = [e["name"].split(":")[0] for e in ev]
        assert ("Concat" in ran) == (fuse == 0), ran
        assert [e["args"]["launches"] for e in ev if e["name"].split(":")[0] == "MatMul"] == [1]
        outs[fuse] = got
    D3 = 3 * cfg.dim
    for g1, g0, b in zip(outs[1], outs[0], (64, 9, 130, 64)):
        assert g1["main_in"].shape == (b, 3 * D3) and g1["main_in"][:, D3:].any()
        np.testing.assert_array_equal(g1["main_in"][:, :D3], g1["q"])
        for k in g1:
            np.testing.assert_array_equal(g1[k], g0[k], err_msg=k)
    # the tail's results as outputs of the net: the rewrite does not apply, everything is stored
    pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("main_in", "hsum", "att"))
    p = pm.create_predictor(1, 0)
    p.register_observers(["profile"])
    din_model.feed(p, inputs, batches[0], np.float16)
    p.forward()
    ran = [e["name"].split(":")[0] for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0]
    assert "Concat" in ran, ran
    np.testing.assert_array_equal(p.output_asnumpy("main_in"), outs[1][0]["main_in"])
    np.testing.assert_array_equal(p.output_asnumpy("hsum"), outs[1][0]["main_in"][:, D3:2 * D3])
    np.testing.assert_array_equal(p.output_asnumpy("att"), outs[1][0]["main_in"][:, 2 * D3:])


def test_sibling_embedding_operators_share_one_launch():
    """DIN's two Embedding operators (target item: ksum of one id a sample; history: kAssign) read only inputs of the net:
    the first runs the second (merge_sibling_embeddings, on by default) and both are looked up in one pooling launch,
    because the target's lookups are light; with three ids a sample in the target's groups they are not, and the two
    launch one after the other.  Same bits as two separate operators in every case, also when the batch changes."""
    import json
    import din_model
    cfg = din_model.Config3(batch=64, rows=3000, T=12)
    small = din_model.Config3(batch=9, rows=3000, T=12)
    batches = [cfg.batch_inputs(), small.batch_inputs(seed_offset=1), cfg.batch_inputs(seed_offset=2)]
    heavy = dict(batches[2])
    for k in din_model.KINDS:  # three ids a sample for the target item: more than "light"
        heavy[k + ".ids"] = np.concatenate([batches[2][k + ".ids"], batches[0][k + ".ids"], batches[2][k + ".ids"][::-1]]).reshape(3, -1).T.reshape(-1).copy()
        heavy[k + ".values"] = np.ones(3 * cfg.batch, np.float32)
        heavy[k + ".segments"] = np.full(cfg.batch, 3, np.int32)
    batches.append(heavy)
    tables, weights = cfg.tables(), cfg.weights()
    outs = {}
    for merge in (1, 0):
        pm, inputs = din_model.build_manager(cfg, tables, weights, np.float16, expose=("q", "his"), net_args={"merge_sibling_embeddings": merge})
        p = pm.create_predictor(1, 0)
        p.register_observers(["profile"])
        got = []
        for i, b in enumerate(batches):
            din_model.feed(p, inputs, b, np.float16)
            p.forward()
            ev = [e for e in json.loads(p.dump_observers()["profile"])["traceEvents"] if e["dur"] > 0 and e["name"].split(":")[0] == "Embedding"]
            launches = [e["args"]["launches"] for e in ev]
            assert launches == ([1, 1] if merge == 0 else ([2] if i == 3 else [1])), (merge, i, launches)
            got.append({k: p.output_asnumpy(k).copy() for k in ("q", "his", "prob")})
        outs[merge] = got
    for g1, g0 in zip(outs[1], outs[0]):
        assert g1["q"].any() and g1["his"].any()
        for k in g1:
            np.testing.assert_array_equal(g1[k], g0[k], err_msg=k)

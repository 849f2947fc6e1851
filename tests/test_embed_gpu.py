"""GPU parity of the Embedding path (bz_segments_to_offsets*, bz_embed_pool) against the CPU oracle.

Bars: offsets bit-exact (int64); pooled fp32 output bit-exact (the kernel sums in the
reference's order with unfused multiply/add; the contract in the benchmark spec is rel 1e-5);
fp16 output equal to the oracle's fp32 result rounded to nearest even (contract: 2e-3).
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


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 2047, 2048, 2049, 8192, 100003])
def test_segments_to_offsets_bit_exact(bz, oracle, n):
    import torch
    rng = np.random.default_rng(n)
    seg = rng.integers(0, 70, size=n).astype(np.int32)
    print("case n=%d" % n, flush=True)
    off = bz.segments_to_offsets(_dev(seg))
    torch.cuda.synchronize()
    assert np.array_equal(off.cpu().numpy(), oracle.segments_to_offsets(seg))


def test_segments_to_offsets_no_32bit_wrap(bz, oracle):
    import torch
    seg = np.full(5, 2**31 - 1, np.int32)
    off = bz.segments_to_offsets(_dev(seg))
    torch.cuda.synchronize()
    assert np.array_equal(off.cpu().numpy(), oracle.segments_to_offsets(seg))


def _run_gpu(bz, tables_np, specs, inputs, batch, out_np_dtype, strides_cols, fused_scan=True):
    """specs: list of (table index|None, udf, tdir, tnum, dim); one block, items packed at given cols."""
    import torch
    stride, cols = strides_cols
    out = torch.full((batch, stride), float("nan"), dtype=torch.float32 if out_np_dtype == np.float32 else torch.float16,
                     device="cuda")
    dts = [None if t is None else bz.DeviceTable(t["data"], scale=t.get("scale"), keys=t.get("keys")) for t in tables_np]
    items = []
    for (ti, udf, tdir, tnum, dim), col, (ids, vals, seg) in zip(specs, cols, inputs):
        items.append(dict(table=None if ti is None else dts[ti], ids=_dev(ids), values=_dev(vals), segments=_dev(seg),
                          out=out, col=col, udf=udf, trunc_dir=tdir, trunc_num=tnum, dim=dim))
    plan = bz.EmbeddingPlan(items, fused_scan=fused_scan)
    plan.run()
    torch.cuda.synchronize()
    offs = [o.cpu().numpy() for o in plan.offsets]
    if plan.args_eligible():
        # the same launch with the slot records handed over as kernel arguments: the same bits (NaN fill included:
        # the columns of no item stay as they were)
        out2 = torch.full_like(out, float("nan"))
        for it in items:
            it["out"] = out2
        bz.EmbeddingPlan(items, fused_scan=fused_scan).pool_args()
        torch.cuda.synchronize()
        assert np.array_equal(out2.cpu().numpy().view(np.uint8), out.cpu().numpy().view(np.uint8)), "kernel-argument form differs"
    return out.cpu().numpy(), offs, plan.launch.variant


def _run_oracle(oracle, tables_np, specs, inputs, batch, strides_cols):
    stride, cols = strides_cols
    out = np.full((batch, stride), np.nan, np.float32)
    for (ti, udf, tdir, tnum, dim), col, (ids, vals, seg) in zip(specs, cols, inputs):
        width = dim * tnum if udf == 2 else dim
        if ti is None:
            out[:, col:col + width] = 0  # Setup memsets the block; an unknown table writes nothing
            continue
        t = tables_np[ti]
        table = oracle.Table(t["data"], scale=t.get("scale"), keys=t.get("keys"))
        oracle.embed_get(table, ids, vals, seg, [(udf, tdir, tnum, out, col)])
    return out


def test_reference_qed_kat_on_gpu(bz, oracle):
    """The reference's QuickEmbeddingDict.Get known answers through the device hash path."""
    from test_oracle_pins import CASE1, CASE2, CASE3, CASE4, QED_KEYS, _qed_expected, _qed_inputs
    import torch
    ins = _qed_inputs()
    b1 = torch.full((2, 12), float("nan"), device="cuda")
    b2 = torch.full((2, 24), float("nan"), device="cuda")
    t1 = bz.DeviceTable(np.array([CASE1], np.float32), keys=np.array(QED_KEYS["101"]))
    t2 = bz.DeviceTable(np.array([CASE2], np.float32), keys=np.array(QED_KEYS["102"]))
    t3 = bz.DeviceTable(np.array([CASE3, CASE4], np.float32), keys=np.array(QED_KEYS["104_7"]))
    items = []
    for (fg, t, out, col, udf, tn) in (("101", t1, b1, 0, 0, 0), ("102", t2, b1, 4, 0, 0), ("104_7", t3, b2, 0, 2, 4)):
        ids, vals, seg = ins[fg]
        items.append(dict(table=t, ids=_dev(ids), values=_dev(vals), segments=_dev(seg), out=out, col=col, udf=udf,
                          trunc_dir=0, trunc_num=tn))
    bz.EmbeddingPlan(items).run()
    torch.cuda.synchronize()
    e1, e2 = _qed_expected()
    np.testing.assert_allclose(b1.cpu().numpy(), e1, rtol=5e-7, atol=0)
    np.testing.assert_allclose(b2.cpu().numpy(), e2, rtol=5e-7, atol=0)


def test_reference_embedding_op_kat_on_gpu(bz, kats):
    """embedding_v1.conf (mock puller: every key resolves to a row of ones)."""
    import torch
    from test_oracle_pins import _tensor
    case = kats["embedding_v1"]
    t = case["tensors"]
    b1 = torch.full((2, 12), float("nan"), device="cuda")
    b2 = torch.full((2, 24), float("nan"), device="cuda")
    items = []
    for fg, dim, out, col, udf, tn in (("101", 4, b1, 0, 0, 0), ("102", 8, b1, 4, 0, 0), ("104_7", 6, b2, 0, 2, 4)):
        ids = _tensor(t[fg + ".ids"])
        keys = np.unique(ids)
        table = bz.DeviceTable(np.ones((keys.size, dim), np.float32), keys=keys)
        items.append(dict(table=table, ids=_dev(ids), values=_dev(_tensor(t[fg + ".values"])),
                          segments=_dev(_tensor(t[fg + ".segments"])), out=out, col=col, udf=udf, trunc_dir=0,
                          trunc_num=tn))
    bz.EmbeddingPlan(items).run()
    torch.cuda.synchronize()
    for got, name in ((b1, "block1_values"), (b2, "block2_values")):
        exp = case["expected"][name]
        np.testing.assert_allclose(got.cpu().numpy(), np.array(exp["values"], np.float32).reshape(exp["shape"]), rtol=0,
                                   atol=1e-6)


def _make_table(rng, kind, rows, dim, with_keys):
    t = {}
    if kind == "f32":
        t["data"] = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float32)
    elif kind == "f16":
        t["data"] = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float16)
    else:
        t["data"] = rng.integers(-127, 128, (rows, dim)).astype(np.int8)
        t["scale"] = rng.uniform(1e-3, 1e-2, rows).astype(np.float32)
    if with_keys:
        t["keys"] = np.unique(rng.integers(-2**62, 2**62, size=rows * 2, dtype=np.int64))[:rows]
        assert t["keys"].size == rows
    return t


@pytest.mark.parametrize("kind", ["f32", "f16", "i8"])
@pytest.mark.parametrize("out_dtype", [np.float32, np.float16])
@pytest.mark.parametrize("with_keys", [False, True])
@pytest.mark.parametrize("fused_scan", [True, False])
def test_pooling_random_bit_exact(bz, oracle, kind, out_dtype, with_keys, fused_scan):
    """Ragged segments (incl. empty), absent ids, random values, odd dims and unaligned columns; slots of mixed
    shape and pooling kind go through the generic kernel, with the fused and with the separate scan."""
    seed = sum(map(ord, kind)) * 7 + (13 if out_dtype == np.float16 else 0) + (101 if with_keys else 0)
    rng = np.random.default_rng(seed)
    batch = 333
    dims = [1, 4, 16, 18, 32, 33, 64, 100, 300]
    tables, specs, inputs, cols = [], [], [], []
    col = 1  # odd start column -> unaligned stores
    for i, dim in enumerate(dims):
        rows = int(rng.integers(5, 400))
        tables.append(_make_table(rng, kind, rows, dim, with_keys))
        udf, tdir, tnum = [(0, 0, 0), (1, 0, 0), (2, 0, 3), (2, 1, 4)][i % 4]
        seg = rng.integers(0, 12, batch).astype(np.int32)
        seg[rng.integers(0, batch, 20)] = 0
        nnz = int(seg.sum())
        if with_keys:
            pool = np.concatenate([tables[-1]["keys"], rng.integers(-2**62, 2**62, size=rows // 4 + 1, dtype=np.int64)])
            ids = rng.choice(pool, nnz)
        else:
            ids = rng.integers(-3, rows + 3, nnz)
        vals = rng.standard_normal(nnz).astype(np.float32)
        specs.append((i, udf, tdir, tnum, dim))
        inputs.append((ids.astype(np.int64), vals, seg))
        cols.append(col)
        col += dim * tnum if udf == 2 else dim
    stride = col + 3
    print("case kind=%s out=%s keys=%s seed=%d" % (kind, out_dtype.__name__, with_keys, seed), flush=True)
    got, offs, variant = _run_gpu(bz, tables, specs, inputs, batch, out_dtype, (stride, cols), fused_scan)
    assert variant == 0
    want = _run_oracle(oracle, tables, specs, inputs, batch, (stride, cols))
    assert len(offs) == (0 if fused_scan else len(inputs))
    for off, (_, _, seg) in zip(offs, inputs):
        assert np.array_equal(off, oracle.segments_to_offsets(seg))
    written = ~np.isnan(want)
    assert np.array_equal(np.isnan(got.astype(np.float32)), ~written), "kernel wrote outside its items' columns"
    if out_dtype == np.float32:
        assert np.array_equal(_bits(got)[written], _bits(want)[written])
    else:
        with np.errstate(invalid="ignore"):
            want16 = want.astype(np.float16)
        assert np.array_equal(_bits(got)[written], _bits(want16)[written])


@pytest.mark.parametrize("kind,out_dtype", [("f16", np.float16), ("f32", np.float32), ("i8", np.float16)])
@pytest.mark.parametrize("tdir", [0, 1])
def test_assign_items_share_the_rows_of_one_history_tensor(bz, oracle, kind, out_dtype, tdir):
    """bz_embed_slot.assign_pitch: three kAssign items of dims 18, 7 and 32 write their positions at columns 0, 18 and 25
    of one [batch, T, 57 + 2] tensor (out_stride = T * pitch, assign_pitch = pitch).  Bit-equal to the oracle's contiguous
    [batch, T * dim] blocks moved there; the two spare columns of every position stay untouched."""
    import torch
    rng = np.random.default_rng(77 + tdir + len(kind))
    batch, T = 201, 9
    dims = [18, 7, 32]
    pitch = sum(dims) + 2
    tdt = torch.float32 if out_dtype == np.float32 else torch.float16
    out = torch.full((batch, T * pitch), float("nan"), dtype=tdt, device="cuda")
    want = np.full((batch, T, pitch), np.nan, np.float32)
    items, col = [], 0
    keep = []
    for dim in dims:
        rows = int(rng.integers(30, 200))
        t = _make_table(rng, kind, rows, dim, False)
        seg = rng.integers(0, 2 * T, batch).astype(np.int32)
        seg[rng.integers(0, batch, 15)] = 0
        nnz = int(seg.sum())
        ids = rng.integers(-3, rows + 3, nnz).astype(np.int64)
        vals = rng.standard_normal(nnz).astype(np.float32)
        dt = bz.DeviceTable(t["data"], scale=t.get("scale"))
        keep.append(dt)
        items.append(dict(table=dt, ids=_dev(ids), values=_dev(vals), segments=_dev(seg), out=out, col=col, udf=2,
                          trunc_dir=tdir, trunc_num=T, assign_pitch=pitch))
        block = np.full((batch, T * dim), np.nan, np.float32)
        oracle.embed_get(oracle.Table(t["data"], scale=t.get("scale")), ids, vals, seg, [(2, tdir, T, block, 0)])
        want[:, :, col:col + dim] = block.reshape(batch, T, dim)
        col += dim
    print("assign_pitch kind=%s out=%s dir=%d" % (kind, out_dtype.__name__, tdir), flush=True)
    for fused in (True, False):
        out.fill_(float("nan"))
        bz.EmbeddingPlan(items, fused_scan=fused).run()
        torch.cuda.synchronize()
        got = out.cpu().numpy().reshape(batch, T, pitch)
        assert np.isnan(got[:, :, col:].astype(np.float32)).all(), "wrote outside the items' columns"
        w = want[:, :, :col]
        assert not np.isnan(w).any()
        assert np.array_equal(_bits(got[:, :, :col]), _bits(w.astype(out_dtype)))
    # an item whose table is unknown zero-fills its own columns of every position and nothing else
    out.fill_(float("nan"))
    unknown = [dict(items[0]), dict(items[1], table=None, dim=dims[1]), dict(items[2])]
    bz.EmbeddingPlan(unknown).run()
    torch.cuda.synchronize()
    got = out.cpu().numpy().reshape(batch, T, pitch)
    w = want[:, :, :col].copy()
    w[:, :, dims[0]:dims[0] + dims[1]] = 0
    assert np.isnan(got[:, :, col:].astype(np.float32)).all()
    assert np.array_equal(_bits(got[:, :, :col]), _bits(w.astype(out_dtype)))
    # a pitch below the item's dim, or on a pooled item, is refused
    bad = dict(items[0], assign_pitch=dims[0] - 1)
    with pytest.raises(RuntimeError, match="assign_pitch"):
        bz.EmbeddingPlan([bad])
    bad = dict(items[0], udf=0, assign_pitch=pitch)
    with pytest.raises(RuntimeError, match="assign_pitch"):
        bz.EmbeddingPlan([bad])


SPECIALISED = [("f32", 4, 1), ("f32", 16, 4), ("f32", 30, 8), ("f32", 64, 16), ("f32", 128, 32), ("f32", 250, 64),
               ("f16", 8, 1), ("f16", 16, 2), ("f16", 18, 4), ("f16", 32, 4), ("f16", 64, 8), ("f16", 100, 16),
               ("f16", 200, 32), ("f16", 512, 64), ("i8", 16, 1), ("i8", 64, 4), ("i8", 100, 8), ("i8", 1000, 64)]


@pytest.mark.parametrize("kind,dim,lpr", SPECIALISED)
@pytest.mark.parametrize("with_keys", [False, True])
def test_pooling_specialised_kernels_bit_exact(bz, oracle, kind, dim, lpr, with_keys):
    """Slots of one shape, ksum/kavg only: every (table dtype, lanes-per-row) instance of the specialised kernel,
    segments longer than one 16-id step, empty segments, absent ids, fp32 and fp16 outputs."""
    rng = np.random.default_rng(dim * 31 + lpr + (7 if with_keys else 0))
    batch = 300
    for out_dtype in (np.float32, np.float16):
        tables, specs, inputs, cols = [], [], [], []
        col = 0
        for i in range(3):
            rows = int(rng.integers(20, 300))
            tables.append(_make_table(rng, kind, rows, dim, with_keys))
            seg = rng.integers(0, 40, batch).astype(np.int32)
            seg[rng.integers(0, batch, 30)] = 0
            nnz = int(seg.sum())
            if with_keys:
                pool = np.concatenate([tables[-1]["keys"], rng.integers(-2**62, 2**62, size=rows // 4 + 1, dtype=np.int64)])
                ids = rng.choice(pool, nnz)
            else:
                ids = rng.integers(-3, rows + 3, nnz)
            specs.append((i, i % 2, 0, 0, dim))
            inputs.append((ids.astype(np.int64), rng.standard_normal(nnz).astype(np.float32), seg))
            cols.append(col)
            col += dim
        print("case kind=%s dim=%d lpr=%d keys=%s out=%s" % (kind, dim, lpr, with_keys, out_dtype.__name__), flush=True)
        for fused in (True, False):
            got, offs, variant = _run_gpu(bz, tables, specs, inputs, batch, out_dtype, (col, cols), fused)
            code = {"f32": bz.F32, "f16": bz.F16, "i8": bz.I8}[kind]
            assert variant == (code << 8 | lpr), "expected the specialised kernel, got variant %#x" % variant
            want = _run_oracle(oracle, tables, specs, inputs, batch, (col, cols))
            if out_dtype == np.float16:
                want = want.astype(np.float16)
            assert np.array_equal(_bits(got), _bits(want))


def test_unknown_table_and_empty_batch(bz, oracle):
    rng = np.random.default_rng(9)
    batch = 70
    t = _make_table(rng, "f32", 10, 8, False)
    seg = rng.integers(0, 4, batch).astype(np.int32)
    nnz = int(seg.sum())
    ins = (rng.integers(0, 10, nnz).astype(np.int64), np.ones(nnz, np.float32), seg)
    specs = [(None, 0, 0, 0, 8), (0, 0, 0, 0, 8), (None, 2, 0, 3, 8)]
    cols = [0, 8, 16]
    got, _, _ = _run_gpu(bz, [t], specs, [ins] * 3, batch, np.float32, (40, cols))
    want = _run_oracle(oracle, [t], specs, [ins] * 3, batch, (40, cols))
    assert np.array_equal(_bits(got), _bits(want))


def _config2_inputs(rng, batch, slots, rows):
    """Config-2 shaped ids: length Poisson(8) clipped to [1,64], Zipf(1.1) ranks scattered over the rows."""
    out = []
    for _ in range(slots):
        seg = np.clip(rng.poisson(8, batch), 1, 64).astype(np.int32)
        nnz = int(seg.sum())
        ranks = rng.zipf(1.1, nnz * 2)
        ranks = ranks[ranks <= rows][:nnz]
        while ranks.size < nnz:
            more = rng.zipf(1.1, nnz)
            ranks = np.concatenate([ranks, more[more <= rows]])[:nnz]
        ids = ((ranks.astype(np.int64) - 1) * 2654435761) % rows
        out.append((ids, np.ones(nnz, np.float32), seg))
    return out


def test_config2_full_size(bz, oracle):
    """26 slots x [1M,32] fp16, batch 2048, ksum into a [2048, 896] fp16 block at column 64 (dense features first)."""
    import torch
    rng = np.random.default_rng(20240613)
    batch, slots, rows, dim = 2048, 26, 1_000_000, 32
    inputs = _config2_inputs(rng, batch, slots, rows)
    out = torch.zeros((batch, 896), dtype=torch.float16, device="cuda")
    items, tables = [], []
    g = torch.Generator(device="cuda").manual_seed(7)
    for s in range(slots):
        data = (torch.randn((rows, dim), generator=g, device="cuda") * 0.01).to(torch.float16)
        tables.append(data)
        ids, vals, seg = inputs[s]
        items.append(dict(table=bz.DeviceTable(data), ids=_dev(ids), values=_dev(vals), segments=_dev(seg), out=out,
                          col=64 + s * dim, udf=0))
    plan = bz.EmbeddingPlan(items)
    assert plan.launch.variant == (bz.F16 << 8 | 4) and plan.launch.fused_scan == 1
    plan.run()
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert not got[:, :64].any(), "dense-feature columns must be left alone"
    for s in (0, 7, 25):  # three slots checked in full against the oracle (touched rows only are copied to the host)
        ids, vals, seg = inputs[s]
        uniq, inv = np.unique(ids, return_inverse=True)
        sub = tables[s][torch.from_numpy(uniq).cuda()].cpu().numpy()
        want = np.zeros((batch, dim), np.float32)
        oracle.embed_get(oracle.Table(sub), inv, vals, seg, [(0, 0, 0, want, 0)])
        assert np.array_equal(_bits(got[:, 64 + s * dim:64 + (s + 1) * dim]), _bits(want.astype(np.float16)))
    plan2 = bz.EmbeddingPlan(items, fused_scan=False)  # separate scan launch: offsets are observable and bit-exact
    out.zero_()
    plan2.run()
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), got)
    for s in range(slots):
        assert np.array_equal(plan2.offsets[s].cpu().numpy(), oracle.segments_to_offsets(inputs[s][2]))


def _lengths_case(rng, kind, batch):
    if kind == "poisson8":
        return np.clip(rng.poisson(8, batch), 0, 64).astype(np.int32)
    if kind == "mostly_empty":      # far more owned segments than ids: the reduction runs in rounds
        return (rng.random(batch) < 0.03).astype(np.int32) * rng.integers(1, 4, batch).astype(np.int32)
    if kind == "all_empty":
        return np.zeros(batch, np.int32)
    if kind == "giants":            # segments far longer than what a workgroup stages behind its range
        seg = rng.integers(0, 3, batch).astype(np.int32)
        seg[rng.choice(batch, 6, replace=False)] = rng.integers(700, 2600, 6)
        return seg
    if kind == "ones":
        return np.ones(batch, np.int32)
    if kind == "empty_ends":
        seg = rng.integers(1, 20, batch).astype(np.int32)
        seg[:37] = 0
        seg[-41:] = 0
        return seg
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["poisson8", "mostly_empty", "all_empty", "giants", "ones", "empty_ends"])
@pytest.mark.parametrize("tdtype,dim,batch", [("f16", 32, 2048), ("f16", 64, 8192), ("f32", 16, 131), ("i8", 64, 4096),
                                              ("f16", 18, 1023), ("f32", 3, 4100), ("f16", 128, 600)])
def test_pooling_segment_shapes_that_stress_the_bookkeeping(bz, oracle, kind, tdtype, dim, batch):
    """Segment shapes that stress the offset bookkeeping of the pooling kernels: very long segments among short ones,
    runs of empty segments (at the ends too), no ids at all, batches that are not multiples of the workgroup's share,
    hashed keys, absent ids, int8 rows with the scale inside the row.  ksum and kavg in one launch, with the fused scan
    and with offsets scanned first; fp32 block bit-exact against the oracle."""
    import torch
    rng = np.random.default_rng(abs(hash((kind, tdtype, dim, batch))) % (2**31))
    rows = 3000
    slots = 3
    if tdtype == "i8":
        data = [rng.integers(-127, 128, (rows, dim)).astype(np.int8) for _ in range(slots)]
        scale = [rng.uniform(1e-3, 1e-2, rows).astype(np.float32) for _ in range(slots)]
    else:
        npdt = np.float16 if tdtype == "f16" else np.float32
        data = [(rng.standard_normal((rows, dim)) * 0.1).astype(npdt) for _ in range(slots)]
        scale = [None] * slots
    keys = [None, np.unique(rng.integers(-2**50, 2**50, rows * 2, dtype=np.int64))[:rows], None]
    out = torch.full((batch, slots * dim), float("nan"), dtype=torch.float32, device="cuda")
    want = np.full((batch, slots * dim), np.nan, np.float32)
    items, keep = [], []
    for s in range(slots):
        seg = _lengths_case(rng, kind, batch)
        nnz = int(seg.sum())
        if keys[s] is None:
            ids = rng.integers(-2, rows + 2, nnz).astype(np.int64)           # a few ids outside the table
        else:
            ids = rng.choice(np.concatenate([keys[s], np.array([7, -7], np.int64)]), nnz).astype(np.int64)
        vals = rng.uniform(0.5, 1.5, nnz).astype(np.float32)
        t = bz.DeviceTable(data[s], scale=scale[s], keys=keys[s])
        d = [_dev(ids), _dev(vals), _dev(seg)]
        keep.append((t, d))
        udf = bz.AVG if s == 1 else bz.SUM
        items.append(dict(table=t, ids=d[0], values=d[1], segments=d[2], out=out, col=s * dim, udf=udf))
        oracle.embed_get(oracle.Table(data[s], scale=scale[s], keys=keys[s]), ids, vals, seg, [(udf, 0, 0, want, s * dim)])
    plan = bz.EmbeddingPlan(items, fused_scan=True)
    print("segment-shape case %s %s dim=%d batch=%d: %d workgroups" % (kind, tdtype, dim, batch, plan.launch.total_wg), flush=True)
    plan.run()
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # ... with the slot records handed over as kernel arguments (bz_embed_pool_args)
    assert plan.args_eligible()
    out3 = torch.full_like(out, float("nan"))
    for it in items:
        it["out"] = out3
    bz.EmbeddingPlan(items, fused_scan=True).pool_args()
    torch.cuda.synchronize()
    assert np.array_equal(out3.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # ... and from offsets scanned in a launch of their own
    out2 = torch.full_like(out, float("nan"))
    for it in items:
        it["out"] = out2
    plan2 = bz.EmbeddingPlan(items, fused_scan=False)
    plan2.run()
    torch.cuda.synchronize()
    assert np.array_equal(out2.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # (records with offsets of their own are not for the kernel-argument form: refused, nothing launched)
    assert not plan2.args_eligible()
    with pytest.raises(RuntimeError, match="bz_embed_pool_args"):
        plan2.pool_args()


def test_pooling_unaligned_counts_and_trailing_empty_segments(bz, oracle):
    """The counts array at an address that is not a multiple of 16, and batches whose ids end long before the samples
    do (only empty segments behind them)."""
    import torch
    rng = np.random.default_rng(99)
    rows, dim, batch = 2000, 32, 515
    data = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float16)
    t = bz.DeviceTable(data)
    for total in (512, 1024, 1536):
        seg = np.zeros(batch, np.int32)
        seg[:total // 4] = 4           # exactly `total` ids, then only empty segments
        ids = rng.integers(0, rows, total).astype(np.int64)
        vals = rng.uniform(0.5, 1.5, total).astype(np.float32)
        holder = torch.zeros(batch + 3, dtype=torch.int32, device="cuda")
        d_seg = holder[3:]             # 12 bytes past a 16-byte boundary
        d_seg.copy_(torch.from_numpy(seg))
        assert d_seg.data_ptr() % 16 == 12
        out = torch.full((batch, dim), float("nan"), dtype=torch.float32, device="cuda")
        d_ids, d_vals = _dev(ids), _dev(vals)
        plan = bz.EmbeddingPlan([dict(table=t, ids=d_ids, values=d_vals, segments=d_seg, out=out, udf=bz.SUM)])
        plan.run()
        torch.cuda.synchronize()
        want = np.full((batch, dim), np.nan, np.float32)
        oracle.embed_get(oracle.Table(data), ids, vals, seg, [(0, 0, 0, want, 0)])
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_device_fill_matches_the_host_generator_bit_for_bit(bz):
    """csrc/synth/philox_fill.hip (tables too large to come from the host) against philox.py on the same (seed, stream,
    index): normal fp32 / fp16, int8, uniform fp32; ranges that start and end inside a call's four words."""
    import torch
    import philox
    st = philox.Stream(12, seed=philox.SEED + 99)
    for kind, dt, a, b in ((philox.KIND_NORMAL_F32, torch.float32, 0.01, 0.0), (philox.KIND_NORMAL_F16, torch.float16, 0.1, 0.0),
                           (philox.KIND_INT8, torch.int8, 1.0, 0.0), (philox.KIND_UNIFORM_F32, torch.float32, 1e-3, 1e-2)):
        for first, n in ((0, 4096), (1, 1), (3, 7), (5, 100003), ((1 << 34) + 2, 513)):
            print("device fill kind %d first %d n %d" % (kind, first, n), flush=True)
            t = torch.empty(n + 2, dtype=dt, device="cuda")
            t.fill_(77)
            philox.fill(t[1:n + 1], kind, st, first, a, b)
            torch.cuda.synchronize()
            got = t.cpu().numpy()
            want = philox.host(kind, st, n, first, a, b)
            assert got[0] == 77 and got[-1] == 77  # nothing outside the range is written
            assert got.dtype == want.dtype and np.array_equal(got[1:-1].view(np.uint8), want.view(np.uint8))
    m = philox.tensor((1000, 18), philox.KIND_NORMAL_F16, st, "cuda", 0.1)
    assert np.array_equal(m.cpu().numpy()[[999, 0]], philox.host_rows(philox.KIND_NORMAL_F16, st, [999, 0], 18, 0.1))


def test_table_of_more_than_2_to_24_rows_takes_the_plain_load_path(bz, oracle):
    """The specialised kernel reads fp32 / fp16 tables of up to 2^24 rows through a buffer resource and larger ones with
    plain loads under a branch: a table of 17 M rows (ids on both sides of 2^24, some outside the table) against the
    oracle, bit for bit, next to a small table in the same launch."""
    rng = np.random.default_rng(2024)
    rows, dim, batch = 17_000_000, 4, 300
    big = {"data": (rng.standard_normal((rows, dim)) * 0.1).astype(np.float32)}
    small = {"data": (rng.standard_normal((1000, dim)) * 0.1).astype(np.float32)}
    specs, inputs, cols = [], [], []
    col = 0
    for ti, udf, n_rows in ((0, 0, rows), (1, 1, 1000), (0, 1, rows)):
        seg = rng.integers(0, 9, batch).astype(np.int32)
        nnz = int(seg.sum())
        ids = rng.integers(-2, n_rows + 2, nnz)
        ids[::5] = rng.integers(max(0, n_rows - 2000), n_rows, ids[::5].size)  # the table's last rows (beyond 2^24 for the big one)
        specs.append((ti, udf, 0, 0, dim))
        inputs.append((ids.astype(np.int64), rng.standard_normal(nnz).astype(np.float32), seg))
        cols.append(col)
        col += dim
    print("table of %d rows" % rows, flush=True)
    got, _, variant = _run_gpu(bz, [big, small], specs, inputs, batch, np.float32, (col, cols))
    assert variant != 0  # one row shape, ksum / kavg: the specialised kernel
    want = _run_oracle(oracle, [big, small], specs, inputs, batch, (col, cols))
    assert np.array_equal(_bits(got), _bits(want))

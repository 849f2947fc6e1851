"""Pins of the CPU oracle (no GPU).

Each oracle function is held against evidence that does not come from the oracle:
the reference's own known-answer data (tests/golden/reference_kats.json, plus the
numbers of its store unit tests restated below as data), the reference's own store
object code where oracle/_ref builds, numpy's independent float16 / float64
arithmetic, and closed forms.
"""
import numpy as np
import pytest

ATOL_KAT = 1e-6  # the reference's strict comparator, test/operator/operator_test_common.h:68


def _tensor(t):
    dt = {1: np.float32, 2: np.int32, 10: np.int64}[t["dtype"]]
    return np.array(t["values"], dtype=dt).reshape(t["shape"])


def _run_op(oracle, case):
    op = case["ops"][0]
    ins = [_tensor(case["tensors"][n]) for n in op["inputs"]]
    a = op["args"]
    ty = op["type"]
    if ty == "Gemm":
        return oracle.gemm_op(ins[0], ins[1], ins[2] if len(ins) > 2 else None, bool(a.get("transA", 0)),
                              bool(a.get("transB", 0)), a.get("alpha", 1.0), a.get("beta", 1.0))
    if ty == "FusedParallelGemm":
        return oracle.fused_parallel_gemm_op(ins[0], ins[1], ins[2] if len(ins) > 2 else None, a.get("parallel_num", 2),
                                             bool(a.get("transA", 0)), bool(a.get("transB", 0)), a.get("alpha", 1.0),
                                             a.get("beta", 1.0))
    if ty == "MatMul":
        return oracle.matmul_op(ins[0], ins[1], bool(a.get("transA", 0)), bool(a.get("transB", 0)),
                                bool(a.get("from_deepnet", 0)))
    if ty == "FusedParallelMatMul":
        return oracle.fused_parallel_matmul_op(ins[0], ins[1], a.get("parallel_num", 2), bool(a.get("transA", 0)),
                                               bool(a.get("transB", 0)))
    if ty == "PRelu":
        return oracle.prelu(ins[0], ins[1])
    if ty == "Dice":
        return oracle.dice(ins[0], ins[1], ins[2], ins[3], bool(a.get("nosqrt", 0)))
    if ty == "LeakyRelu":
        return oracle.leaky_relu(ins[0], a.get("alpha", 0.0))
    if ty == "Sigmoid":
        return oracle.sigmoid(ins[0])
    if ty == "Softmax":
        return oracle.softmax(ins[0], a.get("axis", 1))
    if ty in ("Add", "Sub", "Mul", "Div"):
        return oracle.elementwise(ty, ins[0], ins[1])
    if ty == "BroadcastTo":
        return oracle.broadcast_to(ins[0], like=ins[1]) if len(ins) > 1 else oracle.broadcast_to(ins[0], shape=a["shape"])
    if ty == "Where":
        return oracle.where(ins[0], ins[1], ins[2])
    if ty == "Concat":
        return oracle.concat(ins, a.get("axis", 1))
    if ty == "ReduceSum":
        return oracle.reduce_sum(ins[0], a.get("axis", 0), a.get("keepdims", 1))
    if ty == "Fuse":
        return oracle.fuse(ins[0], ins[1], a.get("comm_index", 0))
    if ty == "Reshape":
        return oracle.reshape(ins[0], [int(v) for v in ins[1].reshape(-1)])
    if ty == "Gather":
        return oracle.gather(ins[0], ins[1], a.get("axis", 0))
    if ty == "Slice":
        return oracle.slice_axis(ins[0], a.get("axis", 0), a.get("start", 0), a.get("end", 1))
    if ty == "BatchNormalization":
        return oracle.batch_norm(ins[0], ins[1], ins[2], ins[3], ins[4], a.get("eps", 0.001), bool(a.get("nosqrt", 0)))
    raise KeyError(ty)


SHAPE_CASES = [
    "concat_net_v1_cpu", "concat_net_v2_cpu", "reduce_sum_net_v1_cpu", "fuse_net_v1_cpu", "fuse_net_v2_cpu",
    "reshape_net_v1_cpu", "batch_normalization_net_v1_cpu", "elementwise_add_net_v1_cpu", "elementwise_add_net_v2_cpu",
    "elementwise_sub_net_v1_cpu", "elementwise_sub_net_v2_cpu", "elementwise_mul_net_v1_cpu", "elementwise_mul_net_v2_cpu",
    "elementwise_div_net_v1_cpu", "elementwise_div_net_v2_cpu", "elementwise_broadcast_to_net_v1_cpu",
    "elementwise_broadcast_to_net_v2_cpu", "elementwise_where_net_v1_cpu", "gather_net_v1_cpu", "gather_net_v2_cpu",
    "slice_net_v1_cpu"
]

DENSE_CASES = SHAPE_CASES + [
    "gemm_net_v1_cpu", "prelu_net_v1_cpu", "dice_net_v1_cpu", "leaky_relu_net_v1_cpu", "sigmoid_net_v1_cpu",
    "softmax_net_v1_cpu", "matmul_net_v1_cpu", "fused_parallel_gemm_net_v1_cpu", "fused_parallel_gemm_net_v2_cpu",
    "fused_parallel_gemm_net_v3_cpu", "fused_parallel_gemm_net_v4_cpu", "fused_parallel_gemm_net_v5_cpu",
    "fused_parallel_matmul_net_v1_cpu", "fused_parallel_matmul_net_v2_cpu", "fused_parallel_matmul_net_v3_cpu"
]


@pytest.mark.parametrize("name", DENSE_CASES)
def test_reference_dense_kat(oracle, kats, name):
    case = kats[name]
    got = _run_op(oracle, case)
    (exp,) = case["expected"].values()
    want = np.array(exp["values"], np.float32).reshape(exp["shape"])
    assert list(got.shape) == exp["shape"]
    np.testing.assert_allclose(got, want, rtol=0, atol=ATOL_KAT)


def test_gather_and_slice_closed_forms(oracle):
    """oracle.gather / oracle.slice_axis (restated memcpy loops) against numpy's take and basic slicing on every axis,
    indices of both integer types and of rank 2, repeated indices."""
    rng = np.random.default_rng(17)
    x = rng.standard_normal((3, 5, 4, 2)).astype(np.float32)
    for axis in range(4):
        for idt in (np.int32, np.int64):
            idx = rng.integers(0, x.shape[axis], (2, 3)).astype(idt)
            assert np.array_equal(oracle.gather(x, idx, axis), np.take(x, idx, axis=axis))
        idx = np.array([x.shape[axis] - 1, 0, 0], np.int32)
        assert np.array_equal(oracle.gather(x, idx, axis), np.take(x, idx, axis=axis))
        for start, end in ((0, 1), (0, x.shape[axis]), (1, 2), (x.shape[axis] - 1, x.shape[axis])):
            sl = [slice(None)] * 4
            sl[axis] = slice(start, end)
            assert np.array_equal(oracle.slice_axis(x, axis, start, end), x[tuple(sl)])


@pytest.mark.parametrize("name", ["split_net_v1_cpu", "split_net_v2_cpu"])
def test_reference_split_kat(oracle, kats, name):
    case = kats[name]
    op = case["ops"][0]
    got = oracle.split(_tensor(case["tensors"][op["inputs"][0]]), len(op["outputs"]), op["args"].get("axis", 1),
                       op["args"].get("split"))
    for y, out in zip(got, op["outputs"]):
        exp = case["expected"][out]
        assert list(y.shape) == exp["shape"]
        np.testing.assert_allclose(y, np.array(exp["values"], np.float32).reshape(exp["shape"]), rtol=0, atol=ATOL_KAT)
    # numpy's own split is the closed form
    x = np.arange(2 * 6 * 3, dtype=np.float32).reshape(2, 6, 3)
    for a, b in zip(oracle.split(x, 3, 1), np.split(x, 3, axis=1)):
        assert np.array_equal(a, b)
    for a, b in zip(oracle.split(x, 2, 0), np.split(x, 2, axis=0)):
        assert np.array_equal(a, b)
    for a, b in zip(oracle.split(x, 2, 2, [1, 2]), np.split(x, [1], axis=2)):
        assert np.array_equal(a, b)


# ---------------------------------------------------------------- embedding op, reference fixture embedding_v1.conf
EMB_FG = {"101": ("a_01", 4), "102": ("a_02", 8), "104_7": ("a_03", 6)}
EMB_BLOCKS = [[{"fg": "101", "udf": 0}, {"fg": "102", "udf": 0}],
              [{"fg": "104_7", "udf": 2, "trunc_dir": 0, "trunc_num": 4}]]


def test_reference_embedding_op_kat(oracle, kats):
    """embedding_v1.conf runs the op over the mock puller: every key resolves to a row of ones
    (store/mock_sparse_puller.cc:11,57-94), so tables of ones keyed by every id reproduce it."""
    case = kats["embedding_v1"]
    t = case["tensors"]
    inputs = {fg: (_tensor(t[fg + ".ids"]), _tensor(t[fg + ".values"]), _tensor(t[fg + ".segments"])) for fg in EMB_FG}
    tables = {}
    for fg, (tname, dim) in EMB_FG.items():
        keys = np.unique(inputs[fg][0])
        tables[tname] = oracle.Table(np.ones((keys.size, dim), np.float32), keys=keys)
    outs = oracle.embedding_op(EMB_FG, EMB_BLOCKS, inputs, tables)
    for got, name in zip(outs, ["block1_values", "block2_values"]):
        exp = case["expected"][name]
        assert list(got.shape) == exp["shape"]
        np.testing.assert_allclose(got, np.array(exp["values"], np.float32).reshape(exp["shape"]), rtol=0, atol=ATOL_KAT)
    strides, placed = oracle.embedding_layout(EMB_FG, EMB_BLOCKS)
    assert strides == [12, 24]
    assert placed == [[("101", 0, 4), ("102", 4, 8)], [("104_7", 0, 24)]]


# ---------------------------------------------------------------- store KATs restated from the reference's unit tests
QED_KEYS = {"101": [1032342412], "102": [849234344343], "104_7": [3434234243, 5230242044]}
CASE1 = [1.0, 1.0, 3.0, 1.0]
CASE2 = [0.15, 0.3, 2.0, 1.0, 1.0, 2.0, 0.23, 3.0]
CASE3 = [2.5, 1.0, 0.15, 0.3, 2.0, 1.0]
CASE4 = [1.0, 0.15, 0.3, 2.0, 1.0, 1.0]


def _qed_inputs():
    """Inputs of TestQuickEmbeddingDict.Get (test/store/quick_embedding/quick_embedding_dict_test.cc:100-190)."""
    return {
        "101": (np.array([1032342412, 12312422], np.int64), np.array([2.0, 1.2], np.float32), np.array([1, 1], np.int32)),
        "102": (np.array([2324222, 849234344343, 849234344343], np.int64), np.array([2.0, 1.2, 1.0], np.float32),
                np.array([1, 2], np.int32)),
        "104_7": (np.array([3434234243, 5230242044, 2424123, 3434234243, 0, 5230242044], np.int64),
                  np.ones(6, np.float32), np.array([4, 2], np.int32)),
    }


def _qed_expected():
    """Expectations of the same test (:192-245): found keys scale their row, absent keys leave zeros."""
    b1 = np.zeros((2, 12), np.float32)
    b1[0, 0:4] = np.float32(2.0) * np.array(CASE1, np.float32)
    b1[1, 4:12] = np.array(CASE2, np.float32) * (np.float32(1.2) + np.float32(1.0))
    b2 = np.zeros((2, 24), np.float32)
    b2[0, 0:6] = CASE3
    b2[0, 6:12] = CASE4
    b2[0, 18:24] = CASE3
    b2[1, 6:12] = CASE4
    return b1, b2


def test_reference_qed_get_kat(oracle):
    tables = {
        "a_01": oracle.Table(np.array([CASE1], np.float32), keys=QED_KEYS["101"]),
        "a_02": oracle.Table(np.array([CASE2], np.float32), keys=QED_KEYS["102"]),
        "a_03": oracle.Table(np.array([CASE3, CASE4], np.float32), keys=QED_KEYS["104_7"]),
    }
    outs = oracle.embedding_op(EMB_FG, EMB_BLOCKS, _qed_inputs(), tables)
    b1, b2 = _qed_expected()
    # the reference compares with EXPECT_FLOAT_EQ (4 ulp)
    np.testing.assert_allclose(outs[0], b1, rtol=5e-7, atol=0)
    np.testing.assert_allclose(outs[1], b2, rtol=5e-7, atol=0)


def test_unknown_table_leaves_zeros(oracle):
    """table name miss -> kOK, block untouched (quick_embedding_dict.cc:95)."""
    outs = oracle.embedding_op(EMB_FG, EMB_BLOCKS, _qed_inputs(), {})
    assert all(not o.any() for o in outs)


def _udf_run(oracle, udf, tdir, tnum, weights, value, dim):
    """Drive one segment of `len(weights)` ids with distinct rows through the pooling loop."""
    n = len(weights)
    table = oracle.Table(np.array(weights, np.float32).reshape(n, dim))
    width = dim * tnum if udf == 2 else dim
    out = np.full((1, width), 7.0, np.float32)  # InitProcess must clear it
    oracle.embed_get(table, np.arange(n), np.full(n, value, np.float32), [n], [(udf, tdir, tnum, out, 0)])
    return out[0]


def test_reference_udf_ksum_kavg(oracle):
    """udf_processor_test.cc:38-122: 10 ids, value 0.5, weights[j]=j -> ksum 5j, kavg 0.5j."""
    dim = 12
    w = [[float(j) for j in range(dim)]] * 10
    np.testing.assert_allclose(_udf_run(oracle, 0, 0, 0, w, 0.5, dim), [0.5 * j * 10 for j in range(dim)], rtol=5e-7)
    np.testing.assert_allclose(_udf_run(oracle, 1, 0, 0, w, 0.5, dim), [0.5 * j for j in range(dim)], rtol=5e-7)


def test_reference_udf_kassign(oracle):
    """udf_processor_test.cc:124-292: weights[i][j] = 0.1*i + j, value 0.5."""
    dim, n = 12, 10
    w = [[0.1 * i + j for j in range(dim)] for i in range(n)]
    # in-order, trunc 5: slots 0..4 hold ids 0..4
    got = _udf_run(oracle, 2, 0, 5, w, 0.5, dim).reshape(5, dim)
    want = np.array([[0.5 * (0.1 * i + j) for j in range(dim)] for i in range(5)])
    np.testing.assert_allclose(got, want, rtol=5e-7)
    # reverse, trunc 4: slots 0..3 hold the last four ids 6..9
    got = _udf_run(oracle, 2, 1, 4, w, 0.5, dim).reshape(4, dim)
    want = np.array([[0.5 * (0.1 * i + j) for j in range(dim)] for i in range(6, 10)])
    np.testing.assert_allclose(got, want, rtol=5e-7)
    # reverse, no truncation: 20 slots, the 10 ids right-aligned, the first 10 slots zero
    got = _udf_run(oracle, 2, 1, 20, w, 0.5, dim).reshape(20, dim)
    assert not got[:10].any()
    want = np.array([[0.5 * (0.1 * i + j) for j in range(dim)] for i in range(10)])
    np.testing.assert_allclose(got[10:], want, rtol=5e-7)


# ---------------------------------------------------------------- the reference's own object code (oracle/_ref)
needs_ref = pytest.mark.skipif("not __import__('blaze_oracle').have_ref()",
                               reason="oracle/_ref not built (needs the reference tree)")


@needs_ref
def test_hash_index_matches_reference_object_code(oracle):
    rng = np.random.default_rng(5)
    for n in (1, 7, 53, 54, 1000, 20000):
        keys = np.unique(rng.integers(0, 2**63, size=n, dtype=np.int64) | rng.integers(0, 2, size=n, dtype=np.int64))
        rows = rng.standard_normal((keys.size, 3)).astype(np.float32)
        ref = oracle.RefStore(keys, rows)
        # the reference stores the blob byte offset (1 + 12*i, weight_blob.h:20,42-52) as the hash value
        mine = oracle.HashTable(keys.astype(np.uint64), 1 + 12 * np.arange(keys.size, dtype=np.uint64))
        assert np.array_equal(mine.dump(), ref.hash_dump()), "serialised index differs from HashTable::Dump"
        probe = np.concatenate([keys[:50], rng.integers(0, 2**63, size=50, dtype=np.int64)])
        for k in probe:
            assert mine.lookup(k) == ref.lookup(k)


@needs_ref
@pytest.mark.parametrize("seed", range(6))
def test_pooling_matches_reference_object_code(oracle, seed):
    """Bit-exact agreement with KSum/KAvg/KAssignProcessor + HashTable + WeightBlob compiled from the reference."""
    rng = np.random.default_rng(100 + seed)
    dim = int(rng.integers(1, 40))
    nkeys = int(rng.integers(1, 300))
    keys = np.unique(rng.integers(-2**40, 2**40, size=nkeys, dtype=np.int64))
    rows = (rng.standard_normal((keys.size, dim)) * 3).astype(np.float32)
    batch = int(rng.integers(1, 40))
    segments = rng.integers(0, 9, size=batch).astype(np.int32)
    nnz = int(segments.sum())
    pool = np.concatenate([keys, rng.integers(-2**40, 2**40, size=max(1, keys.size // 3), dtype=np.int64)])
    ids = rng.choice(pool, size=nnz)
    values = rng.standard_normal(nnz).astype(np.float32)
    specs = [(0, 0, 0), (1, 0, 0), (2, 0, 3), (2, 1, 5), (2, 1, 1)]
    widths = [dim, dim, dim * 3, dim * 5, dim]
    stride = sum(widths) + 2
    got = np.full((batch, stride), np.nan, np.float32)
    want = np.full((batch, stride), np.nan, np.float32)
    items_g, items_w, col = [], [], 1
    for (udf, tdir, tnum), w in zip(specs, widths):
        items_g.append((udf, tdir, tnum, got, col))
        items_w.append((udf, tdir, tnum, want, col))
        col += w
    oracle.embed_get(oracle.Table(rows, keys=keys), ids, values, segments, items_g)
    oracle.RefStore(keys, rows).embed_get(ids, values, segments, items_w)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@needs_ref
def test_qed_kat_on_reference_object_code(oracle):
    """The reference's own processors reproduce its own expectations (sanity of the driver)."""
    ins = _qed_inputs()
    b1 = np.zeros((2, 12), np.float32)
    b2 = np.zeros((2, 24), np.float32)
    oracle.RefStore(QED_KEYS["101"], [CASE1]).embed_get(*ins["101"], [(0, 0, 0, b1, 0)])
    oracle.RefStore(QED_KEYS["102"], [CASE2]).embed_get(*ins["102"], [(0, 0, 0, b1, 4)])
    oracle.RefStore(QED_KEYS["104_7"], [CASE3, CASE4]).embed_get(*ins["104_7"], [(2, 0, 4, b2, 0)])
    e1, e2 = _qed_expected()
    np.testing.assert_allclose(b1, e1, rtol=5e-7)
    np.testing.assert_allclose(b2, e2, rtol=5e-7)


# ---------------------------------------------------------------- scan, conversions, closed forms
def test_segments_to_offsets(oracle, kats):
    for fg, want in (("101", [0, 1, 2]), ("102", [0, 1, 3]), ("104_7", [0, 4, 6])):
        seg = _tensor(kats["embedding_v1"]["tensors"][fg + ".segments"])
        assert oracle.segments_to_offsets(seg).tolist() == want
    rng = np.random.default_rng(0)
    for n in (0, 1, 2, 63, 64, 65, 2048, 100003):
        seg = rng.integers(0, 70, size=n).astype(np.int32)
        off = oracle.segments_to_offsets(seg)
        assert off[0] == 0 and off[-1] == seg.sum(dtype=np.int64)
        assert np.array_equal(np.diff(off), seg)
    big = np.full(3, 2**31 - 1, np.int32)  # the running sum must not wrap in 32 bits
    assert oracle.segments_to_offsets(big).tolist() == [0, 2**31 - 1, 2 * (2**31 - 1), 3 * (2**31 - 1)]


def test_half_conversions_against_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = oracle.half_to_float(bits)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    rng = np.random.default_rng(1)
    f = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0)**rng.integers(-9, 6, 200000).astype(np.float32),
        want[np.isfinite(want)],
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e10, -1e10, np.inf, -np.inf, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001,
                  2.0**-14, 6.0975552e-05, 5.9604645e-08 * 1.5, 5.9604645e-08 * 2.5], np.float32)
    ])
    # midpoints between adjacent halves exercise ties-to-even
    mids = ((want[:-1].astype(np.float64) + want[1:].astype(np.float64)) / 2)
    mids = mids[np.isfinite(mids)].astype(np.float32)
    f = np.concatenate([f, mids])
    with np.errstate(over="ignore"):
        want_h = f.astype(np.float16).view(np.uint16)
    got_h = oracle.float_to_half(f)
    assert np.array_equal(got_h, want_h)


def test_fp16_and_int8_tables_by_brute_force(oracle):
    """fp16 rows widen exactly; the int8 extension is out = (1/n) * sum_j v_j * (scale[r_j] * q[r_j])."""
    rng = np.random.default_rng(2)
    rows, dim, batch = 50, 24, 17
    seg = rng.integers(0, 6, batch).astype(np.int32)
    nnz = int(seg.sum())
    ids = rng.integers(-2, rows + 2, nnz)  # a few out-of-range ids = missing
    vals = rng.standard_normal(nnz).astype(np.float32)
    h = rng.standard_normal((rows, dim)).astype(np.float16)
    q = rng.integers(-127, 128, (rows, dim)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, rows).astype(np.float32)
    for table, w32 in ((oracle.Table(h), h.astype(np.float32)), (oracle.Table(q, scale=sc), sc[:, None] * q.astype(np.float32))):
        for udf in (0, 1):
            got = np.zeros((batch, dim), np.float32)
            oracle.embed_get(table, ids, vals, seg, [(udf, 0, 0, got, 0)])
            want = np.zeros((batch, dim), np.float32)
            p = 0
            for b in range(batch):
                acc = np.zeros(dim, np.float32)
                for j in range(seg[b]):
                    if 0 <= ids[p] < rows:
                        acc = acc + vals[p] * w32[ids[p]]
                    p += 1
                if udf == 1 and seg[b]:
                    acc = acc * np.float32(1.0 / seg[b])
                want[b] = acc
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_gemm_against_float64(oracle):
    rng = np.random.default_rng(3)
    for (M, N, K, ta, tb) in [(5, 7, 11, 0, 0), (8, 3, 20, 1, 0), (4, 9, 6, 0, 1), (6, 6, 33, 1, 1), (1, 1, 1, 0, 0)]:
        A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
        B = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        alpha, beta = 0.75, -1.25
        got = oracle.gemm_op(A, B, bias, bool(ta), bool(tb), alpha, beta)
        a64 = (A.T if ta else A).astype(np.float64)
        b64 = (B.T if tb else B).astype(np.float64)
        want = alpha * (a64 @ b64) + beta * bias.astype(np.float64)
        scale = np.abs(alpha) * (np.abs(a64) @ np.abs(b64)) + np.abs(beta * bias)
        assert np.all(np.abs(got - want) <= 2e-6 * scale + 1e-30)
        g64 = oracle.gemm_ex(A, B, bool(ta), bool(tb), alpha, beta, C0=bias, f64=True)
        np.testing.assert_allclose(g64, want, rtol=1e-12, atol=1e-12)
    # special cases: identity weight, alpha = 0, no bias
    A = rng.standard_normal((4, 4)).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    assert np.array_equal(oracle.gemm_op(A, np.eye(4, dtype=np.float32), bias), A + bias)
    assert np.array_equal(oracle.gemm_op(A, A, bias, alpha=0.0), np.broadcast_to(bias, (4, 4)))
    np.testing.assert_allclose(oracle.gemm_op(A, A), A.astype(np.float64) @ A.astype(np.float64), rtol=1e-5, atol=1e-6)


def test_gemm_3d_is_loop_of_2d(oracle):
    """No reference fixture covers the 3-D branch (gemm_op.h:52-58,77-91); pinned by the loop identity only."""
    rng = np.random.default_rng(4)
    A = rng.standard_normal((3, 4, 5)).astype(np.float32)
    B = rng.standard_normal((5, 6)).astype(np.float32)
    bias = rng.standard_normal(6).astype(np.float32)
    got = oracle.gemm_op(A, B, bias)
    assert got.shape == (3, 4, 6)
    for i in range(3):
        assert np.array_equal(got[i], oracle.gemm_op(A[i], B, bias))
    A1 = rng.standard_normal((7, 1, 5)).astype(np.float32)  # M == 1 collapses to one 2-D gemm with M = batch
    got = oracle.gemm_op(A1, B, bias)
    assert got.shape == (7, 1, 6)
    assert np.array_equal(got[:, 0, :], oracle.gemm_op(A1[:, 0, :], B, bias))


def test_matmul_broadcast_against_numpy(oracle):
    rng = np.random.default_rng(6)
    A = rng.standard_normal((5, 3, 4)).astype(np.float32)
    B1 = rng.standard_normal((1, 4, 2)).astype(np.float32)
    np.testing.assert_allclose(oracle.matmul_op(A, B1), np.matmul(A.astype(np.float64), B1.astype(np.float64)), rtol=1e-5,
                               atol=1e-6)
    # DIN batchdot: weights [B,T] x history [B,T,D], from_deepnet + transA -> [B,1,D]
    w = rng.standard_normal((5, 7)).astype(np.float32)
    H = rng.standard_normal((5, 7, 3)).astype(np.float32)
    got = oracle.matmul_op(w, H, transa=True, transb=False, from_deepnet=True)
    assert got.shape == (5, 1, 3)
    np.testing.assert_allclose(got[:, 0, :], np.einsum("bt,btd->bd", w.astype(np.float64), H.astype(np.float64)),
                               rtol=1e-5, atol=1e-6)


def test_activation_closed_forms(oracle):
    x = np.array([-3.0, -0.5, 0.0, 0.5, 3.0], np.float32)
    # PRelu: x>0 -> x, x<0 -> w*x, 0 -> 0
    np.testing.assert_array_equal(oracle.prelu(x, [0.25]), np.array([-0.75, -0.125, 0, 0.5, 3.0], np.float32))
    # Dice limits: gamma = 1 -> identity; x >> mean -> x; x << mean -> gamma*x
    g1 = oracle.dice(x, np.ones(5), np.zeros(5), np.ones(5))
    np.testing.assert_allclose(g1, x, rtol=1e-6, atol=1e-7)
    big = oracle.dice(np.array([50.0, -50.0], np.float32), [0.3, 0.3], [0.0, 0.0], [1.0, 1.0])
    np.testing.assert_allclose(big, [50.0, -15.0], rtol=1e-6)
    # Dice against float64 closed form incl. nosqrt
    rng = np.random.default_rng(7)
    X = rng.standard_normal((6, 5)).astype(np.float32)
    gm, mu, var = (rng.standard_normal(5).astype(np.float32), rng.standard_normal(5).astype(np.float32),
                   rng.uniform(0.5, 1.5, 5).astype(np.float32))
    for nosqrt in (False, True):
        den = var.astype(np.float64) if nosqrt else np.sqrt(var.astype(np.float64) + 1e-8)
        p = 1 / (1 + np.exp(-(X - mu) / den))
        np.testing.assert_allclose(oracle.dice(X, gm, mu, var, nosqrt), (1 - p) * gm * X + p * X, rtol=2e-6, atol=1e-6)
    # sigmoid / softmax / leaky relu textbook
    np.testing.assert_allclose(oracle.sigmoid(x), 1 / (1 + np.exp(-x.astype(np.float64))), rtol=1e-6)
    sm = oracle.softmax(X, 1)
    e = np.exp(X.astype(np.float64) - X.max(1, keepdims=True))
    np.testing.assert_allclose(sm, e / e.sum(1, keepdims=True), rtol=1e-6)
    np.testing.assert_array_equal(oracle.leaky_relu(x, 0.1), np.where(x >= 0, x, np.float32(0.1) * x))

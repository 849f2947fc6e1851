"""Whole-model forwards composed from the oracle's functions -- test infrastructure, like the rest of oracle/.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg call these; no product code imports this file.
ctr_forward is the CTR tower of configurations 1 and 2 (Embedding ksum -> Concat with the dense features -> Gemm +
PRelu per layer -> Softmax), din_forward the DIN-style attention model of configuration 3; both follow the operator
sequence the reference's SimpleNet runs for such graphs (blaze/graph/simple_net.cc:35-46) with every operator taken
from blaze_oracle (passed in as `oracle`).
"""
import numpy as np

DIN_KINDS = ("item", "cate", "shop")


def ctr_forward(oracle, cfg, tables_np, mlp_np, sparse, dense, in_round=None, blas=False):
    """The same forward on the CPU oracle (fp32 path fed the kernel's rounded inputs).  tables_np: list of
    oracle.Table; mlp_np: [(W [K,N] fp32, b, slope)].  Returns (pooled [B, in_dim] fp32, probs [B, 2]).
    blas=True hands the products to the optimised sgemm numpy links (the reference calls MKL's cblas_sgemm there,
    math/gemm.cc:13-27) for timing a CPU baseline; its summation order is the library's, so parity tests keep the
    default k-ascending sums."""
    B = cfg.batch
    x = np.zeros((B, cfg.in_dim), np.float32)
    x[:, :cfg.dense] = dense if in_round is None else in_round(dense)
    for s, (ids, vals, seg) in enumerate(sparse):
        oracle.embed_get(tables_np[s], ids, vals, seg, [(0, 0, 0, x, cfg.dense + s * cfg.dim)])
    h = x if in_round is None else in_round(x)
    pooled = h.copy()
    n = len(mlp_np)
    for li, (w, b, slope) in enumerate(mlp_np):
        if blas:
            y = np.matmul(h, w)
            y += b  # the Gemm operator's bias broadcast
            h = oracle.softmax(y, 1) if li == n - 1 else oracle.prelu(y, slope)
            continue
        wt = np.ascontiguousarray(w.T)  # [N,K] + transB: same k-ascending sums, contiguous inner loop
        if li == n - 1:
            h = oracle.fc(h, wt, b, act="softmax", transb=True)
        else:
            h = oracle.fc(h, wt, b, act="prelu", act_params=(slope, ), transb=True)
            if in_round is not None:
                h = in_round(h)
    return pooled, h


def din_forward(oracle, cfg, tables_np, weights, batch, rnd):
    """The same graph on the CPU oracle.  tables_np: {kind: oracle.Table}; rnd: rounding applied to every operator
    output (identity for fp32, fp16 round trip for the fp16 model).  -> dict of named fp32 arrays."""
    B, T, D = cfg.batch, cfg.T, cfg.dim
    q = np.zeros((B, 3 * D), np.float32)
    his_k = []
    for i, k in enumerate(DIN_KINDS):
        oracle.embed_get(tables_np[k], batch[k + ".ids"], batch[k + ".values"], batch[k + ".segments"], [(0, 0, 0, q, i * D)])
        blk = np.zeros((B, T * D), np.float32)
        oracle.embed_get(tables_np[k], batch[k + "_his.ids"], batch[k + "_his.values"], batch[k + "_his.segments"],
                         [(2, 0, T, blk, 0)])
        his_k.append(oracle.reshape(rnd(blk), [-1, T, D]))
    q = rnd(q)
    his = oracle.concat(his_k, 2)
    q3 = oracle.reshape(q, [-1, 1, 3 * D])
    sub = rnd(oracle.elementwise("Sub", q3, his))
    mul = rnd(oracle.elementwise("Mul", q3, his))
    bq = oracle.broadcast_to(q3, like=sub)
    x = oracle.concat([bq, his, sub, mul], 2)
    n_att = len(weights["att"])
    for li, l in enumerate(weights["att"]):
        w, b = rnd(l["w"]), rnd(l["b"])
        x = oracle.gemm_op(x, w, b)
        if li < n_att - 1:
            x = oracle.dice(x, rnd(l["gamma"]), rnd(l["mean"]), rnd(l["var"]))
        x = rnd(x)
    score = x
    att_w = rnd(oracle.elementwise("Mul", score, rnd(batch["mask"])))
    att = oracle.reshape(rnd(oracle.matmul_op(att_w, his, True, False)), [-1, 3 * D])
    hsum = rnd(oracle.reduce_sum(his, 1, 0))
    x = oracle.concat([q, hsum, att], 1)
    main_in = x
    n_main = len(weights["main"])
    for li, l in enumerate(weights["main"]):
        w, b = rnd(l["w"]), rnd(l["b"])
        x = oracle.gemm_op(x, w, b)
        if li < n_main - 1:
            x = rnd(oracle.dice(x, rnd(l["gamma"]), rnd(l["mean"]), rnd(l["var"])))
    logit = rnd(x)
    return dict(q=q, his=his, att_in=None, score=score, att=att, hsum=hsum, main_in=main_in, logit=logit,
                prob=oracle.softmax(logit, 1))


def _arg(op, name, default=None):
    for a in op.arg:
        if a.name == name:
            if a.HasField("i"):
                return a.i
            if a.HasField("f"):
                return a.f
            if a.HasField("s"):
                return a.s
            if len(a.ints):
                return list(a.ints)
            if len(a.floats):
                return list(a.floats)
    return default


def run_netdef(oracle, net, feeds, tables):
    """An operator-by-operator forward of a parsed NetDef (a protobuf message with .op[].type/.input/.output/.arg) on
    the oracle's functions, in the order the reference's SimpleNet runs it (blaze/graph/simple_net.cc:35-46).  feeds:
    {external input name: numpy array}; tables: {table name: oracle.Table}.  Covers the operator set of the reference's
    shipped example model (blaze/example/tdm_data/model_blaze_optimized): Embedding with one pooled item per operator,
    Gather, Concat, Reshape, Slice, ReduceSum, Div, Gemm, BatchNormalization, PRelu, Softmax, ConstantFill.  Arguments are
    read as the reference's operators read them -- in particular Slice knows `start` / `end`, `starts` / `ends`, `axis` /
    `axes` (slice_op.h:36-62) and ignores any other name.  -> {tensor name: numpy array}."""
    import re
    t = dict(feeds)
    np_dtype = {1: np.float32, 2: np.int32, 10: np.int64}
    for op in net.op:
        ins = [t[name] for name in op.input]
        ty = op.type
        if ty == "ConstantFill":
            dt = np_dtype[_arg(op, "dtype", 1)]
            y = np.array(_arg(op, "value"), dt).reshape(_arg(op, "shape"))
        elif ty == "Embedding":
            cfg = _arg(op, "embedding_config").decode()
            table, dim = re.search(r'table_name: "([^"]+)"', cfg).group(1), int(re.search(r"dim: (\d+)", cfg).group(1))
            udf = int(re.search(r"udf_type: (\d+)", cfg).group(1))
            assert len(re.findall("embedding_block_config_item", cfg)) == 1 and udf in (0, 1)
            ids, values, segments = ins
            y = np.zeros((segments.size, dim), np.float32)
            oracle.embed_get(tables.get(table), ids, values, segments, [(udf, 0, 0, y, 0)])
        elif ty == "Gather":
            y = oracle.gather(ins[0], ins[1], _arg(op, "axis", 0))
        elif ty == "Concat":
            y = oracle.concat(ins, _arg(op, "axis", 1))
        elif ty == "Reshape":
            y = oracle.reshape(ins[0], [int(v) for v in ins[1].reshape(-1)])
        elif ty == "Slice":
            axes, starts, ends = _arg(op, "axes"), _arg(op, "starts"), _arg(op, "ends")
            axis = axes[0] if axes is not None else _arg(op, "axis", 0)
            start, end = (starts[0], ends[0]) if starts is not None else (_arg(op, "start", 0), _arg(op, "end", 1))
            y = oracle.slice_axis(ins[0], axis, start, end)
        elif ty == "ReduceSum":
            y = oracle.reduce_sum(ins[0], _arg(op, "axis", 0), _arg(op, "keepdims", 1))
        elif ty in ("Add", "Sub", "Mul", "Div"):
            y = oracle.elementwise(ty, ins[0], ins[1])
        elif ty == "Gemm":
            y = oracle.gemm_op(ins[0], ins[1], ins[2] if len(ins) > 2 else None, bool(_arg(op, "transA", 0)),
                               bool(_arg(op, "transB", 0)), _arg(op, "alpha", 1.0), _arg(op, "beta", 1.0))
        elif ty == "BatchNormalization":
            y = oracle.batch_norm(ins[0], ins[1], ins[2], ins[3], ins[4], _arg(op, "eps", 0.001), bool(_arg(op, "nosqrt", 0)))
        elif ty == "PRelu":
            y = oracle.prelu(ins[0], ins[1])
        elif ty == "Softmax":
            y = oracle.softmax(ins[0], _arg(op, "axis", 1))
        else:
            raise KeyError("run_netdef: no oracle for operator " + ty)
        t[op.output[0]] = y
    return t

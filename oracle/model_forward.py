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

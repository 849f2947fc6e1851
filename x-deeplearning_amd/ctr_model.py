"""The config-2 CTR model as a Blaze NetDef served by Predictors (harness for bench.py and tests).

Graph: Embedding (26 feature groups, ksum, fp16 block) -> Concat(dense, block) -> Gemm+PRelu -> Gemm+PRelu ->
Gemm+Softmax, the op sequence the reference's importers emit for such a model (Gemm with the bias as third input,
then a separate activation op: blaze/model_importer/ulf_importer.cc:335-374,661-782); SimpleNet folds each
activation into its Gemm's epilogue.
"""
import numpy as np

import pyblaze_hip as pb


def build_manager(cfg, tables, mlp, dtype=np.float16, expose_block=False, net_args=None):
    """tables: list of torch cuda tensors [rows, dim]; mlp: [(W [K,N], b, slope)] torch tensors.
    expose_block: also declare the pooled Embedding block an output of the net (for parity checks).
    net_args: further integer net arguments, e.g. {"alias_concat_inputs": 0}."""
    code = pb.K_FLOAT16 if dtype == np.float16 else pb.K_FLOAT
    pm = pb.PredictorManager()
    fgs = []
    for s, t in enumerate(tables):
        name = "table_%02d" % s
        pm.add_table(name, t)
        fgs.append(("fg%02d" % s, name, cfg.dim))
    nb = pb.NetBuilder("ctr_config2", device_type=1)
    inputs = []
    for fg, _, _ in fgs:
        nb.external_input(fg + ".ids", pb.K_INT64)
        nb.external_input(fg + ".values", pb.K_FLOAT)
        nb.external_input(fg + ".segments", pb.K_INT32)
        inputs += [fg + ".ids", fg + ".values", fg + ".segments"]
    nb.external_input("dense", code)
    nb.external_output("prob", pb.K_FLOAT)
    for k, v in (net_args or {}).items():
        nb.arg(k, int(v))
    if expose_block:
        nb.external_output("block", code)
    for li, (w, b, slope) in enumerate(mlp):
        nb.constant("w%d" % li, w.float().cpu().numpy(), dtype=code)
        nb.constant("b%d" % li, b.float().cpu().numpy(), dtype=pb.K_FLOAT if li == len(mlp) - 1 else code)
        if li < len(mlp) - 1:
            nb.constant("slope%d" % li, slope.float().cpu().numpy(), dtype=code)
    blocks = [[dict(fg=fg, udf=0) for fg, _, _ in fgs]]
    nb.op("Embedding", inputs, ["block"], embedding_config=pb.embedding_config_text(fgs, blocks),
          **({"out_dtype": code} if code != pb.K_FLOAT else {}))
    nb.op("Concat", ["dense", "block"], ["x0"], axis=1)
    n = len(mlp)
    for li in range(n):
        if li == n - 1:
            nb.op("Gemm", ["x%d" % li, "w%d" % li, "b%d" % li], ["logit"])
            nb.op("Softmax", ["logit"], ["prob"], axis=1)
        else:
            nb.op("Gemm", ["x%d" % li, "w%d" % li, "b%d" % li], ["h%d" % li])
            nb.op("PRelu", ["h%d" % li, "slope%d" % li], ["x%d" % (li + 1)])
    pm.load_model_from_string(nb.text(), True)
    return pm, fgs


def make_predictor(pm, fgs, sparse, dense, dtype=np.float16):
    p = pm.create_predictor(1, 0)
    feed_inputs(p, fgs, sparse, dense, dtype)
    return p


def feed_inputs(p, fgs, sparse, dense, dtype=np.float16):
    for (fg, _, _), (ids, vals, seg) in zip(fgs, sparse):
        p.feed(fg + ".ids", ids)
        p.feed(fg + ".values", vals)
        p.feed(fg + ".segments", seg)
    p.feed("dense", dense.astype(dtype))

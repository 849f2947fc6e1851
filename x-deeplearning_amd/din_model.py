"""Config 3: a DIN-style model (attention over the behaviour history) as a Blaze NetDef (harness for the parity tests and the benchmark).

Graph (operator types and arguments as the reference's importer emits them for such a model,
blaze/model_importer/ulf_importer.cc; structure after tools/example_model/din/model/graph_ulf.txt):

  Embedding(target item/cate/shop, ksum of one id)           -> q        [B, 3*D]
  Embedding(history of each kind, kassign in order, trunc T) -> his_k    [B, T*D]   (k = 0..2)
  Reshape his_k -> [B, T, D]; Concat(axis 2) -> his [B, T, 3D]; Reshape q -> q3 [B, 1, 3D]
  Sub(q3, his), Mul(q3, his), BroadcastTo(q3, like sub); Concat(axis 2) -> att_in [B, T, 12D]
  Gemm+Dice (12D -> 80), Gemm+Dice (80 -> 40), Gemm (40 -> 1)  -> score [B, T, 1]      (3-D Gemm)
  Mul(score, mask) -> w [B, T, 1]                         (mask = 1 for positions below the history length; no softmax)
  MatMul(w, his, transA) -> [B, 1, 3D]; Reshape -> att [B, 3D];  ReduceSum(his, axis 1) -> hsum [B, 3D]
  Concat(axis 1)[q, hsum, att] -> [B, 9D]; Gemm+Dice (-> 200), Gemm+Dice (-> 80), Gemm (-> 2), Softmax -> prob
"""
import numpy as np

import pyblaze_hip as pb
import philox
from philox import Stream
from synth import BoundedZipf, config_seed, lengths

KINDS = ("item", "cate", "shop")


class Config3:
    name = "config3: DIN, 3x[2M,18] fp16, history 50 (kassign), attention MLP 216-80-40-1 Dice, MLP 162-200-80-2 Dice"
    batch, T, rows, dim = 1024, 50, 2_000_000, 18
    att_layers = (216, 80, 40, 1)
    main_layers = (162, 200, 80, 2)
    zipf_s = 1.2

    def __init__(self, batch=None, rows=None, T=None):
        self.batch, self.rows, self.T = batch or self.batch, rows or self.rows, T or self.T
        d3 = 3 * self.dim
        self.att_layers = (4 * d3, ) + tuple(self.att_layers[1:])
        self.main_layers = (3 * d3, ) + tuple(self.main_layers[1:])

    seed = config_seed(3)

    def tables(self, device="cuda"):
        """[rows, dim] fp16 N(0, 0.1) per kind (generator stream = the kind's index)"""
        return [philox.tensor((self.rows, self.dim), philox.KIND_NORMAL_F16, Stream(s, self.seed), device, 0.1) for s in range(len(KINDS))]

    def table_rows(self, kind_index, rows):
        """rows (int array) of that kind's table recomputed on the host -> fp16 [len(rows), dim]"""
        return philox.host_rows(philox.KIND_NORMAL_F16, Stream(kind_index, self.seed), rows, self.dim, 0.1)

    def weights(self):
        """fp32 masters: per layer (W [K,N], b [N], gamma, mean, var); generator stream 3000 + layer (attention layers
        first), elements in that order."""
        out = {}
        layer = 0
        for tag, layers in (("att", self.att_layers), ("main", self.main_layers)):
            ls = []
            for li in range(len(layers) - 1):
                k, n = layers[li], layers[li + 1]
                st = Stream(3000 + layer, self.seed)
                layer += 1
                ls.append(dict(w=st.normal(0, k * n, np.float32(1.0 / np.sqrt(k))).reshape(k, n),
                               b=st.normal(k * n, n, 0.01),
                               gamma=st.normal(k * n + n, n, 0.1),
                               mean=st.normal(k * n + 2 * n, n, 0.1),
                               var=st.uniform32(k * n + 3 * n, n, 0.5, 1.5)))
            out[tag] = ls
        return out

    def batch_inputs(self, seed_offset=0):
        """-> dict name -> array: <kind>.ids/.values/.segments (one id per sample), <kind>_his.* (U{1..T} ids per
        sample, the same length for the three kinds), mask [B, T, 1] float32."""
        zipf = BoundedZipf(self.rows, self.zipf_s)
        B, T = self.batch, self.T
        first = int(seed_offset) << 32  # (generator streams: 2000 lengths, 1000 + kind target ids, 1100 + kind history ids)
        seg = np.minimum(lengths(Stream(2000, self.seed), first, "u1_50", B), T).astype(np.int32)
        nnz = int(seg.sum())
        feed = {}
        for ki, k in enumerate(KINDS):
            feed[k + ".ids"] = zipf.sample(Stream(1000 + ki, self.seed).uniform(first, B))
            feed[k + ".values"] = np.ones(B, np.float32)
            feed[k + ".segments"] = np.ones(B, np.int32)
            feed[k + "_his.ids"] = zipf.sample(Stream(1100 + ki, self.seed).uniform(first, nnz))
            feed[k + "_his.values"] = np.ones(nnz, np.float32)
            feed[k + "_his.segments"] = seg.copy()
        feed["mask"] = (np.arange(T)[None, :] < seg[:, None]).astype(np.float32).reshape(B, T, 1)
        return feed


def build_manager(cfg, tables, weights, dtype=np.float16, expose=(), net_args=None):
    """-> (PredictorManager with the model loaded, list of external input names).  `expose`: names of
    intermediate blobs also declared as outputs (for parity checks).  net_args: integer net arguments, e.g.
    {"fuse_concat_pieces": 0}."""
    code = pb.K_FLOAT16 if dtype == np.float16 else pb.K_FLOAT
    pm = pb.PredictorManager()
    for k, t in zip(KINDS, tables):
        pm.add_table("table_" + k, t)
    D, T = cfg.dim, cfg.T
    nb = pb.NetBuilder("din_config3", device_type=1)
    inputs = []
    for k in KINDS:
        for fg in (k, k + "_his"):
            nb.external_input(fg + ".ids", pb.K_INT64)
            nb.external_input(fg + ".values", pb.K_FLOAT)
            nb.external_input(fg + ".segments", pb.K_INT32)
            inputs += [fg + ".ids", fg + ".values", fg + ".segments"]
    nb.external_input("mask", code)
    inputs.append("mask")
    nb.external_output("prob", pb.K_FLOAT)
    for name in expose:
        nb.external_output(name, code)
    for k, v in (net_args or {}).items():
        nb.arg(k, int(v))
    for tag in ("att", "main"):
        for li, l in enumerate(weights[tag]):
            p = "%s%d_" % (tag, li)
            nb.constant(p + "w", l["w"], dtype=code)
            nb.constant(p + "b", l["b"], dtype=code)
            if li < len(weights[tag]) - 1:
                for q in ("gamma", "mean", "var"):
                    nb.constant(p + q, l[q], dtype=code)
    ext = {"out_dtype": code} if code != pb.K_FLOAT else {}
    # target side: one ksum block of the three kinds
    fgs = [(k, "table_" + k, D) for k in KINDS]
    nb.op("Embedding", [k + s for k in KINDS for s in (".ids", ".values", ".segments")], ["q"], name="ad_embedding",
          embedding_config=pb.embedding_config_text(fgs, [[dict(fg=k, udf=0) for k in KINDS]]), **ext)
    # history side: one kassign block per kind
    fgs = [(k + "_his", "table_" + k, D) for k in KINDS]
    nb.op("Embedding", [k + "_his" + s for k in KINDS for s in (".ids", ".values", ".segments")], ["his_" + k for k in KINDS],
          name="user_embedding",
          embedding_config=pb.embedding_config_text(fgs, [[dict(fg=k + "_his", udf=2, trunc_dir=0, trunc_num=T)] for k in KINDS]),
          **ext)
    nb.constant("shape_his", np.array([-1, T, D], np.int32))
    nb.constant("shape_q3", np.array([-1, 1, 3 * D], np.int32))
    nb.constant("shape_att", np.array([-1, 3 * D], np.int32))
    for k in KINDS:
        nb.op("Reshape", ["his_" + k, "shape_his"], ["his3_" + k])
    nb.op("Concat", ["his3_" + k for k in KINDS], ["his"], axis=2)
    nb.op("Reshape", ["q", "shape_q3"], ["q3"])
    nb.op("Sub", ["q3", "his"], ["sub"])
    nb.op("Mul", ["q3", "his"], ["mul"])
    nb.op("BroadcastTo", ["q3", "sub"], ["bq"])
    nb.op("Concat", ["bq", "his", "sub", "mul"], ["att_in"], axis=2)
    x = "att_in"
    n_att = len(weights["att"])
    for li in range(n_att):
        p = "att%d_" % li
        if li < n_att - 1:
            nb.op("Gemm", [x, p + "w", p + "b"], [p + "g"])
            nb.op("Dice", [p + "g", p + "gamma", p + "mean", p + "var"], [p + "y"])
            x = p + "y"
        else:
            nb.op("Gemm", [x, p + "w", p + "b"], ["score"])
    nb.op("Mul", ["score", "mask"], ["att_w"])
    nb.op("MatMul", ["att_w", "his"], ["att3"], transA=1, transB=0)
    nb.op("Reshape", ["att3", "shape_att"], ["att"])
    nb.op("ReduceSum", ["his"], ["hsum"], axis=1, keepdims=0)
    nb.op("Concat", ["q", "hsum", "att"], ["main_in"], axis=1)
    x = "main_in"
    n_main = len(weights["main"])
    for li in range(n_main):
        p = "main%d_" % li
        if li < n_main - 1:
            nb.op("Gemm", [x, p + "w", p + "b"], [p + "g"])
            nb.op("Dice", [p + "g", p + "gamma", p + "mean", p + "var"], [p + "y"])
            x = p + "y"
        else:
            nb.op("Gemm", [x, p + "w", p + "b"], ["logit"])
    nb.op("Softmax", ["logit"], ["prob"], axis=1)
    pm.load_model_from_string(nb.text(), True)
    return pm, inputs


def feed(p, inputs, batch, dtype=np.float16):
    for name in inputs:
        a = batch[name]
        p.feed(name, a.astype(dtype) if name == "mask" else a)

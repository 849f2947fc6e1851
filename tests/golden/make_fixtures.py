#!/usr/bin/env python3
"""Turn the reference's operator known-answer data files into small JSON fixtures.

Run in a container that has the reference tree mounted:

    python tests/golden/make_fixtures.py [/root/reference]

The reference's operator unit tests are data driven: each `*_cpu.conf` under
blaze/blaze/test/utest_data/operator/ is a text-format NetDef whose inputs are
ConstantFill ops and whose expected outputs are stored as net-level args
`<name>` / `<name>_shape` (compared with |d| <= 1e-6 by
blaze/blaze/test/operator/operator_test_common.h:20-84).  This script only reads
those DATA files -- it imports and executes nothing from the reference -- and
rewrites the numbers as JSON so the tests can run where the reference tree does
not exist.  Output: tests/golden/reference_kats.json.

It also copies two sets of DATA files the reference holds, byte for byte:
  blaze/example/tdm_data/model_blaze_optimized (a binary NetDef, 217 ops)          -> model_blaze_optimized.bin
  blaze/blaze/test/utest_data/store/quick_embedding/{meta,a_01,a_02,a_03}          -> quick_embedding/
(the text tables of embedding_builder_test.cc:13-23), and the input / expected NetDef pair of the optimizer's
parallel-Gemm fusion test (blaze/blaze/test/graph/pattern/in_parallel/in_parallel_gemm_test.cc):
  blaze/blaze/test/utest_data/graph/pattern/in_parallel/parallel_gemm_fusion{,_expected}.blaze               -> pattern/
and the four pairs of its in-order Gemm -> Gemm fusion test (.../test/graph/pattern/in_order/in_order_gemm_gemm_test.cc):
  blaze/blaze/test/utest_data/graph/pattern/in_order/in_order_gemm_gemm_fusion{,2,3,4}{,_expected}.blaze   -> pattern/
"""
import json
import os
import re
import sys

REL = "blaze/blaze/test/utest_data/operator"
CASES = [
    "op/gemm/gemm_net_v1_cpu.conf",
    "op/prelu/prelu_net_v1_cpu.conf",
    "op/dice/dice_net_v1_cpu.conf",
    "op/leaky_relu/leaky_relu_net_v1_cpu.conf",
    "op/sigmoid/sigmoid_net_v1_cpu.conf",
    "op/softmax/softmax_net_v1_cpu.conf",
    "op/matmul/matmul_net_v1_cpu.conf",
    "fused_op/fused_parallel_gemm/fused_parallel_gemm_net_v1_cpu.conf",
    "fused_op/fused_parallel_gemm/fused_parallel_gemm_net_v2_cpu.conf",
    "fused_op/fused_parallel_gemm/fused_parallel_gemm_net_v3_cpu.conf",
    "fused_op/fused_parallel_gemm/fused_parallel_gemm_net_v4_cpu.conf",
    "fused_op/fused_parallel_gemm/fused_parallel_gemm_net_v5_cpu.conf",
    "fused_op/fused_parallel_matmul/fused_parallel_matmul_net_v1_cpu.conf",
    "fused_op/fused_parallel_matmul/fused_parallel_matmul_net_v2_cpu.conf",
    "fused_op/fused_parallel_matmul/fused_parallel_matmul_net_v3_cpu.conf",
    "sparse_op/embedding/embedding_v1.conf",
    "op/concat/concat_net_v1_cpu.conf",
    "op/concat/concat_net_v2_cpu.conf",
    "op/reduce_sum/reduce_sum_net_v1_cpu.conf",
    "op/fuse/fuse_net_v1_cpu.conf",
    "op/fuse/fuse_net_v2_cpu.conf",
    "op/reshape/reshape_net_v1_cpu.conf",
    "op/batch_normalization/batch_normalization_net_v1_cpu.conf",
    "op/elementwise/elementwise_add_net_v1_cpu.conf",
    "op/elementwise/elementwise_add_net_v2_cpu.conf",
    "op/elementwise/elementwise_sub_net_v1_cpu.conf",
    "op/elementwise/elementwise_sub_net_v2_cpu.conf",
    "op/elementwise/elementwise_mul_net_v1_cpu.conf",
    "op/elementwise/elementwise_mul_net_v2_cpu.conf",
    "op/elementwise/elementwise_div_net_v1_cpu.conf",
    "op/elementwise/elementwise_div_net_v2_cpu.conf",
    "op/elementwise/elementwise_broadcast_to_net_v1_cpu.conf",
    "op/elementwise/elementwise_broadcast_to_net_v2_cpu.conf",
    "op/elementwise/elementwise_where_net_v1_cpu.conf",
    "op/split/split_net_v1_cpu.conf",
    "op/split/split_net_v2_cpu.conf",
    "op/gather/gather_net_v1_cpu.conf",
    "op/gather/gather_net_v2_cpu.conf",
    "op/slice/slice_net_v1_cpu.conf",
]

_TOK = re.compile(r'\s*(?:(#[^\n]*)|("(?:\\.|[^"\\])*")|([{}:])|([^\s{}:"#]+))')


def _tokens(text):
    pos = 0
    while True:
        m = _TOK.match(text, pos)
        if not m:
            if text[pos:].strip():
                raise ValueError("bad text proto near %r" % text[pos:pos + 40])
            return
        pos = m.end()
        if m.group(1):
            continue
        yield m.group(2) or m.group(3) or m.group(4)


def _unescape(s):
    return bytes(s[1:-1], "utf-8").decode("unicode_escape")


def _scalar(tok):
    if tok.startswith('"'):
        return _unescape(tok)
    t = tok.rstrip("fF") if re.match(r"^[-+]?[0-9.]+(?:[eE][-+]?\d+)?[fF]$", tok) else tok
    try:
        return int(t)
    except ValueError:
        pass
    try:
        return float(t)
    except ValueError:
        return tok  # enum / bool identifier


def parse_text_proto(text):
    """Generic protobuf text format -> {field: [values...]} with nested dicts for messages."""
    toks = list(_tokens(text))
    i = 0

    def msg(end):
        nonlocal i
        out = {}
        while i < len(toks) and toks[i] != end:
            name = toks[i]
            i += 1
            if toks[i] == ":":
                i += 1
            if toks[i] == "{":
                i += 1
                val = msg("}")
                i += 1
            else:
                val = _scalar(toks[i])
                i += 1
            out.setdefault(name, []).append(val)
        return out

    return msg(None)


def _args(arg_list):
    out = {}
    for a in arg_list or []:
        name = a["name"][0]
        for k in ("i", "f", "s"):
            if k in a:
                out[name] = a[k][0]
        for k in ("ints", "floats", "strings"):
            if k in a:
                out[name] = a[k]
    return out


def convert(path):
    with open(path) as f:
        net = parse_text_proto(f.read())
    tensors, ops = {}, []
    for op in net["op"]:
        args = _args(op.get("arg"))
        if op["type"][0] == "ConstantFill":
            tensors[op["output"][0]] = {"shape": args["shape"], "dtype": args["dtype"], "values": args["value"]}
        else:
            ops.append({"type": op["type"][0], "inputs": op.get("input", []), "outputs": op["output"], "args": args})
    nargs = _args(net.get("arg"))
    expected = {}
    for eo in net.get("external_output", []):
        name = eo["name"][0]
        expected[name] = {"shape": nargs[name + "_shape"], "dtype": eo.get("dtype", [1])[0], "values": nargs[name]}
    return {"tensors": tensors, "ops": ops, "expected": expected}


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    for rel in CASES:
        key = os.path.splitext(os.path.basename(rel))[0]
        out[key] = convert(os.path.join(root, REL, rel))
        out[key]["source"] = REL + "/" + rel
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_kats.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", dst, "cases:", len(out))
    import shutil
    here = os.path.dirname(os.path.abspath(__file__))
    shutil.copyfile(os.path.join(root, "blaze/example/tdm_data/model_blaze_optimized"), os.path.join(here, "model_blaze_optimized.bin"))
    os.makedirs(os.path.join(here, "quick_embedding"), exist_ok=True)
    for name in ("meta", "a_01", "a_02", "a_03"):
        shutil.copyfile(os.path.join(root, "blaze/blaze/test/utest_data/store/quick_embedding", name),
                        os.path.join(here, "quick_embedding", name))
    os.makedirs(os.path.join(here, "pattern"), exist_ok=True)
    for name in ("parallel_gemm_fusion.blaze", "parallel_gemm_fusion_expected.blaze"):
        shutil.copyfile(os.path.join(root, "blaze/blaze/test/utest_data/graph/pattern/in_parallel", name),
                        os.path.join(here, "pattern", name))
    for case in ("", "2", "3", "4"):
        for name in ("in_order_gemm_gemm_fusion%s.blaze" % case, "in_order_gemm_gemm_fusion%s_expected.blaze" % case):
            shutil.copyfile(os.path.join(root, "blaze/blaze/test/utest_data/graph/pattern/in_order", name),
                            os.path.join(here, "pattern", name))
    print("copied model_blaze_optimized.bin, quick_embedding/ and pattern/")


if __name__ == "__main__":
    main()

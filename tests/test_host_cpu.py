"""Host-layer checks that need no GPU: exported ABI, NetDef codecs against real protobuf, the QED builder against
the reference's own store object code, and error conventions of the C API."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, macro):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(macro + r"\s+[\w\s\*]+?\b(\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    """The shared library loads and exports exactly what include/*.h declares (no compute calls here)."""
    import blaze_hip
    import pyblaze_hip
    lib = C.CDLL(blaze_hip.LIB_PATH)
    kernel_api = _declared("blaze_hip.h", "BZ_API")
    predictor_api = _declared("blaze_c_api.h", "BLAZE_API")
    assert len(kernel_api) >= 11 and len(predictor_api) >= 36
    for name in kernel_api + predictor_api:
        assert hasattr(lib, name), "declared in include/ but not exported: " + name
    assert sorted(kernel_api) == sorted(blaze_hip.EXPORTS)
    assert sorted(predictor_api) == sorted(pyblaze_hip.EXPORTS)


def test_struct_layouts_match_header():
    """ctypes mirrors of the descriptor structs have the sizes the C compiler gives them."""
    import subprocess
    import tempfile
    import blaze_hip
    src = ('#include "blaze_hip.h"\n#include <stdio.h>\nint main(){printf("%zu %zu %zu %zu %zu ", sizeof(bz_embed_slot), '
           'sizeof(bz_embed_launch), sizeof(bz_fc_desc), sizeof(bz_bgemm_desc), sizeof(bz_act_desc));'
           'printf("%zu %zu %zu ", sizeof(bz_concat_desc), sizeof(bz_bcast_desc), sizeof(bz_bn_desc));printf("%zu %zu\\n", sizeof(bz_concat_ew_desc), sizeof(bz_weighted_pool_desc));printf("%zu\\n", sizeof(bz_fc_next));return 0;}\n')
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(src)
        subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), os.path.join(d, "s.c"), "-o", os.path.join(d, "s")])
        sizes = [int(x) for x in subprocess.check_output([os.path.join(d, "s")]).split()]
    assert sizes == [C.sizeof(blaze_hip.EmbedSlot), C.sizeof(blaze_hip.EmbedLaunch), C.sizeof(blaze_hip.FcDesc),
                     C.sizeof(blaze_hip.BgemmDesc), C.sizeof(blaze_hip.ActDesc), C.sizeof(blaze_hip.ConcatDesc),
                     C.sizeof(blaze_hip.BcastDesc), C.sizeof(blaze_hip.BnDesc),
                     C.sizeof(blaze_hip.ConcatEwDesc), C.sizeof(blaze_hip.WeightedPoolDesc), C.sizeof(blaze_hip.FcNext)]


def _sample_net():
    import pyblaze_hip as pb
    nb = pb.NetBuilder("ctr", device_type=1)
    nb.external_input("101.ids", pb.K_INT64)
    nb.external_input("101.values", pb.K_FLOAT)
    nb.external_input("101.segments", pb.K_INT32)
    nb.external_output("prob")
    nb.arg("fuse_gemm_activation", 0)
    nb.constant("w", np.array([[0.5, -1.25], [3.0, 1e-7]], np.float32))
    nb.constant("i64", np.array([1032342412, 849234344343, -5], np.int64))
    nb.op("Embedding", ["101.ids", "101.values", "101.segments"], ["block"],
          embedding_config=pb.embedding_config_text([("101", "a_01", 2)], [[dict(fg="101", udf=0)]]))
    nb.op("Gemm", ["block", "w"], ["fc"], transB=True, alpha=0.75)
    nb.op("Softmax", ["fc"], ["prob"], axis=1)
    return nb.text()


def test_netdef_text_to_wire_matches_protobuf():
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    wire = pb.convert_netdef(_sample_net(), True, False)
    net = NetDef()
    net.ParseFromString(wire)
    assert net.name == "ctr" and net.run_mode == "simple" and net.device_option.device_type == 1
    assert [o.type for o in net.op] == ["ConstantFill", "ConstantFill", "Embedding", "Gemm", "Softmax"]
    assert [v.name for v in net.external_input] == ["101.ids", "101.values", "101.segments"]
    assert [v.dtype for v in net.external_input] == [10, 1, 2]
    fill = {a.name: a for a in net.op[0].arg}
    assert list(fill["shape"].ints) == [2, 2] and fill["dtype"].i == 1
    assert np.array_equal(np.array(fill["value"].floats, np.float32), np.array([0.5, -1.25, 3.0, 1e-7], np.float32))
    assert list({a.name: a for a in net.op[1].arg}["value"].ints) == [1032342412, 849234344343, -5]
    gemm = {a.name: a for a in net.op[3].arg}
    assert gemm["transB"].i == 1 and gemm["alpha"].f == 0.75
    cfg = {a.name: a for a in net.op[2].arg}["embedding_config"].s.decode()
    assert 'table_name : "a_01"' in cfg and "\n" in cfg
    assert {a.name: a.i for a in net.arg} == {"fuse_gemm_activation": 0}


def test_netdef_wire_to_text_round_trip_through_protobuf():
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    from google.protobuf import text_format
    ref = NetDef()
    ref.name = "rt"
    ref.run_mode = "dag"
    ref.version = 1007
    ref.device_option.device_type = 1
    ref.device_option.device_id = 3
    op = ref.op.add()
    op.type, op.name = "Gemm", 'quote"and\\slash'
    op.input.extend(["a", "b"])
    op.output.append("y")
    op.device_option.device_type = 0
    op.device_option.device_id = 0
    a = op.arg.add()
    a.name, a.f = "alpha", 0.1
    a = op.arg.add()
    a.name = "blob"
    a.s = bytes(range(256))
    a.floats.extend([1.5, -2.25e-30, 3e38])
    a.ints.extend([0, -1, 2**62, -2**63])
    a.strings.extend([b"x", b""])
    vi = ref.external_input.add()
    vi.name, vi.dtype, vi.level, vi.input_type, vi.feature_name = "in", 12, 1, 3, "feat"
    vi.tensor_shape.dims.extend([7, 9])
    vo = ref.external_output.add()  # scalar fields are written out with their values whether or not they were set
    vo.name, vo.dtype, vo.level, vo.input_type = "y", 1, 0, 0
    wire = ref.SerializeToString()
    text = pb.convert_netdef(wire, False, True).decode("latin-1")
    back = NetDef()
    text_format.Parse(text, back)
    assert back == ref
    # and C++ wire writer -> protobuf reader
    again = NetDef()
    again.ParseFromString(pb.convert_netdef(wire, False, False))
    assert again == ref


def test_malformed_models_are_rejected():
    import pyblaze_hip as pb
    with pytest.raises(pb.BlazeError):
        pb.convert_netdef(b"\x0a\xff\xff\xff\xff\x0f", False, True)  # length runs past the buffer
    with pytest.raises(pb.BlazeError):
        pb.convert_netdef('op { type : "Gemm" ', True, False)  # missing brace
    with pytest.raises(pb.BlazeError):
        pb.convert_netdef('op { type : "Gemm" arg { name : "alpha" f : abc } }', True, False)
    pm = pb.PredictorManager()
    with pytest.raises(pb.BlazeError, match="can not open|failed"):
        pm.load_model("/nonexistent/model.blaze")
    with pytest.raises(pb.BlazeError, match="importer|failed"):
        pm.load_deepnet_model("a.conf", "a.dat")
    with pytest.raises(pb.BlazeError):
        pm.load_sparse_model_weight("/nonexistent/qed.bin")


def test_cpu_predictor_fails_loudly():
    """device_type 0 is accepted by the API but no operator of the path has a CPU implementation here."""
    import pyblaze_hip as pb
    pm = pb.PredictorManager()
    pm.load_model_from_string(_sample_net(), True)
    with pytest.raises(pb.BlazeError, match="no CPU fallback|not registered"):
        pm.create_predictor(device_type=0)


def test_null_handles_return_minus_one():
    import pyblaze_hip as pb
    l = pb.lib()
    assert l.Blaze_PredictorForward(None) == -1
    assert l.Blaze_PredictorDelete(None) == -1
    assert l.Blaze_PredictorFeed(None, b"x", None, 0) == -1
    assert l.Blaze_LoadSparseModelWeight(None, b"x") == -1
    assert l.Blaze_ConvertBlaze(None, None, 0, 0, 0, 0, None, None, None, 0) == -1
    assert "not part of this build" in pb.last_error()


# ---------------------------------------------------------------- QED builder
def _write_tables(tmp_path, tables):
    names = []
    for name, (keys, rows) in tables.items():
        with open(tmp_path / name, "w") as f:
            for k, r in zip(keys, rows):
                f.write(",".join([str(int(k))] + [repr(float(x)) for x in r]) + "\n")
        names.append(name)
    with open(tmp_path / "meta", "w") as f:
        f.write("\n".join(names) + "\n")


def _parse_qed(path):
    """Independent python reader of the QED container, returns (version, trie bytes, [(gid, hash image, blob image)])."""
    data = open(path, "rb").read()
    assert data[:31] == b"ALIMAMA_MODEL_SERVING_EMBEDDING"
    version = int.from_bytes(data[31:35], "little")
    pos = 35
    tlen = int.from_bytes(data[pos:pos + 8], "little")
    trie = data[pos:pos + 8 + tlen]
    pos += 8 + tlen
    tables = []
    while pos < len(data):
        gid = int.from_bytes(data[pos:pos + 2], "little")
        pos += 2
        nb = int.from_bytes(data[pos:pos + 4], "little")
        pb_ = int.from_bytes(data[pos + 4 + 8 * nb:pos + 12 + 8 * nb], "little")
        hlen = 4 + 8 * nb + 8 + pb_
        himg = data[pos:pos + hlen]
        pos += hlen
        blen = int.from_bytes(data[pos:pos + 8], "little")
        bimg = data[pos:pos + 8 + blen]
        pos += 8 + blen
        tables.append((gid, himg, bimg))
    return version, trie, tables


def test_qed_builder_file_image(tmp_path, oracle):
    import pyblaze_hip as pb
    rng = np.random.default_rng(12)
    tables = {}
    for name, n, dim in (("a_01", 60, 4), ("a_02", 1, 8), ("104_7", 200, 6)):
        keys = np.unique(rng.integers(-2**62, 2**62, size=n * 2, dtype=np.int64))[:n]
        tables[name] = (keys, rng.standard_normal((n, dim)).astype(np.float32))
    _write_tables(tmp_path, tables)
    out = str(tmp_path / "qed.bin")
    pb.build_qed(str(tmp_path), "meta", out)
    version, trie, parsed = _parse_qed(out)
    assert version == 2000 and [g for g, _, _ in parsed] == [0, 1, 2]
    for (name, (keys, rows)), (gid, himg, bimg) in zip(tables.items(), parsed):
        dim = rows.shape[1]
        # hash image: the oracle's restatement (itself byte-equal to the reference's HashTable::Dump)
        mine = oracle.HashTable(keys.astype(np.uint64), 1 + 4 * dim * np.arange(len(keys), dtype=np.uint64))
        assert bytes(mine.dump()) == himg
        assert int.from_bytes(bimg[:8], "little") == 1 + rows.nbytes
        assert bimg[9:] == rows.tobytes()
        if oracle.have_ref():
            ref = oracle.RefStore(keys, rows)
            assert bytes(ref.hash_dump()) == himg, "differs from the reference's HashTable::Dump"
            rb = bytes(ref.blob_dump())
            assert rb[:8] == bimg[:8] and rb[9:] == bimg[9:], "differs from the reference's WeightBlob::Dump"
    if oracle.have_ref():
        rt = oracle.RefTrie(list(tables.keys()), [0, 1, 2])
        assert bytes(rt.dump()) == trie, "differs from the reference's Trie::Dump"
    # fp16 flavour: same index, narrowed rows
    out16 = str(tmp_path / "qed16.bin")
    pb.build_qed(str(tmp_path), "meta", out16, fp16=True)
    v16, trie16, parsed16 = _parse_qed(out16)
    assert v16 == 2001 and trie16 == trie
    rows0 = tables["a_01"][1]
    assert parsed16[0][2][9:] == rows0.astype(np.float16).tobytes()


def test_qed_builder_meta_quirk_and_errors(tmp_path):
    """A last meta line without newline is dropped, as the reference's ParseMeta does; a missing table fails."""
    import pyblaze_hip as pb
    open(tmp_path / "t1", "w").write("1,0.5\n2,0.25\n")
    open(tmp_path / "t2", "w").write("1,0.5\n")
    open(tmp_path / "meta", "w").write("t1\nt2")
    out = str(tmp_path / "q.bin")
    pb.build_qed(str(tmp_path), "meta", out)
    _, _, parsed = _parse_qed(out)
    assert len(parsed) == 1
    open(tmp_path / "meta2", "w").write("t1\nmissing\n")
    with pytest.raises(pb.BlazeError, match="can not open"):
        pb.build_qed(str(tmp_path), "meta2", out)


def test_embedding_planner_geometry_and_scan_advice():
    """bz_embed_plan runs on the host only (the pointers are never followed): workgroup counts per slot -- a lane group
    per sample for ksum / kavg, per output position for kassign -- and the advice to scan the counts in a launch of
    their own once the fused scan would re-read them too often (config 5's shape), not for config 2's."""
    import ctypes as C
    import blaze_hip as bz

    def plan(n_slots, batch, dim, udf=bz.SUM, trunc=0, offsets=False, dtype=bz.F16, nnz=0):
        slots = (bz.EmbedSlot * n_slots)()
        for s in slots:
            s.nnz = nnz
            s.table, s.ids, s.values, s.segments, s.out = 0x10000, 0x20000, 0x30000, 0x40000, 0x50000
            s.rows, s.dim, s.pitch = 1000, dim, (dim * 2 + 15) // 16 * 16
            s.table_dtype, s.out_dtype, s.udf, s.batch = dtype, bz.F16, udf, batch
            s.trunc_num, s.trunc_dir, s.out_stride = trunc, 0, dim * max(trunc, 1)
            if offsets:
                s.offsets = 0x60000
        launch = bz.EmbedLaunch()
        assert bz.lib().bz_embed_plan(slots, n_slots, C.byref(launch)) == 0, bz.lib().bz_last_error()
        return slots, launch

    slots, launch = plan(26, 2048, 32, nnz=16400)  # config 2: dim 32 fp16 = 4 chunks -> 128 samples per 512-thread workgroup
    assert launch.total_wg == 26 * 16 and launch.wg_per_slot == 16 and launch.fused_scan == 1 and launch.scan_first == 0
    assert launch.variant == (bz.F16 << 8) | 4
    assert [s.wg_begin for s in slots][:3] == [0, 16, 32]
    assert launch.max_batch == 2048
    _, launch = plan(200, 8192, 64, nnz=20480)   # config 5: 8 chunks -> 64 samples per workgroup, 128 workgroups a slot
    assert launch.total_wg == 200 * 128 and launch.fused_scan == 1 and launch.scan_first == 1
    _, launch = plan(200, 8192, 64, offsets=True, nnz=20480)
    assert launch.fused_scan == 0 and launch.scan_first == 0
    # config 3's history: 3 chunks -> 4 lanes a group, 128 groups a workgroup, a group takes 4 of a sample's 50 positions
    slots, launch = plan(3, 1024, 18, udf=bz.ASSIGN, trunc=50)
    assert launch.variant == 0 and [s.wg_count for s in slots] == [1024 * 13 // 128] * 3


def test_baseline_forward_with_library_sgemm_agrees_with_the_pinned_sums(oracle):
    """bench.py times the oracle with the products handed to the BLAS numpy links (as the reference hands them to
    MKL, math/gemm.cc:13-27).  That variant must be the same computation: on a scaled-down config 2 it agrees with
    the k-ascending sums the parity tests use to fp32 summation-order noise (rel 1e-5)."""
    from model_forward import ctr_forward as oracle_forward
    from synth import Config2
    cfg = Config2(batch=96, rows=5000, slots=5)
    tables = cfg.tables(device="cpu")
    mlp_np = [(w.numpy(), b.numpy(), s.numpy()) for (w, b, s) in cfg.mlp(device="cpu")]
    sparse, dense = cfg.batches(1)
    tabs = [oracle.Table(t.numpy()) for t in tables]
    pooled, want = oracle_forward(oracle, cfg, tabs, mlp_np, sparse[0], dense[0])
    pooled_b, got = oracle_forward(oracle, cfg, tabs, mlp_np, sparse[0], dense[0], blas=True)
    np.testing.assert_array_equal(pooled_b, pooled)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)
    assert got.shape == (96, 2) and np.allclose(got.sum(1), 1.0, atol=1e-6)


# ---------------------------------------------------------------- documents and reference-held data files
def test_integration_c_snippet_compiles_against_the_header():
    """The C example of the integration guide names only entry points include/blaze_c_api.h declares (gcc -fsyntax-only)."""
    import subprocess
    import tempfile
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```c\n(.*?)```", text, flags=re.S)
    assert blocks, "no ```c block in the integration guide"
    body = blocks[0].replace("...", "")
    m = re.match(r"(\s*#include[^\n]*\n)(.*)", body, flags=re.S)
    src = (m.group(1) + "#include <stdint.h>\nvoid example(const int* shape, void* ids, int nnz, void* out, size_t out_bytes) {\n" +
           m.group(2) + "\n}\n")
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "snippet.c")
        open(path, "w").write(src)
        r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror=implicit-function-declaration", "-fsyntax-only", "-I",
                            os.path.join(ROOT, "include"), path], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def _arg_value(a):
    return (a.name, a.f if a.HasField("f") else None, a.i if a.HasField("i") else None, a.s if a.HasField("s") else None,
            list(a.floats), list(a.ints), list(a.strings))


def test_reference_binary_model_decodes_like_protobuf():
    """tests/golden/model_blaze_optimized.bin is the binary NetDef the reference ships with its TDM example
    (blaze/example/tdm_data/model_blaze_optimized, 217 operators; what Blaze_PredcitorManagerLoadModel reads,
    predictor_manager_impl.cc:31-116).  The library's own wire reader must see exactly what protobuf sees: the file is
    decoded by the C++ codec to text, the text is parsed by protobuf, and the result is compared field by field with
    protobuf's direct parse of the bytes."""
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    from google.protobuf import text_format
    wire = open(os.path.join(ROOT, "tests", "golden", "model_blaze_optimized.bin"), "rb").read()
    ref = NetDef()
    ref.ParseFromString(wire)
    assert len(ref.op) == 217
    text = pb.convert_netdef(wire, False, True).decode("latin-1")
    got = NetDef()
    text_format.Parse(text, got)
    assert got.name == ref.name and got.run_mode == ref.run_mode and got.version == ref.version
    assert [(v.name, v.dtype, v.level, v.input_type, v.feature_name) for v in got.external_input] == \
           [(v.name, v.dtype, v.level, v.input_type, v.feature_name) for v in ref.external_input]
    assert [(v.name, v.dtype) for v in got.external_output] == [(v.name, v.dtype) for v in ref.external_output]
    assert len(got.op) == len(ref.op)
    for a, b in zip(got.op, ref.op):
        assert (a.type, a.name, list(a.input), list(a.output)) == (b.type, b.name, list(b.input), list(b.output))
        assert [_arg_value(x) for x in a.arg] == [_arg_value(x) for x in b.arg]
        # the text writer spells scalar fields out with their values whether or not the file set them, so presence
        # may differ (device_id: 0) while the values may not
        assert (a.device_option.device_type, a.device_option.device_id, a.device_option.is_pipe) == \
               (b.device_option.device_type, b.device_option.device_id, b.device_option.is_pipe)
    assert [_arg_value(x) for x in got.arg] == [_arg_value(x) for x in ref.arg]
    # wire -> wire through the C++ codec: protobuf parses it to the same message apart from that presence
    again = NetDef()
    again.ParseFromString(pb.convert_netdef(wire, False, False))
    assert len(again.op) == 217 and [o.type for o in again.op] == [o.type for o in ref.op]
    assert sum(len(o.arg) for o in again.op) == sum(len(o.arg) for o in ref.op)
    types = {o.type for o in ref.op}
    assert "ConstantFill" in types and "Gemm" in types


def test_parallel_gemm_fusion_pass_on_the_reference_fixture(tmp_path):
    """Blaze_OptimizeBlaze on the input of the reference's parallel-Gemm fusion test gives the NetDef that test
    expects (blaze/blaze/test/graph/pattern/in_parallel/in_parallel_gemm_test.cc; compared as
    pattern_test_common.h:17-90 compares: operator types, names, inputs, outputs and arguments in order): two Gemms on one
    input become FusedParallelGemm over the stacked weight + Split(axis 0), and the orphaned constant is gone."""
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    from google.protobuf import text_format
    src = os.path.join(ROOT, "tests", "golden", "pattern", "parallel_gemm_fusion.blaze")
    want = NetDef()
    text_format.Parse(open(os.path.join(ROOT, "tests", "golden", "pattern", "parallel_gemm_fusion_expected.blaze")).read(), want)
    for binary in (False, True):
        dst = str(tmp_path / ("opt.%d" % binary))
        pb.optimize_blaze(src, dst, binary)
        got = NetDef()
        if binary:
            got.ParseFromString(open(dst, "rb").read())
        else:
            text_format.Parse(open(dst).read(), got)
        assert [o.type for o in got.op] == [o.type for o in want.op] == ["ConstantFill", "ConstantFill", "FusedParallelGemm", "Split", "Concat"]
        for a, b in zip(got.op, want.op):
            assert (a.type, a.name, list(a.input), list(a.output)) == (b.type, b.name, list(b.input), list(b.output))
            assert [_arg_value(x) for x in a.arg] == [_arg_value(x) for x in b.arg]
        assert [(v.name, v.dtype) for v in got.external_output] == [(v.name, v.dtype) for v in want.external_output]
        assert got.run_mode == want.run_mode
    # a net without sibling Gemms passes through unchanged; a second run of the pass finds nothing more to fuse
    again = str(tmp_path / "again")
    pb.optimize_blaze(str(tmp_path / "opt.1"), again, True)
    assert open(again, "rb").read() == open(str(tmp_path / "opt.1"), "rb").read()


@pytest.mark.parametrize("case", ["", "2", "3", "4"])
def test_gemm_gemm_folding_pass_on_the_reference_fixtures(tmp_path, case):
    """Blaze_OptimizeBlaze on the four inputs of the reference's in-order Gemm -> Gemm fusion test (no bias, a bias on the
    first, on the second, on both; blaze/blaze/test/graph/pattern/in_order/in_order_gemm_gemm_test.cc) gives the NetDefs
    that test expects: one Gemm on the product of the weights, alpha and beta as its only arguments, the folded bias in the
    surviving bias constant, the first Gemm and its orphaned constants gone.  Compared operator by operator in order
    (types, names, inputs, outputs, argument names, ints exactly, floats to fp32 rounding)."""
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    from google.protobuf import text_format
    d = os.path.join(ROOT, "tests", "golden", "pattern")
    want = NetDef()
    text_format.Parse(open(os.path.join(d, "in_order_gemm_gemm_fusion%s_expected.blaze" % case)).read(), want)
    dst = str(tmp_path / "opt")
    pb.optimize_blaze(os.path.join(d, "in_order_gemm_gemm_fusion%s.blaze" % case), dst, False)
    got = NetDef()
    text_format.Parse(open(dst).read(), got)
    assert [o.type for o in got.op] == [o.type for o in want.op]
    assert got.op[-1].type == "Gemm" and sum(o.type == "Gemm" for o in got.op) == 1
    for a, b in zip(got.op, want.op):
        assert (a.type, a.name, list(a.input), list(a.output)) == (b.type, b.name, list(b.input), list(b.output))
        assert [x.name for x in a.arg] == [x.name for x in b.arg]
        for x, y in zip(a.arg, b.arg):
            assert (list(x.ints), x.i if x.HasField("i") else None) == (list(y.ints), y.i if y.HasField("i") else None), x.name
            np.testing.assert_allclose(list(x.floats), list(y.floats), rtol=2e-7, atol=0, err_msg=a.name + "." + x.name)
            assert x.HasField("f") == y.HasField("f") and (not x.HasField("f") or x.f == y.f)
    assert [(v.name, v.dtype) for v in got.external_output] == [(v.name, v.dtype) for v in want.external_output]
    # nothing left to fold on a second run
    again = str(tmp_path / "again")
    pb.optimize_blaze(dst, again, False)
    assert open(again).read() == open(dst).read()


def test_gemm_gemm_folding_carries_the_second_alpha_into_the_first_bias(tmp_path):
    """alpha1 * (alpha0 * x * W0 + beta0 * b0) * W1 + beta1 * b1: the first layer's bias is scaled by the second layer's
    alpha as well (the reference's fixtures all have alpha1 = 1 and its CalcNewBias leaves the factor out).  The folded
    constants are compared with numpy's float64 products."""
    import pyblaze_hip as pb
    from blaze_proto import NetDef
    from google.protobuf import text_format
    rng = np.random.default_rng(5)
    K, H, N = 6, 5, 4
    w0 = rng.standard_normal((K, H)).astype(np.float32)
    w1 = rng.standard_normal((H, N)).astype(np.float32)
    b0, b1 = rng.standard_normal(H).astype(np.float32), rng.standard_normal(N).astype(np.float32)
    a0, be0, a1, be1 = 0.75, 2.0, 0.5, 3.0
    nb = pb.NetBuilder("chain", device_type=1)
    nb.external_input("x", pb.K_FLOAT)
    for name, v in (("w0", w0), ("b0", b0), ("w1", w1), ("b1", b1)):
        nb.constant(name, v)
    nb.op("Gemm", ["x", "w0", "b0"], ["h"], alpha=a0, beta=be0)
    nb.op("Gemm", ["h", "w1", "b1"], ["out"], alpha=a1, beta=be1)
    nb.external_output("out", pb.K_FLOAT)
    raw, opt = str(tmp_path / "raw.blaze"), str(tmp_path / "opt.blaze")
    open(raw, "w").write(nb.text())
    pb.optimize_blaze(raw, opt, False)
    got = NetDef()
    text_format.Parse(open(opt).read(), got)
    gemms = [o for o in got.op if o.type == "Gemm"]
    assert len(gemms) == 1 and list(gemms[0].input)[0] == "x"
    consts = {o.output[0]: np.array([a for a in o.arg if a.name == "value"][0].floats, np.float64) for o in got.op
              if o.type == "ConstantFill"}
    args = {a.name: a.f for a in gemms[0].arg}
    w, b = consts[gemms[0].input[1]].reshape(K, N), consts[gemms[0].input[2]]
    x = rng.standard_normal((3, K))
    want = a1 * ((a0 * x @ w0.astype(np.float64) + be0 * b0) @ w1.astype(np.float64)) + be1 * b1
    np.testing.assert_allclose(args["alpha"] * x @ w + args["beta"] * b, want, rtol=1e-5, atol=1e-6)


def _reference_text_tables():
    """-> {table: (keys int64 [n], rows fp32 [n, dim])} of tests/golden/quick_embedding (the reference's
    utest_data/store/quick_embedding: `key,w0,...` lines; the first weight column happens to hold a big integer)."""
    d = os.path.join(ROOT, "tests", "golden", "quick_embedding")
    out = {}
    for name in ("a_01", "a_02", "a_03"):
        keys, rows = [], []
        for line in open(os.path.join(d, name)).read().split("\n"):
            if not line:
                continue
            f = line.split(",")
            keys.append(int(f[0]))
            rows.append([np.float32(x) for x in f[1:]])
        out[name] = (np.array(keys, np.int64), np.array(rows, np.float32))
    return d, out


def test_qed_builder_on_the_reference_text_tables(tmp_path, oracle):
    """embedding_builder_test.cc:13-23 builds utest_data/store/quick_embedding and loads the result.  Same files here:
    meta names three tables but its last line has no newline, so -- as the reference's ParseMeta -- two are built; the
    file image holds the hash index the reference's HashTable dumps and the parsed rows."""
    import pyblaze_hip as pb
    d, tables = _reference_text_tables()
    out = str(tmp_path / "ref_tables.qed")
    pb.build_qed(d, "meta", out)
    version, trie, parsed = _parse_qed(out)
    assert version == 2000 and [g for g, _, _ in parsed] == [0, 1]
    for (gid, himg, bimg), name in zip(parsed, ("a_01", "a_02")):
        keys, rows = tables[name]
        assert rows.shape[1] == 9 and len(keys) == {"a_01": 10, "a_02": 51}[name]
        mine = oracle.HashTable(keys.astype(np.uint64), 1 + 4 * 9 * np.arange(len(keys), dtype=np.uint64))
        assert bytes(mine.dump()) == himg
        assert bimg[9:] == rows.tobytes()
        if oracle.have_ref():
            ref = oracle.RefStore(keys, rows)
            assert bytes(ref.hash_dump()) == himg, "differs from the reference's HashTable::Dump"
    if oracle.have_ref():
        assert bytes(oracle.RefTrie(["a_01", "a_02"], [0, 1]).dump()) == trie


# ---------------------------------------------------------------- the synthetic workloads' generator
def test_philox4x32_10_known_answers_and_element_independence():
    """philox.py against the published known-answer vectors of Philox4x32-10 (Random123's kat_vectors: zero, all-ones
    and the digits-of-pi counter / key), and its streams' contract: an element is a function of (seed, stream, index)
    only, whatever range it is asked for in."""
    import philox
    kat = (((0, 0, 0, 0), (0, 0), "6627e8d5 e169c58d bc57ac4c 9b00dbd8"),
           ((0xffffffff, ) * 4, (0xffffffff, ) * 2, "408f276d 41c83b0e a20bc7c6 6d5451fd"),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), "d16cfe09 94fdcceb 5001e420 24126ea1"))
    for ctr, key, want in kat:
        assert " ".join("%08x" % int(x) for x in philox.philox4x32_10(*ctr, *key)) == want
    # vectorised over counters = one call at a time
    st = philox.Stream(7, seed=(0x299f31d0 << 32) | 0xa4093822)
    i = 0x85a308d3243f6a88
    assert [int(x) for x in st.calls(i, 3)[0]] == [int(x) for x in philox.philox4x32_10(i & 0xffffffff, i >> 32, 7, 0, 0xa4093822, 0x299f31d0)]
    # any sub-range, any alignment to the four words of a call, rows of a matrix: the same elements
    whole = st.words(0, 1000)
    for first, n in ((0, 1), (1, 6), (3, 1), (4, 4), (997, 3), (123, 500)):
        assert np.array_equal(st.words(first, n), whole[first:first + n])
    for dim in (16, 18):
        full = philox.host(philox.KIND_NORMAL_F16, st, 40 * dim, 0, 0.1).reshape(40, dim)
        assert np.array_equal(philox.host_rows(philox.KIND_NORMAL_F16, st, [0, 39, 7, 7], dim, 0.1), full[[0, 39, 7, 7]])
    assert np.array_equal(philox.host_rows(philox.KIND_INT8, st, [5], 64), philox.host(philox.KIND_INT8, st, 64, 5 * 64).reshape(1, 64))
    a = philox.Stream(1).words(0, 64)
    assert not np.array_equal(a, philox.Stream(2).words(0, 64)) and not np.array_equal(a, philox.Stream(1, seed=1).words(0, 64))
    # the draws are what they claim to be
    x = philox.Stream(3).normal(0, 1 << 20)
    assert abs(float(x.mean())) < 4e-3 and abs(float(x.std()) - 1.0) < 4e-3 and abs(float((x**4).mean()) - 3.0) < 0.05
    q = philox.Stream(4).int8(0, 1 << 20)
    assert q.min() == -127 and q.max() == 127 and abs(float(q.astype(np.float64).mean())) < 0.3
    u = philox.Stream(5).uniform32(0, 1 << 20, 1e-3, 1e-2)
    assert u.dtype == np.float32 and u.min() >= np.float32(1e-3) and u.max() <= np.float32(1e-2) and abs(float(u.mean()) - 5.5e-3) < 2e-5
    u = philox.Stream(6).uniform(0, 1 << 18)
    assert 0.0 < u.min() and u.max() < 1.0 and abs(u.mean() - 0.5) < 3e-3
    k = philox.Stream(7).integers(0, 1 << 18, 1, 11)
    assert k.min() == 1 and k.max() == 10 and abs(k.mean() - 5.5) < 0.03
    cdf = philox.poisson_cdf(8.0)
    lens = np.searchsorted(cdf, philox.Stream(8).uniform(0, 1 << 18), side="left")
    assert abs(lens.mean() - 8.0) < 0.03 and abs(lens.var() - 8.0) < 0.1


def test_synthetic_configs_come_from_the_generator_streams():
    """Batches and tables of a configuration are the generator's streams: batch b of a longer run equals batch b asked
    for alone, and a table's rows recomputed one by one equal the table."""
    from synth import Config2, Config4
    cfg = Config2(batch=64, rows=3000, slots=3)
    sparse, dense = cfg.batches(3)
    one_s, one_d = cfg.batches(1, seed_offset=2)
    assert np.array_equal(dense[2], one_d[0]) and not np.array_equal(dense[1], one_d[0])
    for (a_ids, _, a_seg), (b_ids, _, b_seg) in zip(sparse[2], one_s[0]):
        assert np.array_equal(a_ids, b_ids) and np.array_equal(a_seg, b_seg)
    assert all(1 <= seg.min() and seg.max() <= 64 for _, _, seg in sparse[0])
    tables = cfg.tables(device="cpu")
    assert np.array_equal(cfg.table_rows(2, [0, 2999, 17]), tables[2][[0, 2999, 17]].numpy())
    c4 = Config4(batch=32, rows=2000, slots=2)
    q, sc = c4.tables(device="cpu")[1]
    rq, rsc = c4.table_rows(1, [1999, 3])
    assert np.array_equal(rq, q[[1999, 3]].numpy()) and np.array_equal(rsc, sc[[1999, 3]].numpy())


@pytest.mark.timeout(600)
def test_file_parsers_under_address_and_undefined_behaviour_sanitizers(tmp_path, kats):
    """The host code that reads files from outside (NetDef text and wire format, the optimizer passes, the Embedding
    config text, the QED builder's text tables) is compiled with -fsanitize=address,undefined and fed seeded mutations
    of the golden inputs (tests/sanitize_host_parsers.cc): rejecting an input is fine, a sanitizer finding aborts."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    csrc = os.path.join(ROOT, "x-deeplearning_amd", "csrc")
    exe = str(tmp_path / "sanitize_host_parsers")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-pthread", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), "-I" + csrc,
           os.path.join(ROOT, "tests", "sanitize_host_parsers.cc")] + [os.path.join(csrc, "blaze", f) for f in
                                                                       ("proto.cc", "optimizer.cc", "common.cc", "qed_builder.cc")] + ["-o", exe]
    subprocess.run(cmd, check=True, capture_output=True, timeout=300)
    # an embedding config of the reference's own operator tests as the seed for that parser
    ec = None
    for case in kats.values():
        for op in case.get("ops", []):
            if "embedding_config" in op.get("args", {}):
                ec = op["args"]["embedding_config"]
                break
        if ec:
            break
    assert ec, "no embedding_config among the reference operator fixtures"
    ec_file = tmp_path / "embedding_config.txt"
    ec_file.write_text(ec)
    golden = os.path.join(ROOT, "tests", "golden")
    nets = [os.path.join(golden, "model_blaze_optimized.bin")] + [os.path.join(golden, "pattern", f) for f in
                                                                  ("parallel_gemm_fusion.blaze", "in_order_gemm_gemm_fusion.blaze",
                                                                   "in_order_gemm_gemm_fusion4.blaze")]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=1")
    r = subprocess.run([exe, "1500", "7", str(tmp_path / "scratch"), os.path.join(golden, "quick_embedding"), str(ec_file)] + nets,
                       capture_output=True, text=True, errors="replace", timeout=500, env=env)
    assert r.returncode == 0 and "sanitize_host_parsers: done" in r.stdout, (r.returncode, r.stderr[-3000:])

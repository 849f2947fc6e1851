"""ctypes/numpy front end of the CPU oracle (oracle/blaze_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark.  The shipped library never imports it.

The C file restates Blaze's CPU implementation function by function; this
module adds the integer layout arithmetic of the Embedding operator
(operator/sparse_op/embedding/embedding_op.h:65-108 in the reference tree) and
numpy-friendly wrappers.  `RefStore` wraps oracle/_ref/libblaze_ref.so, the
reference's own store sources compiled as they are, when that file exists.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libblaze_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libblaze_ref.so")

FP32, FP16, INT8 = 0, 1, 2
SUM, AVG, ASSIGN = 0, 1, 2
ORDER, REVERSE = 0, 1


def build(force=False):
    """Compile the C restatement (and the reference-backed lib when the reference tree is mounted)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(
            os.path.join(_HERE, "blaze_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libblaze_oracle.so"], stdout=subprocess.DEVNULL)
    if os.path.isdir("/root/reference/blaze") and (force or not os.path.exists(_REF_PATH)):
        subprocess.check_call(["make", "-C", _HERE, "-B", "ref"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


class _OrcTable(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("dim", C.c_int32), ("rows", C.c_int64), ("pitch", C.c_int64),
                ("data", C.c_void_p), ("scale", C.c_void_p), ("hash", C.c_void_p)]


class _OrcItem(C.Structure):
    _fields_ = [("udf", C.c_int32), ("trunc_dir", C.c_int32), ("trunc_num", C.c_int32), ("pad_", C.c_int32),
                ("out", C.c_void_p), ("stride", C.c_int64)]


def _declare(l):
    vp, i32, i64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
    l.orc_segments_to_offsets.argtypes = [vp, vp, i64]
    l.orc_half_to_float_n.argtypes = [vp, vp, i64]
    l.orc_float_to_half_n.argtypes = [vp, vp, i64]
    l.orc_hash_bucket_size.argtypes = [C.c_uint32]
    l.orc_hash_bucket_size.restype = C.c_uint32
    l.orc_hash_build.argtypes = [vp, vp, C.c_uint64]
    l.orc_hash_build.restype = vp
    l.orc_hash_free.argtypes = [vp]
    l.orc_hash_lookup.argtypes = [vp, C.c_uint64, C.POINTER(C.c_uint64)]
    l.orc_hash_lookup.restype = C.c_int
    l.orc_hash_dump.argtypes = [vp, vp]
    l.orc_hash_dump.restype = C.c_uint64
    l.orc_embed_get.argtypes = [C.POINTER(_OrcTable), vp, vp, vp, i64, C.POINTER(_OrcItem), i32]
    l.orc_embed_get.restype = C.c_int
    l.orc_gemm_ex.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, f32, vp, C.c_int, vp, C.c_int, f32, vp,
                              C.c_int]
    l.orc_gemm_ex_f64.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, f32, vp, C.c_int, vp, C.c_int, f32, vp,
                                  vp, C.c_int]
    l.orc_gemm_op.argtypes = [C.c_int, C.c_int, f32, f32, vp, C.c_int, vp, vp, vp, vp, i64, vp, vp]
    l.orc_gemm_op.restype = C.c_int
    l.orc_fused_parallel_gemm_op.argtypes = [C.c_int, C.c_int, C.c_int, f32, f32, vp, vp, vp, vp, vp, i64, vp]
    l.orc_fused_parallel_gemm_op.restype = C.c_int
    l.orc_matmul_op.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, vp, i64, vp, i64, vp]
    l.orc_matmul_op.restype = C.c_int
    l.orc_fused_parallel_matmul_op.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, vp, i64, vp, i64,
                                               vp]
    l.orc_fused_parallel_matmul_op.restype = C.c_int
    l.orc_prelu.argtypes = [vp, vp, vp, i64, i64]
    l.orc_dice.argtypes = [vp, vp, vp, vp, vp, i64, i64, C.c_int]
    l.orc_leaky_relu.argtypes = [vp, vp, i64, f32]
    l.orc_sigmoid.argtypes = [vp, vp, i64]
    l.orc_softmax.argtypes = [vp, vp, i64, i64, i64]
    l.orc_reduce_sum.argtypes = [vp, i64, i64, i64, vp]
    l.orc_batch_norm.argtypes = [vp, i64, vp, vp, vp, vp, i64, C.c_int, f32, vp]


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ----------------------------------------------------------------------------- scalar helpers
def half_to_float(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().orc_half_to_float_n(_p(h), _p(out), h.size)
    return out


def float_to_half(f):
    f = _f32(f)
    out = np.empty(f.shape, np.uint16)
    lib().orc_float_to_half_n(_p(f), _p(out), f.size)
    return out


def segments_to_offsets(segments):
    seg = np.ascontiguousarray(segments, dtype=np.int32)
    off = np.empty(seg.size + 1, np.int64)
    lib().orc_segments_to_offsets(_p(seg), _p(off), seg.size)
    return off


# ----------------------------------------------------------------------------- hash index
class HashTable:
    """key -> value index; restates the reference's BulkLoadHashTable + HashTable::Lookup."""

    def __init__(self, keys, values):
        self.keys = np.ascontiguousarray(keys, dtype=np.uint64)
        self.values = np.ascontiguousarray(values, dtype=np.uint64)
        assert self.keys.shape == self.values.shape
        self.h = lib().orc_hash_build(_p(self.keys), _p(self.values), self.keys.size)

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_hash_free(self.h)
            self.h = None

    def lookup(self, key):
        v = C.c_uint64(0)
        ok = lib().orc_hash_lookup(self.h, C.c_uint64(int(key) & 0xFFFFFFFFFFFFFFFF), C.byref(v))
        return int(v.value) if ok else None

    def dump(self):
        n = lib().orc_hash_dump(self.h, None)
        buf = np.empty(n, np.uint8)
        lib().orc_hash_dump(self.h, _p(buf))
        return buf

    @property
    def bucket_size(self):
        return int(lib().orc_hash_bucket_size(self.keys.size))


# ----------------------------------------------------------------------------- tables + pooling
class Table:
    """An embedding table as the oracle sees it: rows of `dim` weights, optional key index.

    data: [rows, dim] float32 | float16 (or uint16 bit patterns) | int8;  scale: [rows] float32 for int8.
    keys: None -> ids are row numbers (id outside [0, rows) = missing); else ids are looked up in a
    HashTable built from keys (value = row number).
    """

    def __init__(self, data, scale=None, keys=None):
        data = np.ascontiguousarray(data)
        if data.dtype == np.float32:
            self.dtype = FP32
        elif data.dtype in (np.float16, np.uint16):
            self.dtype = FP16
        elif data.dtype == np.int8:
            self.dtype = INT8
            assert scale is not None
        else:
            raise TypeError(data.dtype)
        self.data = data
        self.scale = None if scale is None else _f32(scale)
        self.hash = None if keys is None else HashTable(keys, np.arange(len(keys), dtype=np.uint64))
        self.rows, self.dim = data.shape
        self._c = _OrcTable(self.dtype, self.dim, self.rows, data.strides[0], data.ctypes.data,
                            None if self.scale is None else self.scale.ctypes.data,
                            None if self.hash is None else self.hash.h)


def embed_get(table, ids, values, segments, items):
    """One feature group.  items: list of (udf, trunc_dir, trunc_num, block float32 [B, stride] array, col offset).

    Mirrors QuickEmbeddingDict::Get(input, output): the group writes `dim` (sum/avg) or dim*trunc_num
    (assign) floats per sample at column `offset` of each listed block.  table None = unknown table name.
    """
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    values = _f32(values)
    segments = np.ascontiguousarray(segments, dtype=np.int32)
    assert ids.size == values.size == int(segments.sum()), "ids/values/segments disagree"
    arr = (_OrcItem * len(items))()
    for k, (udf, tdir, tnum, block, col) in enumerate(items):
        assert block.dtype == np.float32 and block.flags.c_contiguous and block.ndim == 2
        assert block.shape[0] == segments.size
        arr[k] = _OrcItem(udf, tdir, tnum, 0, block.ctypes.data + 4 * col, block.shape[1])
    rc = lib().orc_embed_get(None if table is None else C.byref(table._c), _p(ids), _p(values), _p(segments),
                             segments.size, arr, len(items))
    assert rc == 0


def embedding_layout(feature_groups, blocks):
    """Block layout arithmetic of EmbeddingOp::InitEmbeddingBlockConfigMeta (embedding_op.h:65-94).

    feature_groups: {fg_name: (table_name, dim)};  blocks: list of lists of dicts
    {fg, udf, trunc_dir, trunc_num}.  Returns (strides, [[(fg, offset, width), ...], ...]).
    """
    strides, placed = [], []
    for blk in blocks:
        off, row = 0, []
        for it in blk:
            if it["fg"] not in feature_groups:
                raise KeyError("feature group config not exist, fg: " + it["fg"])
            dim = feature_groups[it["fg"]][1]
            udf = it.get("udf", SUM)
            if udf in (SUM, AVG):
                width = dim
            elif udf == ASSIGN:
                width = dim * it["trunc_num"]
            else:
                raise ValueError("Unsupported udf type: %r" % udf)
            row.append((it["fg"], off, width))
            off += width
        strides.append(off)
        placed.append(row)
    return strides, placed


def embedding_op(feature_groups, blocks, inputs, tables):
    """The whole Embedding operator on CPU (embedding_op.cc:63-85, embedding_op.h:141-247).

    inputs: {fg: (ids, values, segments)};  tables: {table_name: Table}.
    Returns the list of float32 blocks [B, stride].
    """
    strides, placed = embedding_layout(feature_groups, blocks)
    outs = []
    for bi, blk in enumerate(blocks):
        batch = None
        for it in blk:
            if it["fg"] not in inputs:
                raise KeyError("feature group of block item is not in input list, fg: " + it["fg"])
            b = len(inputs[it["fg"]][2])
            if batch is not None and b != batch:
                raise ValueError("batch size of each feature group in block must be equal")
            batch = b
        outs.append(np.zeros((batch or 0, strides[bi]), np.float32))
    for fg, (tname, dim) in feature_groups.items():
        if fg not in inputs:
            continue
        items = []
        for bi, blk in enumerate(blocks):
            for ii, it in enumerate(blk):
                if it["fg"] == fg:
                    items.append((it.get("udf", SUM), it.get("trunc_dir", REVERSE), it.get("trunc_num", 0), outs[bi],
                                  placed[bi][ii][1]))
        table = tables.get(tname)
        if table is not None:
            assert table.dim == dim
        ids, values, segments = inputs[fg]
        if items:
            embed_get(table, ids, values, segments, items)
    return outs


# ----------------------------------------------------------------------------- dense
def gemm_ex(A, B, transa=False, transb=False, alpha=1.0, beta=0.0, C0=None, f64=False):
    """Row-major cblas_sgemm contract with natural leading dimensions."""
    A, B = _f32(A), _f32(B)
    M, K = (A.shape[1], A.shape[0]) if transa else A.shape
    N = B.shape[0] if transb else B.shape[1]
    if f64:
        out = np.zeros((M, N), np.float64)
        cin = None if C0 is None else _f32(np.broadcast_to(C0, (M, N)))
        lib().orc_gemm_ex_f64(int(transa), int(transb), M, N, K, alpha, _p(A), A.shape[1], _p(B), B.shape[1], beta,
                              None if cin is None else _p(cin), _p(out), N)
        return out
    out = np.zeros((M, N), np.float32) if C0 is None else _f32(np.broadcast_to(C0, (M, N))).copy()
    lib().orc_gemm_ex(int(transa), int(transb), M, N, K, alpha, _p(A), A.shape[1], _p(B), B.shape[1], beta, _p(out), N)
    return out


def gemm_op(A, B, bias=None, transa=False, transb=False, alpha=1.0, beta=1.0):
    A, B = _f32(A), _f32(B)
    a_shape = np.array(A.shape, np.int64)
    b_shape = np.array(B.shape, np.int64)
    y_shape = np.zeros(3, np.int64)
    Mk = A.shape[-2:] if not transa else A.shape[-2:][::-1]
    N = B.shape[0] if transb else B.shape[1]
    ysz = (A.shape[0] if A.ndim == 3 else 1) * Mk[0] * N
    Y = np.zeros(ysz, np.float32)
    cb = None if bias is None else _f32(bias)
    rc = lib().orc_gemm_op(int(transa), int(transb), alpha, beta, _p(A), A.ndim, _p(a_shape), _p(B), _p(b_shape),
                           None if cb is None else _p(cb), 0 if cb is None else cb.size, _p(Y), _p(y_shape))
    if rc != 0:
        raise ValueError("a_k != b_k")
    shp = [int(s) for s in y_shape[:A.ndim]]
    return Y.reshape(shp)


def fused_parallel_gemm_op(A, B, bias=None, parallel_num=2, transa=False, transb=False, alpha=1.0, beta=1.0):
    A, B = _f32(A), _f32(B)
    assert A.ndim == 2
    M = A.shape[1] if transa else A.shape[0]
    N = B.shape[0] // parallel_num if transb else B.shape[1]
    Y = np.zeros((parallel_num * M, N), np.float32)
    cb = None if bias is None else _f32(bias)
    rc = lib().orc_fused_parallel_gemm_op(parallel_num, int(transa), int(transb), alpha, beta, _p(A),
                                          _p(np.array(A.shape, np.int64)), _p(B), _p(np.array(B.shape, np.int64)),
                                          None if cb is None else _p(cb), 0 if cb is None else cb.size, _p(Y))
    if rc != 0:
        raise ValueError("a_k != b_k")
    return Y


def _mm_dims(A, B, transa, transb):
    M, K = A.shape[-2:]
    if transa:
        M, K = K, M
    N = B.shape[-2] if transb else B.shape[-1]
    return int(M), int(N), int(K)


def matmul_op(A, B, transa=False, transb=False, from_deepnet=False):
    A, B = _f32(A), _f32(B)
    if from_deepnet:  # matmul_op.h:147-165
        if B.ndim == 2:
            B = B.reshape(B.shape[0], 1, B.shape[1])
        if A.ndim == 2:
            A = A.reshape(A.shape[0], A.shape[1], 1)
    M, N, K = _mm_dims(A, B, transa, transb)
    ab = int(np.prod(A.shape[:-2], dtype=np.int64))
    bb = int(np.prod(B.shape[:-2], dtype=np.int64))
    outer = A.shape[:-2] if ab >= bb else B.shape[:-2]
    if len(A.shape) - 2 > 1 or len(B.shape) - 2 > 1:
        raise NotImplementedError("Not Implemented BroadcastGemm!")  # math/broadcast.h:240-244
    Cm = np.zeros(tuple(outer) + (M, N), np.float32)
    rc = lib().orc_matmul_op(int(transa), int(transb), M, N, K, _p(A), ab, _p(B), bb, _p(Cm))
    if rc != 0:
        raise ValueError("batch mismatch")
    return Cm


def fused_parallel_matmul_op(A, B, parallel_num=2, transa=False, transb=False):
    A, B = _f32(A), _f32(B)
    M, N, K = _mm_dims(A, B, transa, transb)
    ab = int(np.prod(A.shape[:-2], dtype=np.int64)) // parallel_num
    bb = int(np.prod(B.shape[:-2], dtype=np.int64)) // parallel_num
    cb = max(ab, bb)
    Cm = np.zeros((parallel_num * cb, M, N), np.float32)
    rc = lib().orc_fused_parallel_matmul_op(parallel_num, int(transa), int(transb), M, N, K, _p(A), ab, _p(B), bb,
                                            _p(Cm))
    if rc != 0:
        raise ValueError("batch mismatch")
    return Cm


def prelu(x, w):
    x, w = _f32(x), _f32(w)
    y = np.empty_like(x)
    lib().orc_prelu(_p(x), _p(w), _p(y), x.size, w.size)
    return y


def dice(x, gamma, mean, var, nosqrt=False):
    x, gamma, mean, var = _f32(x), _f32(gamma), _f32(mean), _f32(var)
    y = np.empty_like(x)
    lib().orc_dice(_p(x), _p(gamma), _p(mean), _p(var), _p(y), x.size, gamma.size, int(nosqrt))
    return y


def leaky_relu(x, alpha):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_leaky_relu(_p(x), _p(y), x.size, alpha)
    return y


def sigmoid(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_sigmoid(_p(x), _p(y), x.size)
    return y


def softmax(x, axis=1):
    x = _f32(x)
    n = int(np.prod(x.shape[:axis], dtype=np.int64))
    c = x.shape[axis]
    w = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = np.empty_like(x)
    lib().orc_softmax(_p(x), _p(y), n, c, w)
    return y


# ------------------------------------------------------------- shape / elementwise ops around the attention unit
def reshape(x, shape):
    """Reshape op (operator/op/reshape_op.h:22-52): 0 keeps the input's dim at that position, one negative
    entry is inferred; the output aliases the input."""
    x = np.asarray(x)
    new = []
    unknown = -1
    known = 1
    for i, d in enumerate(shape):
        if d == 0:
            new.append(x.shape[i])
            known *= new[-1]
        elif d < 0:
            assert unknown < 0, "can not support two unknown dims"
            unknown = i
            new.append(-1)
        else:
            new.append(int(d))
            known *= int(d)
    if unknown >= 0:
        new[unknown] = x.size // known
    else:
        assert known == x.size
    return x.reshape(new)


def concat(xs, axis=1):
    """Concat op (operator/op/concat_op.h:46-121, concat_op.cc): same rank, equal dims off the axis."""
    xs = [np.asarray(x) for x in xs]
    assert all(x.ndim == xs[0].ndim and x.dtype == xs[0].dtype for x in xs) and axis < xs[0].ndim
    return np.concatenate(xs, axis=axis)


def _broadcast_shape(a, b):
    """MBroadcasting::BroadcastShape (math/broadcast.h:39-67): right-aligned, dims equal or one of them 1."""
    n = max(len(a), len(b))
    a = (1, ) * (n - len(a)) + tuple(a)
    b = (1, ) * (n - len(b)) + tuple(b)
    out = []
    for x, y in zip(a, b):
        assert x == y or x == 1 or y == 1, "not equal or meet broadcast rule"
        out.append(max(x, y))
    return tuple(out)


def elementwise(op, a, b):
    """Add / Sub / Mul / Div ops (operator/op/elementwise_op.cc:28-165): one IEEE fp32 operation per output
    element under multidirectional broadcasting."""
    a, b = _f32(a), _f32(b)
    shape = _broadcast_shape(a.shape, b.shape)
    a, b = np.broadcast_to(a, shape), np.broadcast_to(b, shape)
    with np.errstate(all="ignore"):
        y = {"Add": np.add, "Sub": np.subtract, "Mul": np.multiply, "Div": np.divide}[op](a, b, dtype=np.float32)
    return np.ascontiguousarray(y)


def broadcast_to(a, like=None, shape=None):
    """BroadcastTo op (operator/op/elementwise_op.h:193-226): to the shape of a second input, or to the `shape`
    argument where entries > 0 replace the input's dim (same rank)."""
    a = np.asarray(a)
    if like is not None:
        target = tuple(np.asarray(like).shape)
    else:
        assert len(shape) == a.ndim
        target = tuple(int(s) if s > 0 else a.shape[i] for i, s in enumerate(shape))
    return np.ascontiguousarray(np.broadcast_to(a, target))


def where(cond, x, y):
    """Where op (operator/op/elementwise_op.h:228-283, elementwise_op.cc WhereKernel): nonzero condition
    (int32 | int64) picks x, else y, all three broadcast together."""
    cond, x, y = np.asarray(cond), _f32(x), _f32(y)
    assert cond.dtype in (np.int32, np.int64)
    shape = _broadcast_shape(_broadcast_shape(cond.shape, x.shape), y.shape)
    return np.ascontiguousarray(np.where(np.broadcast_to(cond, shape) != 0, np.broadcast_to(x, shape), np.broadcast_to(y, shape)))


def split(x, n_out, axis=1, splits=None):
    """Split op (operator/op/split_op.h:33-132, split_op.cc:11-31): `n_out` parts along `axis`, equal unless `splits`
    gives their sizes; RunSplit's walk: for every outer index, the parts' runs of split_size * inner elements follow
    each other in x."""
    x = np.asarray(x)
    assert axis < x.ndim
    if splits is None:
        assert x.shape[axis] % n_out == 0
        splits = [x.shape[axis] // n_out] * n_out
    assert len(splits) == n_out and sum(splits) == x.shape[axis]
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    flat = x.reshape(-1)
    ys = [np.empty(outer * s * inner, x.dtype) for s in splits]
    at, y_off = 0, [0] * n_out
    for _ in range(outer):
        for k, s in enumerate(splits):
            run = s * inner
            ys[k][y_off[k]:y_off[k] + run] = flat[at:at + run]
            at += run
            y_off[k] += run
    return [y.reshape(x.shape[:axis] + (s, ) + x.shape[axis + 1:]) for y, s in zip(ys, splits)]


def gather(data, indices, axis=0):
    """Gather op (operator/op/gather_op.h:45-84, gather_op.cc:9-21): output shape = data.shape[:axis] + indices.shape +
    data.shape[axis+1:]; for every outer index i and every index j a memcpy of inner_size values from
    data + (i * axis_size + indices[j]) * inner_size to y + i * y_inner_size + j * inner_size."""
    data = np.ascontiguousarray(data)
    indices = np.asarray(indices)
    assert np.issubdtype(indices.dtype, np.integer), "indices->data_type()"
    axis_size = data.shape[axis]
    inner = int(np.prod(data.shape[axis + 1:], dtype=np.int64))
    o_shape = list(data.shape[:axis]) + list(indices.shape) + list(data.shape[axis + 1:])
    y_inner = int(indices.size) * inner
    y = np.empty(o_shape, data.dtype)
    outer = y.size // y_inner if y_inner else 0
    src, dst, idx = data.reshape(-1), y.reshape(-1), indices.reshape(-1)
    for i in range(outer):
        so, do = i * axis_size * inner, i * y_inner
        for j in range(idx.size):
            dst[do + j * inner:do + (j + 1) * inner] = src[so + int(idx[j]) * inner:so + (int(idx[j]) + 1) * inner]
    return y


def slice_axis(x, axis=0, start=0, end=1):
    """Slice op (operator/op/slice_op.h:36-110, slice_op.cc:9-29): one axis, [start, end); outer_size memcpys of
    (end - start) * inner_size values, source advancing size * inner_size, destination (end - start) * inner_size."""
    x = np.ascontiguousarray(x)
    assert start < end and axis < x.ndim and end <= x.shape[axis]
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    size = x.shape[axis]
    shape = list(x.shape)
    shape[axis] = end - start
    y = np.empty(shape, x.dtype)
    src, dst = x.reshape(-1), y.reshape(-1)
    x_off, y_off, n = start * inner, 0, (end - start) * inner
    for _ in range(outer):
        dst[y_off:y_off + n] = src[x_off:x_off + n]
        x_off += size * inner
        y_off += n
    return y


def reduce_sum(x, axis=0, keepdims=1):
    """ReduceSum op (operator/op/reduce_sum_op.h:17-58)."""
    x = _f32(x)
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    dim = x.shape[axis]
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    shape = list(x.shape[:axis]) + ([1] if keepdims else []) + list(x.shape[axis + 1:])
    y = np.empty(shape, np.float32)
    lib().orc_reduce_sum(_p(x), outer, dim, inner, _p(y))
    return y


def fuse(x1, x2, comm_index=0):
    """Fuse op (operator/op/fuse_op.h:35-75, fuse_op.cc:11-33): column concat of two 2-D inputs where the
    `comm_index` one has a single row that is repeated for every row of the other."""
    x1, x2 = np.asarray(x1), np.asarray(x2)
    assert x1.ndim == 2 and x2.ndim == 2 and (x1, x2)[comm_index].shape[0] == 1
    m = max(x1.shape[0], x2.shape[0])
    if x1.shape[0] == 1:
        x1 = np.broadcast_to(x1, (m, x1.shape[1]))
    else:
        x2 = np.broadcast_to(x2[:1], (m, x2.shape[1]))
    return np.ascontiguousarray(np.concatenate([x1, x2], axis=1))


def batch_norm(x, gamma, beta, mean, var, eps=0.001, nosqrt=False):
    """BatchNormalization op, inference form (operator/op/batch_normalization_op.cc:11-45)."""
    x, gamma, beta, mean, var = _f32(x), _f32(gamma), _f32(beta), _f32(mean), _f32(var)
    assert gamma.size == beta.size == mean.size == var.size
    y = np.empty_like(x)
    lib().orc_batch_norm(_p(x), x.size, _p(gamma), _p(beta), _p(mean), _p(var), gamma.size, int(nosqrt), eps, _p(y))
    return y


def fc(x, W, bias, act=None, act_params=None, transb=False):
    """One FC layer as Blaze runs it: Gemm op (bias as third input) then a separate activation op."""
    y = gemm_op(x, W, bias, transb=transb)
    if act == "prelu":
        y = prelu(y, act_params[0])
    elif act == "dice":
        y = dice(y, *act_params)
    elif act == "relu":
        y = leaky_relu(y, 0.0)
    elif act == "sigmoid":
        y = sigmoid(y)
    elif act == "softmax":
        y = softmax(y, 1)
    elif act is not None:
        raise ValueError(act)
    return y


# ----------------------------------------------------------------------------- reference-backed store
def have_ref():
    return os.path.exists(_REF_PATH)


class RefStore:
    """fp32 table served by the reference's own HashTable / WeightBlob / UdfProcessor object code."""

    _l = None

    @classmethod
    def _lib(cls):
        if cls._l is None:
            l = C.CDLL(_REF_PATH)
            vp = C.c_void_p
            l.ref_table_build.argtypes = [vp, vp, C.c_int64, C.c_int]
            l.ref_table_build.restype = vp
            l.ref_table_free.argtypes = [vp]
            l.ref_table_lookup.argtypes = [vp, C.c_uint64, C.POINTER(C.c_uint64)]
            l.ref_table_lookup.restype = C.c_int
            l.ref_table_hash_dump.argtypes = [vp, vp]
            l.ref_table_hash_dump.restype = C.c_uint64
            l.ref_table_blob_dump.argtypes = [vp, vp]
            l.ref_table_blob_dump.restype = C.c_uint64
            l.ref_embed_get.argtypes = [vp, vp, vp, vp, C.c_int64, C.POINTER(_OrcItem), C.c_int32]
            l.ref_embed_get.restype = C.c_int
            l.ref_trie_build.argtypes = [C.POINTER(C.c_char_p), vp, C.c_int]
            l.ref_trie_build.restype = vp
            l.ref_trie_free.argtypes = [vp]
            l.ref_trie_lookup.argtypes = [vp, C.c_char_p, C.POINTER(C.c_uint16)]
            l.ref_trie_lookup.restype = C.c_int
            l.ref_trie_dump.argtypes = [vp, vp]
            l.ref_trie_dump.restype = C.c_uint64
            cls._l = l
        return cls._l

    def __init__(self, keys, rows):
        rows = _f32(rows)
        keys = np.ascontiguousarray(keys, dtype=np.int64)
        assert rows.ndim == 2 and rows.shape[0] == keys.size
        self.dim = rows.shape[1]
        self.h = self._lib().ref_table_build(_p(keys), _p(rows), keys.size, self.dim)
        assert self.h, "reference table build failed"

    def __del__(self):
        if getattr(self, "h", None):
            self._lib().ref_table_free(self.h)
            self.h = None

    def lookup(self, key):
        v = C.c_uint64(0)
        ok = self._lib().ref_table_lookup(self.h, C.c_uint64(int(key) & 0xFFFFFFFFFFFFFFFF), C.byref(v))
        return int(v.value) if ok else None

    def hash_dump(self):
        n = self._lib().ref_table_hash_dump(self.h, None)
        buf = np.empty(n, np.uint8)
        self._lib().ref_table_hash_dump(self.h, _p(buf))
        return buf

    def blob_dump(self):
        n = self._lib().ref_table_blob_dump(self.h, None)
        buf = np.empty(n, np.uint8)
        self._lib().ref_table_blob_dump(self.h, _p(buf))
        return buf

    def embed_get(self, ids, values, segments, items):
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        values = _f32(values)
        segments = np.ascontiguousarray(segments, dtype=np.int32)
        arr = (_OrcItem * len(items))()
        for k, (udf, tdir, tnum, block, col) in enumerate(items):
            assert block.dtype == np.float32 and block.flags.c_contiguous
            arr[k] = _OrcItem(udf, tdir, tnum, 0, block.ctypes.data + 4 * col, block.shape[1])
        rc = self._lib().ref_embed_get(self.h, _p(ids), _p(values), _p(segments), segments.size, arr, len(items))
        assert rc == 0


class RefTrie:
    def __init__(self, names, gids):
        l = RefStore._lib()
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        g = np.ascontiguousarray(gids, dtype=np.uint16)
        self.h = l.ref_trie_build(arr, _p(g), len(names))
        assert self.h

    def __del__(self):
        if getattr(self, "h", None):
            RefStore._lib().ref_trie_free(self.h)
            self.h = None

    def lookup(self, name):
        g = C.c_uint16(0)
        ok = RefStore._lib().ref_trie_lookup(self.h, name.encode(), C.byref(g))
        return int(g.value) if ok else None

    def dump(self):
        l = RefStore._lib()
        n = l.ref_trie_dump(self.h, None)
        buf = np.empty(n, np.uint8)
        l.ref_trie_dump(self.h, _p(buf))
        return buf

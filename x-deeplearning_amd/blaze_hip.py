"""ctypes binding of lib/libblaze_hip.so (the C ABI of include/blaze_hip.h) for tests and the benchmark.

PyTorch is used here only to own device memory and streams.  There is no CPU or
PyTorch fallback: if the library is missing or the device is not gfx950 this
module raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libblaze_hip.so")

# enum bz_dtype / bz_udf / bz_trunc / bz_act
F32, I32, I8, I64, F16, BF16 = 1, 2, 7, 10, 12, 100
SUM, AVG, ASSIGN = 0, 1, 2
ORDER, REVERSE = 0, 1
ACT_NONE, ACT_PRELU, ACT_DICE, ACT_LEAKY_RELU, ACT_SIGMOID, ACT_SOFTMAX = 0, 1, 2, 3, 4, 5

EXPORTS = [
    "bz_last_error", "bz_device_check", "bz_table_pitch", "bz_embed_plan", "bz_segments_to_offsets", "bz_segments_to_offsets_slots",
    "bz_embed_pool", "bz_embed_pool_args", "bz_embed_pool_static_scratch", "bz_embed_pool_kernel_name", "bz_fc_fused", "bz_fc_pack_weight", "bz_gemm_strided_batched", "bz_weighted_pool",
    "bz_activation", "bz_concat_cols", "bz_broadcast_op", "bz_reduce_sum", "bz_batch_norm", "bz_softmax_axis",
    "bz_concat_ew", "bz_gather_rows", "bz_spin"
]
EW_ADD, EW_SUB, EW_MUL, EW_DIV, EW_ASSIGN, EW_WHERE = 0, 1, 2, 3, 4, 5
OK, EINVAL, ENOTSUP, EHIP = 0, -22, -95, -5  # bz_status
MAX_RANK = 6


class EmbedSlot(C.Structure):
    _fields_ = [("table", C.c_void_p), ("row_scale", C.c_void_p), ("hash_buckets", C.c_void_p),
                ("hash_pairs", C.c_void_p), ("ids", C.c_void_p), ("values", C.c_void_p), ("segments", C.c_void_p),
                ("offsets", C.c_void_p), ("out", C.c_void_p), ("rows", C.c_int64), ("out_stride", C.c_int64),
                ("nnz", C.c_int64), ("hash_bucket_size", C.c_uint32), ("pitch", C.c_int32), ("dim", C.c_int32), ("table_dtype", C.c_int32),
                ("out_dtype", C.c_int32), ("udf", C.c_int32), ("trunc_dir", C.c_int32), ("trunc_num", C.c_int32),
                ("batch", C.c_int32), ("wg_begin", C.c_int32), ("wg_count", C.c_int32), ("scale_pitch", C.c_int32),
                ("assign_pitch", C.c_int32), ("reserved_", C.c_int32)]


class EmbedLaunch(C.Structure):
    _fields_ = [("n_slots", C.c_int32), ("total_wg", C.c_int32), ("wg_per_slot", C.c_int32), ("variant", C.c_int32),
                ("fused_scan", C.c_int32), ("scan_first", C.c_int32), ("max_batch", C.c_int32), ("reserved_", C.c_int32)]


class FcDesc(C.Structure):
    _fields_ = [("a", C.c_void_p), ("w", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p), ("act_p0", C.c_void_p),
                ("act_p1", C.c_void_p), ("act_p2", C.c_void_p), ("lda", C.c_int64), ("ldw", C.c_int64),
                ("ldy", C.c_int64), ("m", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("in_dtype", C.c_int32),
                ("out_dtype", C.c_int32), ("bias_rows", C.c_int32), ("act", C.c_int32), ("act_size", C.c_int32),
                ("dice_nosqrt", C.c_int32), ("alpha", C.c_float), ("beta", C.c_float), ("act_alpha", C.c_float),
                ("reserved_", C.c_int32), ("head_w", C.c_void_p), ("head_bias", C.c_void_p), ("head_y", C.c_void_p),
                ("head_ldw", C.c_int64), ("head_ldy", C.c_int64), ("head_n", C.c_int32), ("head_act", C.c_int32),
                ("head_out_dtype", C.c_int32), ("n_split", C.c_int32), ("y_split_stride", C.c_int64), ("a_pieces", C.c_void_p), ("next", C.c_void_p)]


class FcNext(C.Structure):
    _fields_ = [("w", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p), ("act_p0", C.c_void_p), ("act_p1", C.c_void_p),
                ("act_p2", C.c_void_p), ("ldw", C.c_int64), ("ldy", C.c_int64), ("n", C.c_int32), ("act", C.c_int32),
                ("act_size", C.c_int32), ("dice_nosqrt", C.c_int32), ("alpha", C.c_float), ("beta", C.c_float),
                ("act_alpha", C.c_float), ("reserved_", C.c_int32)]


class BgemmDesc(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p), ("stride_a", C.c_int64),
                ("stride_b", C.c_int64), ("stride_c", C.c_int64), ("trans_a", C.c_int32), ("trans_b", C.c_int32),
                ("m", C.c_int32), ("n", C.c_int32), ("k", C.c_int32), ("batch", C.c_int32), ("dtype", C.c_int32),
                ("alpha", C.c_float), ("beta", C.c_float)]


class WeightedPoolDesc(C.Structure):
    _fields_ = [("w", C.c_void_p), ("mask", C.c_void_p), ("x", C.c_void_p), ("att", C.c_void_p), ("sum", C.c_void_p),
                ("batch", C.c_int64), ("t", C.c_int32), ("c", C.c_int32), ("dtype", C.c_int32), ("copy_c", C.c_int32),
                ("ld_att", C.c_int64), ("ld_sum", C.c_int64), ("copy_src", C.c_void_p), ("copy_dst", C.c_void_p),
                ("ld_copy_src", C.c_int64), ("ld_copy_dst", C.c_int64)]


class ActDesc(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("p0", C.c_void_p), ("p1", C.c_void_p), ("p2", C.c_void_p),
                ("rows", C.c_int64), ("cols", C.c_int64), ("dtype", C.c_int32), ("act", C.c_int32),
                ("act_size", C.c_int32), ("dice_nosqrt", C.c_int32), ("act_alpha", C.c_float), ("reserved_", C.c_int32)]


class ConcatDesc(C.Structure):
    _fields_ = [("src", C.c_void_p * 16), ("width", C.c_int64 * 16), ("src_pitch", C.c_int64 * 16), ("dst", C.c_void_p),
                ("dst_pitch", C.c_int64), ("rows", C.c_int64), ("n", C.c_int32), ("reserved_", C.c_int32)]


class BcastDesc(C.Structure):
    _fields_ = [("a", C.c_void_p), ("b", C.c_void_p), ("c", C.c_void_p), ("out", C.c_void_p), ("dims", C.c_int64 * 6),
                ("a_stride", C.c_int64 * 6), ("b_stride", C.c_int64 * 6), ("c_stride", C.c_int64 * 6), ("rank", C.c_int32),
                ("op", C.c_int32), ("dtype", C.c_int32), ("cond_dtype", C.c_int32)]


class ConcatEwDesc(C.Structure):
    _fields_ = [("x", C.c_void_p * 8), ("y", C.c_void_p * 8), ("x_stride", (C.c_int64 * 2) * 8), ("y_stride", (C.c_int64 * 2) * 8),
                ("op", C.c_int32 * 8), ("width", C.c_int32 * 8), ("dst", C.c_void_p), ("dst_pitch", C.c_int64),
                ("r0", C.c_int64), ("r1", C.c_int64), ("n", C.c_int32), ("dtype", C.c_int32)]


class BnDesc(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("gamma", C.c_void_p), ("beta", C.c_void_p), ("mean", C.c_void_p),
                ("var", C.c_void_p), ("size", C.c_int64), ("channels", C.c_int64), ("dtype", C.c_int32), ("nosqrt", C.c_int32),
                ("eps", C.c_float), ("reserved_", C.c_int32)]


class BlazeHipError(RuntimeError):
    pass


_lib = None


def lib():
    """Load the library (never builds it: build with __graft_entry__.build() or csrc/Makefile)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise BlazeHipError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                                "(there is no CPU fallback)" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        vp, i32, i64 = C.c_void_p, C.c_int32, C.c_int64
        missing = [name for name in EXPORTS if not hasattr(l, name)]
        if missing:
            raise BlazeHipError("%s does not export %s (stale build?)" % (LIB_PATH, ", ".join(missing)))
        l.bz_last_error.restype = C.c_char_p
        l.bz_device_check.argtypes = [C.c_char_p, C.c_size_t]
        l.bz_table_pitch.argtypes = [i64, C.c_int]
        l.bz_table_pitch.restype = i32
        l.bz_embed_plan.argtypes = [C.POINTER(EmbedSlot), C.c_int, C.POINTER(EmbedLaunch)]
        l.bz_spin.argtypes = [i64, vp]
        l.bz_segments_to_offsets.argtypes = [vp, vp, i64, vp]
        l.bz_segments_to_offsets_slots.argtypes = [vp, C.c_int, vp]
        l.bz_embed_pool.argtypes = [vp, C.POINTER(EmbedLaunch), vp]
        l.bz_embed_pool_static_scratch.argtypes = [vp, C.POINTER(EmbedLaunch), vp]
        l.bz_embed_pool_args.argtypes = [C.POINTER(EmbedSlot), C.POINTER(EmbedLaunch), vp]
        l.bz_embed_pool_kernel_name.restype = C.c_char_p
        l.bz_fc_fused.argtypes = [C.POINTER(FcDesc), vp]
        l.bz_fc_pack_weight.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, C.c_int, i64, vp]
        l.bz_gemm_strided_batched.argtypes = [C.POINTER(BgemmDesc), vp]
        l.bz_weighted_pool.argtypes = [C.POINTER(WeightedPoolDesc), vp]
        l.bz_concat_ew.argtypes = [C.POINTER(ConcatEwDesc), vp]
        l.bz_activation.argtypes = [C.POINTER(ActDesc), vp]
        l.bz_concat_cols.argtypes = [C.POINTER(ConcatDesc), vp]
        l.bz_broadcast_op.argtypes = [C.POINTER(BcastDesc), vp]
        l.bz_reduce_sum.argtypes = [vp, vp, i64, i64, i64, C.c_int, vp]
        l.bz_batch_norm.argtypes = [C.POINTER(BnDesc), vp]
        l.bz_softmax_axis.argtypes = [vp, vp, i64, i64, i64, C.c_int, vp]
        _lib = l
    return _lib


def check(rc):
    if rc != 0:
        raise BlazeHipError("rc=%d: %s" % (rc, lib().bz_last_error().decode()))


def device_check():
    buf = C.create_string_buffer(64)
    check(lib().bz_device_check(buf, 64))
    return buf.value.decode()


def _stream_ptr(stream=None):
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def torch_dtype(dt):
    import torch
    return {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16, I8: torch.int8, I32: torch.int32,
            I64: torch.int64}[dt]


def bz_dtype(t):
    import torch
    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.int8: I8, torch.int32: I32,
            torch.int64: I64}[t]


# ----------------------------------------------------------------------------------- tables
class DeviceTable:
    """An embedding table repacked for the kernels: rows at the pitch bz_table_pitch gives (rows stay inside 128-byte
    lines), zero padding; the per-row scale of an int8 table sits behind the row's elements, in the same line.

    rows: torch tensor [rows, dim] on cuda (float32 | float16 | int8) or a numpy array (uploaded).
    keys: optional int64/uint64 numpy array -> device hash index with the reference's bucket rule.
    pitch: "line" (default), "tight" (row bytes rounded up to 16, scale in an array of its own), or a byte count.
    """

    def __init__(self, rows, scale=None, keys=None, device="cuda", pitch="line"):
        import torch
        if isinstance(rows, np.ndarray):
            if rows.dtype == np.uint16:
                rows = rows.view(np.float16)
            rows = torch.from_numpy(np.ascontiguousarray(rows)).to(device)
        self.dtype = bz_dtype(rows.dtype)
        assert self.dtype in (F32, F16, I8)
        self.rows, self.dim = rows.shape
        esz = rows.element_size()
        row_bytes = self.dim * esz
        in_row_scale = scale is not None and pitch != "tight"
        if pitch == "line":
            self.pitch = lib().bz_table_pitch(row_bytes, 4 if in_row_scale else 0)
        elif pitch == "tight":
            self.pitch = (row_bytes + 15) // 16 * 16
        else:
            self.pitch = int(pitch)
            assert self.pitch % 16 == 0 and self.pitch >= row_bytes + (4 if in_row_scale else 0)
        if self.pitch == row_bytes:
            self.data = rows.contiguous()
        else:
            pad = torch.zeros((self.rows, self.pitch // esz), dtype=rows.dtype, device=device)
            pad[:, :self.dim] = rows
            self.data = pad
        assert self.data.data_ptr() % 16 == 0
        self.scale = None
        self.scale_ptr, self.scale_pitch = None, 0
        if scale is not None:
            if isinstance(scale, np.ndarray):
                scale = torch.from_numpy(np.ascontiguousarray(scale, dtype=np.float32))
            scale = scale.to(device=device, dtype=torch.float32).contiguous()
            if in_row_scale:
                at = (row_bytes + 3) // 4 * 4
                assert self.data.dtype == torch.int8 and at + 4 <= self.pitch
                self.data.view(torch.uint8).view(self.rows, self.pitch)[:, at:at + 4] = scale.view(torch.uint8).view(self.rows, 4)
                self.scale_ptr, self.scale_pitch = self.data.data_ptr() + at, self.pitch
            else:
                self.scale = scale
                self.scale_ptr, self.scale_pitch = scale.data_ptr(), 4
        self.hash_buckets = self.hash_pairs = None
        self.hash_bucket_size = 0
        if keys is not None:
            self._build_hash(np.ascontiguousarray(keys).astype(np.uint64), device)

    def _build_hash(self, keys, device):
        """Device image of BulkLoadHashTable (hashtable.cc:137-187): prime bucket count, pairs sorted by
        (bucket, key), bucket record = offset:40 | size:24 -- with the row number as the value."""
        import torch
        steps = [53, 97, 193, 389, 769, 1543, 3079, 6151, 12289, 24593, 49157, 98317, 196613, 393241, 786433, 1572869,
                 3145739, 6291469, 12582917, 25165843, 50331653, 100663319, 201326611, 402653189, 805306457]
        n = keys.size
        nb = next((s for s in steps if s > n), steps[-1])
        bucket = (keys & np.uint64(0xFFFFFFFF)) % np.uint64(nb)
        order = np.lexsort((keys, bucket))
        sk, sb = keys[order], bucket[order].astype(np.int64)
        pairs = np.empty(2 * n, np.uint64)
        pairs[0::2] = sk
        pairs[1::2] = order.astype(np.uint64)
        counts = np.bincount(sb, minlength=nb).astype(np.uint64)
        first = np.zeros(nb, np.uint64)
        uniq, idx = np.unique(sb, return_index=True)
        first[uniq] = idx.astype(np.uint64) * np.uint64(16)
        rec = (first & np.uint64(0xFFFFFFFFFF)) | (counts << np.uint64(40))
        self.hash_bucket_size = nb
        self.hash_buckets = torch.from_numpy(rec.view(np.int64)).to(device)
        self.hash_pairs = torch.from_numpy(pairs.view(np.int64)).to(device)


# ----------------------------------------------------------------------------------- embedding
class EmbeddingPlan:
    """Device-resident slot descriptors of one Embedding operator invocation.

    items: list of dicts {table: DeviceTable|None, ids, values, segments (cuda tensors), out (cuda tensor
    [B, stride]), col (element offset inside the block), udf, trunc_dir, trunc_num, dim}.
    """

    def __init__(self, items, fused_scan=None):
        """fused_scan: True = the pooling kernel derives offsets from the segments itself (one launch); False = run()
        first scans every slot's segments into an offsets buffer (two launches); None = what bz_embed_plan advises
        for these shapes (launch.scan_first)."""
        import torch
        if fused_scan is None:
            probe = EmbeddingPlan(items, fused_scan=True)
            if not probe.launch.scan_first:
                self.__dict__.update(probe.__dict__)
                return
            fused_scan = False
        self.items = items
        self.fused_scan = fused_scan
        n = len(items)
        arr = (EmbedSlot * n)()
        self.offsets = []
        for i, it in enumerate(items):
            t = it["table"]
            seg, out = it["segments"], it["out"]
            assert seg.dtype == torch.int32 and it["ids"].dtype == torch.int64 and it["values"].dtype == torch.float32
            assert out.dim() == 2 and out.stride(1) == 1
            batch = seg.numel()
            off = None
            if not fused_scan:
                off = torch.empty(batch + 1, dtype=torch.int64, device=out.device)
                self.offsets.append(off)
            s = arr[i]
            if t is not None:
                s.table = t.data.data_ptr()
                s.row_scale = t.scale_ptr
                s.scale_pitch = t.scale_pitch
                s.hash_buckets = t.hash_buckets.data_ptr() if t.hash_buckets is not None else None
                s.hash_pairs = t.hash_pairs.data_ptr() if t.hash_pairs is not None else None
                s.hash_bucket_size = t.hash_bucket_size
                s.rows, s.pitch, s.table_dtype = t.rows, t.pitch, t.dtype
                s.dim = t.dim
            else:
                s.table = None
                s.rows, s.pitch, s.table_dtype = 0, 0, F32
                s.dim = it["dim"]
            s.ids = it["ids"].data_ptr()
            s.values = it["values"].data_ptr()
            s.nnz = it.get("nnz", min(it["ids"].numel(), it["values"].numel()))
            s.segments = seg.data_ptr()
            s.offsets = off.data_ptr() if off is not None else None
            s.out = out.data_ptr() + it.get("col", 0) * out.element_size()
            s.out_stride = out.stride(0)
            s.out_dtype = bz_dtype(out.dtype)
            s.udf = it.get("udf", SUM)
            s.trunc_dir = it.get("trunc_dir", REVERSE)
            s.trunc_num = it.get("trunc_num", 0)
            s.assign_pitch = it.get("assign_pitch", 0)
            s.batch = batch
        self.launch = EmbedLaunch()
        check(lib().bz_embed_plan(arr, n, C.byref(self.launch)))
        self.n, self.total_wg = n, self.launch.total_wg
        self.host = arr
        raw = np.frombuffer(bytes(arr), dtype=np.uint8).copy()
        self.slots_dev = torch.from_numpy(raw).to(items[0]["out"].device)

    def scan(self, stream=None):
        check(lib().bz_segments_to_offsets_slots(self.slots_dev.data_ptr(), self.n, _stream_ptr(stream)))

    def pool(self, stream=None):
        check(lib().bz_embed_pool(self.slots_dev.data_ptr(), C.byref(self.launch), _stream_ptr(stream)))

    def args_eligible(self):
        """what bz_embed_pool_args takes: scan fused in, few slots"""
        return bool(self.launch.fused_scan and not self.launch.scan_first and self.n <= 26)

    def pool_args(self, stream=None):
        """the same launch with the slot records handed over as kernel arguments"""
        check(lib().bz_embed_pool_args(self.host, C.byref(self.launch), _stream_ptr(stream)))

    def run(self, stream=None):
        if not self.fused_scan:
            self.scan(stream)
        self.pool(stream)

    def run_static_scratch(self, stream=None):
        """scan + pool with the offsets in the library's own static buffer (the entry point that allocates nothing)"""
        check(lib().bz_embed_pool_static_scratch(self.slots_dev.data_ptr(), C.byref(self.launch), _stream_ptr(stream)))


def segments_to_offsets(segments, stream=None):
    import torch
    assert segments.dtype == torch.int32 and segments.is_cuda
    off = torch.empty(segments.numel() + 1, dtype=torch.int64, device=segments.device)
    check(lib().bz_segments_to_offsets(segments.data_ptr(), off.data_ptr(), segments.numel(), _stream_ptr(stream)))
    return off


# ----------------------------------------------------------------------------------- dense
def pack_weight(w, trans_b, dst_dtype, stream=None):
    """Blaze weight [K,N] (trans_b False) or [N,K] (True) -> packed [N, ldw] for fc_fused."""
    import torch
    k, n = (w.shape[1], w.shape[0]) if trans_b else (w.shape[0], w.shape[1])
    ldw = (k + 7) // 8 * 8
    dst = torch.empty((n, ldw), dtype=torch_dtype(dst_dtype), device=w.device)
    check(lib().bz_fc_pack_weight(w.data_ptr(), bz_dtype(w.dtype), int(trans_b), k, n, dst.data_ptr(), dst_dtype, ldw,
                                  _stream_ptr(stream)))
    return dst


def fc_fused(a, w_packed, k, bias=None, act=ACT_NONE, act_params=(), out=None, out_dtype=None, alpha=1.0, beta=1.0,
             act_alpha=0.0, dice_nosqrt=False, stream=None, head=None, store_out=True):
    """head: dict(w=packed [n2, ldw] weight of a second layer with n2 <= 8 outputs, bias=fp32 [n2] or None, act=ACT_NONE |
    ACT_SIGMOID | ACT_SOFTMAX, out=tensor [m, n2]) computed in the same launch; then returns (out, head out), and
    store_out=False skips storing the first layer's output (out is returned as None)."""
    import torch
    m = a.shape[0]
    n = w_packed.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=torch_dtype(out_dtype or bz_dtype(a.dtype)), device=a.device)
    d = FcDesc()
    d.a, d.w, d.y = a.data_ptr(), w_packed.data_ptr(), out.data_ptr()
    d.lda, d.ldw, d.ldy = a.stride(0), w_packed.stride(0), out.stride(0)
    d.m, d.n, d.k = m, n, k
    d.in_dtype, d.out_dtype = bz_dtype(a.dtype), bz_dtype(out.dtype)
    assert w_packed.dtype == a.dtype
    if bias is not None:
        assert bias.dtype == torch.float32
        d.bias = bias.data_ptr()
        d.bias_rows = 1 if bias.numel() == n else m
    d.act = act
    ps = list(act_params) + [None] * 3
    for name, p in zip(("act_p0", "act_p1", "act_p2"), ps):
        if p is not None:
            assert p.dtype == torch.float32
            setattr(d, name, p.data_ptr())
    d.act_size = ps[0].numel() if ps[0] is not None else 0
    d.dice_nosqrt = int(dice_nosqrt)
    d.alpha, d.beta, d.act_alpha = alpha, beta, act_alpha
    if head is not None:
        hw, hy = head["w"], head["out"]
        assert hw.dtype == a.dtype and hy.shape[0] == m
        d.head_w, d.head_y, d.head_ldw, d.head_ldy = hw.data_ptr(), hy.data_ptr(), hw.stride(0), hy.stride(0)
        d.head_n, d.head_act, d.head_out_dtype = hw.shape[0], head.get("act", ACT_NONE), bz_dtype(hy.dtype)
        if head.get("bias") is not None:
            assert head["bias"].dtype == torch.float32
            d.head_bias = head["bias"].data_ptr()
        if not store_out:
            d.y = None
    check(lib().bz_fc_fused(C.byref(d), _stream_ptr(stream)))
    if head is not None:
        return (out if store_out else None), head["out"]
    return out


def gemm_strided_batched(a, b, c, m, n, k, batch, stride_a, stride_b, stride_c, trans_a=False, trans_b=False, alpha=1.0,
                         beta=0.0, stream=None):
    d = BgemmDesc()
    d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    d.stride_a, d.stride_b, d.stride_c = stride_a, stride_b, stride_c
    d.trans_a, d.trans_b = int(trans_a), int(trans_b)
    d.m, d.n, d.k, d.batch = m, n, k, batch
    d.dtype = bz_dtype(a.dtype)
    d.alpha, d.beta = alpha, beta
    check(lib().bz_gemm_strided_batched(C.byref(d), _stream_ptr(stream)))
    return c


def weighted_pool(x, w=None, mask=None, want_sum=True, stream=None, att_out=None, sum_out=None, copy=None):
    """x [B, T, C]; w, mask [B, T] (or [B, T, 1]) -> (att [B, C] or None, sum [B, C] or None), see bz_weighted_pool.
    att_out / sum_out: [B, C] views (row stride >= C, unit column stride) to write instead of new tensors;
    copy = (src [B, n] view, dst [B, n] view): the piece copied alongside."""
    import torch
    B, T, Cn = x.shape
    d = WeightedPoolDesc()
    att = (att_out if att_out is not None else torch.empty((B, Cn), dtype=x.dtype, device=x.device)) if w is not None else None
    tot = (sum_out if sum_out is not None else torch.empty((B, Cn), dtype=x.dtype, device=x.device)) if want_sum else None
    for t in (att, tot):
        assert t is None or (tuple(t.shape) == (B, Cn) and t.stride(1) == 1 and t.dtype == x.dtype)
    d.x = x.data_ptr()
    d.w = w.data_ptr() if w is not None else None
    d.mask = mask.data_ptr() if mask is not None else None
    d.att = att.data_ptr() if att is not None else None
    d.sum = tot.data_ptr() if tot is not None else None
    d.ld_att = att.stride(0) if att is not None else 0
    d.ld_sum = tot.stride(0) if tot is not None else 0
    if copy is not None:
        src, dst = copy
        assert src.shape == dst.shape and src.shape[0] == B and src.stride(1) == 1 and dst.stride(1) == 1 and src.dtype == dst.dtype == x.dtype
        d.copy_src, d.copy_dst, d.copy_c = src.data_ptr(), dst.data_ptr(), src.shape[1]
        d.ld_copy_src, d.ld_copy_dst = src.stride(0), dst.stride(0)
    d.batch, d.t, d.c, d.dtype = B, T, Cn, bz_dtype(x.dtype)
    check(lib().bz_weighted_pool(C.byref(d), _stream_ptr(stream)))
    return att, tot


def activation(x, act, params=(), out=None, act_alpha=0.0, dice_nosqrt=False, stream=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    d = ActDesc()
    d.x, d.y = x.data_ptr(), out.data_ptr()
    d.cols = x.shape[-1]
    d.rows = x.numel() // x.shape[-1]
    d.dtype, d.act = bz_dtype(x.dtype), act
    ps = list(params) + [None] * 3
    for name, p in zip(("p0", "p1", "p2"), ps):
        if p is not None:
            setattr(d, name, p.data_ptr())
    d.act_size = ps[0].numel() if ps[0] is not None else 0
    d.dice_nosqrt, d.act_alpha = int(dice_nosqrt), act_alpha
    check(lib().bz_activation(C.byref(d), _stream_ptr(stream)))
    return out


def _bcast_strides(t, out_shape):
    """Element strides of torch tensor `t` seen through `out_shape` (right aligned; 0 on broadcast dims)."""
    n = len(out_shape)
    off = n - t.dim()
    st = [0] * n
    for k in range(t.dim()):
        st[off + k] = 0 if t.shape[k] == 1 else t.stride(k)
    return st


def broadcast_op(op, a, b=None, c=None, out_shape=None, stream=None):
    """Add / Sub / Mul / Div (a, b), BroadcastTo (a -> out_shape), Where (a = int condition, b = x, c = y)."""
    import torch
    ops = [t for t in (a, b, c) if t is not None]
    if out_shape is None:
        out_shape = torch.broadcast_shapes(*[tuple(t.shape) for t in ops])
    val = b if op == EW_WHERE else a
    out = torch.empty(tuple(out_shape), dtype=val.dtype, device=val.device)
    d = BcastDesc()
    d.a, d.out = a.data_ptr(), out.data_ptr()
    d.rank, d.op, d.dtype = len(out_shape), op, bz_dtype(val.dtype)
    for k, n in enumerate(out_shape):
        d.dims[k] = n
    for name, t in (("a_stride", a), ("b_stride", b), ("c_stride", c)):
        if t is not None:
            for k, s in enumerate(_bcast_strides(t, out_shape)):
                getattr(d, name)[k] = s
    if b is not None:
        d.b = b.data_ptr()
    if c is not None:
        d.c = c.data_ptr()
    if op == EW_WHERE:
        d.cond_dtype = bz_dtype(a.dtype)
    check(lib().bz_broadcast_op(C.byref(d), _stream_ptr(stream)))
    return out


def concat_ew(pieces, stream=None):
    """Concat along the last axis of pieces computed on the fly.  pieces: list of (op, x, y) with op one of EW_ADD /
    EW_SUB / EW_MUL / EW_DIV (y a tensor) or EW_ASSIGN (y None); operands are contiguous tensors [r0 | 1, r1 | 1, w]
    broadcast over the two row coordinates.  -> tensor [r0, r1, sum of w]."""
    import torch
    ops = [t for _, x, y in pieces for t in (x, y) if t is not None]
    r0 = max(t.shape[0] for t in ops)
    r1 = max(t.shape[1] for t in ops)
    total = sum(x.shape[2] for _, x, _ in pieces)
    out = torch.empty((r0, r1, total), dtype=ops[0].dtype, device=ops[0].device)
    d = ConcatEwDesc()
    d.n, d.dtype, d.dst, d.dst_pitch, d.r0, d.r1 = len(pieces), bz_dtype(out.dtype), out.data_ptr(), total, r0, r1
    for i, (op, x, y) in enumerate(pieces):
        d.op[i], d.width[i], d.x[i] = op, x.shape[2], x.data_ptr()
        for name, t in (("x_stride", x), ("y_stride", y)):
            if t is None:
                continue
            assert t.is_contiguous() and t.shape[2] == x.shape[2] and t.shape[0] in (1, r0) and t.shape[1] in (1, r1)
            getattr(d, name)[i][0] = 0 if t.shape[0] == 1 and r0 > 1 else t.shape[1] * t.shape[2]
            getattr(d, name)[i][1] = 0 if t.shape[1] == 1 and r1 > 1 else t.shape[2]
        if y is not None:
            d.y[i] = y.data_ptr()
    check(lib().bz_concat_ew(C.byref(d), _stream_ptr(stream)))
    return out


def pieces_desc(pieces, r0, r1, dtype):
    """bz_concat_ew_desc (without a destination) of (op, x, y) pieces with operands [r0 | 1, r1 | 1, w]: what
    bz_fc_desc.a_pieces takes"""
    d = ConcatEwDesc()
    d.n, d.dtype, d.r0, d.r1 = len(pieces), dtype, r0, r1
    for i, (op, x, y) in enumerate(pieces):
        d.op[i], d.width[i], d.x[i] = op, x.shape[2], x.data_ptr()
        for name, t in (("x_stride", x), ("y_stride", y)):
            if t is None:
                continue
            getattr(d, name)[i][0] = 0 if t.shape[0] == 1 and r0 > 1 else t.shape[1] * t.shape[2]
            getattr(d, name)[i][1] = 0 if t.shape[1] == 1 and r1 > 1 else t.shape[2]
        if y is not None:
            d.y[i] = y.data_ptr()
    return d


class AttentionMlp:
    """DIN's attention MLP as ONE bz_fc_fused launch (a_pieces + next + head): rows [q, k, q - k, q * k] of a history
    k [r0, r1, w] against a target q [r0, 1, w] -> layer 1 + Dice -> layer 2 + Dice -> a skinny head into `out`
    [r0 * r1, n3] (fp32).  Weights are packed [n, ld] tensors (pack_weight), biases and Dice triples fp32."""

    def __init__(self, q, k, w1, b1, dice1, w2, b2, dice2, w3, b3, out, head_act=ACT_NONE):
        r0, r1, w = k.shape
        self.keep = (q, k, w1, b1, dice1, w2, b2, dice2, w3, b3, out)
        dt = bz_dtype(k.dtype)
        self.pieces = pieces_desc([(EW_ASSIGN, q, None), (EW_ASSIGN, k, None), (EW_SUB, q, k), (EW_MUL, q, k)], r0, r1, dt)
        nx = self.next = FcNext()
        nx.w, nx.ldw, nx.n, nx.bias = w2.data_ptr(), w2.stride(0), w2.shape[0], b2.data_ptr()
        nx.alpha = nx.beta = 1.0
        nx.act, nx.act_size = ACT_DICE, w2.shape[0]
        nx.act_p0, nx.act_p1, nx.act_p2 = (t.data_ptr() for t in dice2)
        d = self.desc = FcDesc()
        d.a_pieces = C.cast(C.pointer(self.pieces), C.c_void_p)
        d.next = C.cast(C.pointer(nx), C.c_void_p)
        d.w, d.ldw, d.bias = w1.data_ptr(), w1.stride(0), b1.data_ptr()
        d.m, d.n, d.k, d.ldy = r0 * r1, w1.shape[0], 4 * w, w1.shape[0]
        d.in_dtype = d.out_dtype = dt
        d.bias_rows, d.alpha, d.beta = 1, 1.0, 1.0
        d.act, d.act_size = ACT_DICE, w1.shape[0]
        d.act_p0, d.act_p1, d.act_p2 = (t.data_ptr() for t in dice1)
        d.head_w, d.head_ldw, d.head_bias = w3.data_ptr(), w3.stride(0), b3.data_ptr()
        d.head_y, d.head_ldy, d.head_n = out.data_ptr(), out.stride(0), w3.shape[0]
        d.head_act, d.head_out_dtype = head_act, bz_dtype(out.dtype)
        self.flops = 2.0 * r0 * r1 * (4 * w * w1.shape[0] + w1.shape[0] * w2.shape[0] + w2.shape[0] * w3.shape[0])

    def run(self, stream=None):
        check(lib().bz_fc_fused(C.byref(self.desc), _stream_ptr(stream)))


def reduce_sum(x, axis, keepdims=True, stream=None):
    import torch
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    shape = list(x.shape[:axis]) + ([1] if keepdims else []) + list(x.shape[axis + 1:])
    y = torch.empty(shape, dtype=x.dtype, device=x.device)
    check(lib().bz_reduce_sum(x.data_ptr(), y.data_ptr(), outer, x.shape[axis], inner, bz_dtype(x.dtype), _stream_ptr(stream)))
    return y


def batch_norm(x, gamma, beta, mean, var, eps=0.001, nosqrt=False, stream=None):
    import torch
    y = torch.empty_like(x)
    d = BnDesc()
    d.x, d.y = x.data_ptr(), y.data_ptr()
    d.gamma, d.beta, d.mean, d.var = gamma.data_ptr(), beta.data_ptr(), mean.data_ptr(), var.data_ptr()
    d.size, d.channels, d.dtype, d.nosqrt, d.eps = x.numel(), gamma.numel(), bz_dtype(x.dtype), int(nosqrt), eps
    check(lib().bz_batch_norm(C.byref(d), _stream_ptr(stream)))
    return y


def softmax_axis(x, axis, stream=None):
    import torch
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = torch.empty_like(x)
    check(lib().bz_softmax_axis(x.data_ptr(), y.data_ptr(), outer, x.shape[axis], inner, bz_dtype(x.dtype), _stream_ptr(stream)))
    return y

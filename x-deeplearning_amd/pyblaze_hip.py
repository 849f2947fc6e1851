"""ctypes binding of the Blaze_* predictor ABI (include/blaze_c_api.h) exported by lib/libblaze_hip.so.

Same method names as the reference's python binding (blaze/binding/python/pyblaze/predictor.py: Predictor,
PredictorManager) so scripts written against it read the same; used by the tests and the benchmark.  Also
carries NetDef text builders for programmatically built models.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libblaze_hip.so")

# blaze DataType wire values (blaze/proto/blaze.proto:6-19)
K_FLOAT, K_INT32, K_INT8, K_INT64, K_FLOAT16 = 1, 2, 7, 10, 12
_NP = {K_FLOAT: np.float32, K_INT32: np.int32, K_INT64: np.int64, K_FLOAT16: np.float16, K_INT8: np.int8}

EXPORTS = [
    "Blaze_GetLastErrorString", "Blaze_SetLastErrorString", "Blaze_InitScheduler", "Blaze_PredictorManagerCreate",
    "Blaze_PredictorManagerDelete", "Blaze_PredictorManagerSetDataType", "Blaze_PredictorManagerSetRunMode",
    "Blaze_LoadSparseModelWeight", "Blaze_PredcitorManagerLoadModel", "Blaze_PredictorManagerLoadModel",
    "Blaze_PredictorManagerLoadDeepNetModel", "Blaze_PredictorCreate", "Blaze_PredictorDelete",
    "Blaze_PredictorReshapeInput", "Blaze_PredictorFeed", "Blaze_PredictorForward", "Blaze_PredictorOutputShape",
    "Blaze_PredictorOutputDataType", "Blaze_PredictorOutput", "Blaze_PredictorParamName", "Blaze_PredictorParamShape",
    "Blaze_PredictorParamDataType", "Blaze_PredictorParam", "Blaze_PredictorListInputNames",
    "Blaze_PredictorListOutputNames", "Blaze_PredictorRegisterObservers", "Blaze_PredictorDumpObservers",
    "Blaze_ConvertBlaze", "Blaze_OptimizeBlaze", "Blaze_QuickEmbeddingBuildFp32", "Blaze_QuickEmbeddingBuildFp16",
    "Blaze_HipStoreAddTable", "Blaze_PredictorManagerLoadModelFromString", "Blaze_PredictorInputDevicePtr",
    "Blaze_PredictorOutputDevicePtr", "Blaze_PredictorForwardN", "Blaze_ConvertNetDef", "Blaze_ServePoolCreate",
    "Blaze_ServePoolRun", "Blaze_ServePoolDelete", "Blaze_ServePoolSetDepth", "Blaze_ServePoolLatencies", "Blaze_PredictorForwardLaunch",
    "Blaze_PredictorForwardWait", "Blaze_PredictorFeedMany", "Blaze_AllocationCount", "Blaze_HipStoreGet", "Blaze_ServePoolStreamQueues"
]


class BlazeError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise BlazeError("%s is missing: build it first (there is no CPU fallback)" % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        vp, cp, i, sz = C.c_void_p, C.c_char_p, C.c_int, C.c_size_t
        l.Blaze_GetLastErrorString.argtypes = [C.POINTER(cp)]
        l.Blaze_PredictorManagerCreate.argtypes = [C.POINTER(vp)]
        l.Blaze_PredictorManagerDelete.argtypes = [vp]
        l.Blaze_PredictorManagerSetDataType.argtypes = [vp, i]
        l.Blaze_PredictorManagerSetRunMode.argtypes = [vp, cp]
        l.Blaze_LoadSparseModelWeight.argtypes = [vp, cp]
        l.Blaze_PredcitorManagerLoadModel.argtypes = [vp, cp, i]
        l.Blaze_PredictorManagerLoadModel.argtypes = [vp, cp, i]
        l.Blaze_PredictorManagerLoadModelFromString.argtypes = [vp, cp, sz, i]
        l.Blaze_PredictorManagerLoadDeepNetModel.argtypes = [vp, cp, cp, i]
        l.Blaze_PredictorCreate.argtypes = [vp, i, i, C.POINTER(vp)]
        l.Blaze_PredictorDelete.argtypes = [vp]
        l.Blaze_PredictorReshapeInput.argtypes = [vp, cp, C.POINTER(i), i]
        l.Blaze_PredictorFeed.argtypes = [vp, cp, vp, i]
        l.Blaze_PredictorForward.argtypes = [vp]
        l.Blaze_PredictorForwardN.argtypes = [vp, i]
        l.Blaze_PredictorOutputShape.argtypes = [vp, cp, C.POINTER(sz), C.POINTER(C.POINTER(sz))]
        l.Blaze_PredictorOutputDataType.argtypes = [vp, cp, C.POINTER(i)]
        l.Blaze_PredictorOutput.argtypes = [vp, cp, vp, sz]
        l.Blaze_PredictorParamName.argtypes = [vp, C.POINTER(sz), C.POINTER(C.POINTER(cp))]
        l.Blaze_PredictorParamShape.argtypes = [vp, cp, C.POINTER(sz), C.POINTER(C.POINTER(sz))]
        l.Blaze_PredictorParamDataType.argtypes = [vp, cp, C.POINTER(i)]
        l.Blaze_PredictorParam.argtypes = [vp, cp, vp, sz]
        l.Blaze_PredictorListInputNames.argtypes = [vp, C.POINTER(sz), C.POINTER(C.POINTER(cp))]
        l.Blaze_PredictorListOutputNames.argtypes = [vp, C.POINTER(sz), C.POINTER(C.POINTER(cp))]
        l.Blaze_PredictorRegisterObservers.argtypes = [vp, sz, C.POINTER(cp)]
        l.Blaze_PredictorDumpObservers.argtypes = [vp, C.POINTER(sz), C.POINTER(C.POINTER(cp)), C.POINTER(C.POINTER(cp))]
        l.Blaze_QuickEmbeddingBuildFp32.argtypes = [cp, cp, cp, i]
        l.Blaze_QuickEmbeddingBuildFp16.argtypes = [cp, cp, cp, i]
        l.Blaze_HipStoreAddTable.argtypes = [vp, cp, i, C.c_int64, i, vp, i, vp, vp]
        l.Blaze_HipStoreGet.argtypes = [vp, cp, vp, vp, sz, vp, i, i, vp, vp, vp, vp, vp, i]
        l.Blaze_ConvertNetDef.argtypes = [cp, sz, i, i, vp, sz, C.POINTER(sz)]
        l.Blaze_OptimizeBlaze.argtypes = [cp, cp, i]
        l.Blaze_PredictorInputDevicePtr.argtypes = [vp, cp, C.POINTER(vp)]
        l.Blaze_PredictorOutputDevicePtr.argtypes = [vp, cp, C.POINTER(vp)]
        l.Blaze_ServePoolCreate.argtypes = [i, C.POINTER(vp)]
        l.Blaze_ServePoolRun.argtypes = [vp, C.POINTER(vp), i, C.c_int64]
        l.Blaze_ServePoolDelete.argtypes = [vp]
        l.Blaze_ServePoolSetDepth.argtypes = [vp, i]
        l.Blaze_ServePoolLatencies.argtypes = [vp, C.POINTER(C.c_float), C.c_int64, C.POINTER(C.c_int64)]
        l.Blaze_PredictorForwardLaunch.argtypes = [vp]
        l.Blaze_PredictorForwardWait.argtypes = [vp]
        l.Blaze_PredictorFeedMany.argtypes = [vp, i, C.POINTER(C.c_char_p), C.POINTER(vp), C.POINTER(C.c_size_t)]
        l.Blaze_AllocationCount.argtypes = [C.POINTER(C.c_int64)]
        _lib = l
    return _lib


def allocation_count():
    """device / pinned-host allocations the library has made in this process so far"""
    n = C.c_int64()
    check_call(lib().Blaze_AllocationCount(C.byref(n)))
    return n.value


def last_error():
    msg = C.c_char_p()
    lib().Blaze_GetLastErrorString(C.byref(msg))
    return (msg.value or b"").decode(errors="replace")


def check_call(rc):
    if rc != 0:
        raise BlazeError(last_error())


def _names(fn, handle):
    n = C.c_size_t()
    arr = C.POINTER(C.c_char_p)()
    check_call(fn(handle, C.byref(n), C.byref(arr)))
    return [arr[i].decode() for i in range(n.value)]


class Predictor(object):
    def __init__(self, handle):
        self.handle = handle

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:  # module globals are gone at interpreter exit
            lib().Blaze_PredictorDelete(self.handle)
            self.handle = None

    def reshape_input(self, name, shape):
        arr = (C.c_int * len(shape))(*[int(s) for s in shape])
        check_call(lib().Blaze_PredictorReshapeInput(self.handle, name.encode(), arr, len(shape)))

    def feed(self, name, data):
        data = np.ascontiguousarray(data)
        self.reshape_input(name, data.shape)
        check_call(lib().Blaze_PredictorFeed(self.handle, name.encode(), data.ctypes.data_as(C.c_void_p), data.nbytes))

    def feed_raw(self, name, data, nbytes):
        """Feed without reshaping (to exercise the length check of the ABI)."""
        data = np.ascontiguousarray(data)
        check_call(lib().Blaze_PredictorFeed(self.handle, name.encode(), data.ctypes.data_as(C.c_void_p), nbytes))

    @staticmethod
    def feed_batch(items):
        """items: [(name, contiguous numpy array)] -> an object for feed_many (argument arrays built once; it keeps
        the arrays alive)."""
        arrays = [np.ascontiguousarray(a) for _, a in items]
        n = len(items)
        names = (C.c_char_p * n)(*[name.encode() for name, _ in items])
        data = (C.c_void_p * n)(*[a.ctypes.data for a in arrays])
        lens = (C.c_size_t * n)(*[a.nbytes for a in arrays])
        return (n, names, data, lens, arrays)

    def feed_many(self, batch):
        """Feed every input of a feed_batch in one call; the shapes must already be set (a first feed() does)."""
        check_call(lib().Blaze_PredictorFeedMany(self.handle, batch[0], batch[1], batch[2], batch[3]))

    def forward(self):
        check_call(lib().Blaze_PredictorForward(self.handle))

    def forward_launch(self):
        """Queue the pass on the calling thread's stream; forward_wait (same thread) returns when it has finished."""
        check_call(lib().Blaze_PredictorForwardLaunch(self.handle))

    def forward_wait(self):
        check_call(lib().Blaze_PredictorForwardWait(self.handle))

    def forward_n(self, count):
        check_call(lib().Blaze_PredictorForwardN(self.handle, count))

    def output_shape(self, name):
        n = C.c_size_t()
        p = C.POINTER(C.c_size_t)()
        check_call(lib().Blaze_PredictorOutputShape(self.handle, name.encode(), C.byref(n), C.byref(p)))
        return tuple(p[i] for i in range(n.value))

    def list_input_names(self):
        return _names(lib().Blaze_PredictorListInputNames, self.handle)

    def list_output_names(self):
        return _names(lib().Blaze_PredictorListOutputNames, self.handle)

    def output_dtype(self, name):
        dt = C.c_int()
        check_call(lib().Blaze_PredictorOutputDataType(self.handle, name.encode(), C.byref(dt)))
        return _NP[dt.value]

    def output_asnumpy(self, name):
        out = np.empty(self.output_shape(name), self.output_dtype(name))
        check_call(lib().Blaze_PredictorOutput(self.handle, name.encode(), out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def list_internal_names(self):
        return _names(lib().Blaze_PredictorParamName, self.handle)

    def internal_shape(self, name):
        n = C.c_size_t()
        p = C.POINTER(C.c_size_t)()
        check_call(lib().Blaze_PredictorParamShape(self.handle, name.encode(), C.byref(n), C.byref(p)))
        return tuple(p[i] for i in range(n.value))

    def internal_dtype(self, name):
        dt = C.c_int()
        check_call(lib().Blaze_PredictorParamDataType(self.handle, name.encode(), C.byref(dt)))
        return _NP[dt.value]

    def internal_asnumpy(self, name):
        out = np.empty(self.internal_shape(name), self.internal_dtype(name))
        check_call(lib().Blaze_PredictorParam(self.handle, name.encode(), out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def register_observers(self, observer_names):
        arr = (C.c_char_p * len(observer_names))(*[n.encode() for n in observer_names])
        check_call(lib().Blaze_PredictorRegisterObservers(self.handle, len(observer_names), arr))

    def dump_observers(self):
        n = C.c_size_t()
        k = C.POINTER(C.c_char_p)()
        v = C.POINTER(C.c_char_p)()
        check_call(lib().Blaze_PredictorDumpObservers(self.handle, C.byref(n), C.byref(k), C.byref(v)))
        return {k[i].decode(): v[i].decode() for i in range(n.value)}

    def input_device_ptr(self, name):
        p = C.c_void_p()
        check_call(lib().Blaze_PredictorInputDevicePtr(self.handle, name.encode(), C.byref(p)))
        return p.value

    def output_device_ptr(self, name):
        p = C.c_void_p()
        check_call(lib().Blaze_PredictorOutputDevicePtr(self.handle, name.encode(), C.byref(p)))
        return p.value


class ServePool(object):
    """Persistent serving threads inside the library; run(predictors, steps) executes pass i on predictor
    i % len(predictors) and thread i % n_threads, returning when all passes have finished on the device."""

    def __init__(self, n_threads, depth=None):
        """depth: passes a thread keeps queued on its stream (library default 2; 1 = synchronous Forward calls)."""
        self.handle = C.c_void_p()
        self.n_threads = n_threads
        check_call(lib().Blaze_ServePoolCreate(n_threads, C.byref(self.handle)))
        if depth is not None:
            check_call(lib().Blaze_ServePoolSetDepth(self.handle, depth))

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib().Blaze_ServePoolDelete(self.handle)
            self.handle = None

    def run(self, predictors, steps):
        arr = (C.c_void_p * len(predictors))(*[getattr(p.handle, "value", p.handle) for p in predictors])
        check_call(lib().Blaze_ServePoolRun(self.handle, arr, len(predictors), steps))

    def set_depth(self, depth):
        check_call(lib().Blaze_ServePoolSetDepth(self.handle, depth))

    def stream_queues(self):
        """the hardware-queue group of each thread's stream, as the pool measured it at its first job ([] before)"""
        n = C.c_int(0)
        check_call(lib().Blaze_ServePoolStreamQueues(self.handle, None, 0, C.byref(n)))
        out = (C.c_int * max(n.value, 1))()
        check_call(lib().Blaze_ServePoolStreamQueues(self.handle, out, n.value, C.byref(n)))
        return list(out[:n.value])

    def latencies_ms(self):
        """per-pass latency (launch to the return of the wait) of the last run, all threads, as a float32 array"""
        n = C.c_int64(0)
        check_call(lib().Blaze_ServePoolLatencies(self.handle, None, 0, C.byref(n)))
        out = np.empty(n.value, np.float32)
        check_call(lib().Blaze_ServePoolLatencies(self.handle, out.ctypes.data_as(C.POINTER(C.c_float)), n.value, C.byref(n)))
        return out


class PredictorManager(object):
    def __init__(self):
        self.handle = C.c_void_p()
        check_call(lib().Blaze_PredictorManagerCreate(C.byref(self.handle)))

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib().Blaze_PredictorManagerDelete(self.handle)
            self.handle = None

    def set_data_type(self, data_type=np.float32):
        check_call(lib().Blaze_PredictorManagerSetDataType(self.handle, K_FLOAT16 if data_type == np.float16 else K_FLOAT))

    def set_run_mode(self, run_mode):
        check_call(lib().Blaze_PredictorManagerSetRunMode(self.handle, run_mode.encode()))

    def load_sparse_model_weight(self, path):
        check_call(lib().Blaze_LoadSparseModelWeight(self.handle, path.encode()))

    def load_model(self, blaze_model_file, optimization_pass=0):
        check_call(lib().Blaze_PredcitorManagerLoadModel(self.handle, blaze_model_file.encode(), optimization_pass))

    def load_model_from_string(self, data, is_text=True):
        if isinstance(data, str):
            data = data.encode()
        check_call(lib().Blaze_PredictorManagerLoadModelFromString(self.handle, data, len(data), int(is_text)))

    def load_deepnet_model(self, conf_file, param_file, optimization_pass=0):
        check_call(lib().Blaze_PredictorManagerLoadDeepNetModel(self.handle, conf_file.encode(), param_file.encode(),
                                                                optimization_pass))

    def add_table(self, name, rows, keys=None, scale=None):
        """rows: numpy [n, dim] float32/float16/int8, or a torch cuda tensor (then scale must be one too)."""
        on_device = not isinstance(rows, np.ndarray)
        if on_device:
            import torch
            vt = {torch.float32: K_FLOAT, torch.float16: K_FLOAT16, torch.int8: K_INT8}[rows.dtype]
            rows = rows.contiguous()
            rp, n, dim = rows.data_ptr(), rows.shape[0], rows.shape[1]
            sp = scale.contiguous().data_ptr() if scale is not None else None
        else:
            rows = np.ascontiguousarray(rows)
            vt = {np.dtype(np.float32): K_FLOAT, np.dtype(np.float16): K_FLOAT16, np.dtype(np.int8): K_INT8}[rows.dtype]
            rp, n, dim = rows.ctypes.data, rows.shape[0], rows.shape[1]
            if scale is not None:
                scale = np.ascontiguousarray(scale, dtype=np.float32)
            sp = scale.ctypes.data if scale is not None else None
        kp = None
        if keys is not None:
            keys = np.ascontiguousarray(keys).astype(np.int64)
            kp = keys.ctypes.data
        check_call(lib().Blaze_HipStoreAddTable(self.handle, name.encode(), vt, n, dim, rp, int(on_device), kp, sp))

    def store_get(self, table, ids, key_num, values, dim, items):
        """The store's host-memory Get for one feature group.  ids int64 [sum(key_num)], key_num int32 [batch], values
        float32 like ids: numpy arrays.  items: list of (udf, trunc_direction, trunc_num, block, column): block is a
        C-contiguous numpy [batch, stride] float32 or float16 array written in place from column `column` on."""
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        key_num = np.ascontiguousarray(key_num, dtype=np.int32)
        values = np.ascontiguousarray(values, dtype=np.float32)
        n = len(items)
        dt = items[0][3].dtype if n else np.dtype(np.float32)
        udf, tdir, tnum = ((C.c_int * n)(*[it[k] for it in items]) for k in range(3))
        outs, strides = (C.c_void_p * n)(), (C.c_size_t * n)()
        for k, (_, _, _, block, col) in enumerate(items):
            assert block.flags.c_contiguous and block.ndim == 2 and block.dtype == dt and block.shape[0] == key_num.size
            outs[k] = block.ctypes.data + col * block.itemsize
            strides[k] = block.shape[1]
        check_call(lib().Blaze_HipStoreGet(self.handle, table.encode(), ids.ctypes.data, key_num.ctypes.data, key_num.size,
                                           values.ctypes.data, dim, n, udf, tdir, tnum, outs, strides,
                                           K_FLOAT if dt == np.float32 else K_FLOAT16))

    def create_predictor(self, device_type=1, device_id=0):
        h = C.c_void_p()
        check_call(lib().Blaze_PredictorCreate(self.handle, device_type, device_id, C.byref(h)))
        p = Predictor(h)
        p._manager = self  # the manager owns the workspace (weights and blobs) the predictor points into
        return p


def optimize_blaze(raw_model_file, optimized_model_file, binary=True):
    """Blaze_OptimizeBlaze: model file (binary or text NetDef) -> optimized model file."""
    check_call(lib().Blaze_OptimizeBlaze(raw_model_file.encode(), optimized_model_file.encode(), int(binary)))


def convert_netdef(data, in_is_text, out_is_text):
    if isinstance(data, str):
        data = data.encode()
    n = C.c_size_t()
    check_call(lib().Blaze_ConvertNetDef(data, len(data), int(in_is_text), int(out_is_text), None, 0, C.byref(n)))
    buf = C.create_string_buffer(n.value + 1)
    check_call(lib().Blaze_ConvertNetDef(data, len(data), int(in_is_text), int(out_is_text), buf, n.value, C.byref(n)))
    return buf.raw[:n.value]


def build_qed(path, meta, output_file, fp16=False, thread_num=1):
    fn = lib().Blaze_QuickEmbeddingBuildFp16 if fp16 else lib().Blaze_QuickEmbeddingBuildFp32
    check_call(fn(path.encode(), meta.encode(), output_file.encode(), thread_num))


# --------------------------------------------------------------------------------------------- NetDef text
def _fmt_float(v):
    return repr(float(np.float32(v)))


class NetBuilder:
    """Builds a text-format NetDef (the format of the reference's operator test fixtures)."""

    def __init__(self, name="net", device_type=1, run_mode="simple"):
        self.lines = ['name : "%s"' % name, 'run_mode : "%s"' % run_mode,
                      "device_option { device_type : %d device_id : 0 }" % device_type]

    def external_input(self, name, dtype):
        self.lines.append('external_input { name : "%s" dtype : %d }' % (name, dtype))

    def external_output(self, name, dtype=K_FLOAT):
        self.lines.append('external_output { name : "%s" dtype : %d }' % (name, dtype))

    def arg(self, name, i):
        self.lines.append('arg { name : "%s" i : %d }' % (name, i))

    def constant(self, name, array, dtype=None):
        array = np.asarray(array)
        if dtype is None:
            dtype = {np.dtype(np.float32): K_FLOAT, np.dtype(np.float64): K_FLOAT, np.dtype(np.float16): K_FLOAT16,
                     np.dtype(np.int32): K_INT32, np.dtype(np.int64): K_INT64}[array.dtype]
        shape = " ".join("ints : %d" % d for d in array.shape)
        if dtype in (K_FLOAT, K_FLOAT16):
            vals = " ".join("floats : %s" % _fmt_float(v) for v in array.reshape(-1))
        else:
            vals = " ".join("ints : %d" % int(v) for v in array.reshape(-1))
        self.lines.append('op { name : "%s_fill" type : "ConstantFill" arg { name : "shape" %s } arg { name : "dtype" i : %d } '
                          'arg { name : "value" %s } output : "%s" }' % (name, shape, dtype, vals, name))

    def op(self, type_, inputs, outputs, name=None, **args):
        parts = ['op { name : "%s" type : "%s"' % (name or (type_.lower() + "_" + outputs[0]), type_)]
        parts += ['input : "%s"' % i for i in inputs]
        parts += ['output : "%s"' % o for o in outputs]
        for k, v in args.items():
            if isinstance(v, bool):
                parts.append('arg { name : "%s" i : %d }' % (k, int(v)))
            elif isinstance(v, int):
                parts.append('arg { name : "%s" i : %d }' % (k, v))
            elif isinstance(v, float):
                parts.append('arg { name : "%s" f : %s }' % (k, _fmt_float(v)))
            elif isinstance(v, str):
                esc = v.replace("\\", "\\\\").replace('"', '\\"').replace("\n", "\\n")
                parts.append('arg { name : "%s" s : "%s" }' % (k, esc))
            elif isinstance(v, (list, tuple)) and all(isinstance(e, int) for e in v):
                parts.append('arg { name : "%s" %s }' % (k, " ".join("ints : %d" % e for e in v)))
            elif isinstance(v, (list, tuple)):
                parts.append('arg { name : "%s" %s }' % (k, " ".join("floats : %s" % _fmt_float(float(e)) for e in v)))
            else:
                raise TypeError((k, v))
        parts.append("}")
        self.lines.append(" ".join(parts))

    def text(self):
        return "\n".join(self.lines) + "\n"


def embedding_config_text(feature_groups, blocks):
    """feature_groups: [(fg, table, dim)]; blocks: [[dict(fg, udf, trunc_dir, trunc_num)]]."""
    out = []
    for fg, table, dim in feature_groups:
        out.append('feature_group_config { feature_group : "%s" table_name : "%s" dim : %d }' % (fg, table, dim))
    for blk in blocks:
        items = []
        for it in blk:
            s = 'embedding_block_config_item { feature_group : "%s" udf_type : %d' % (it["fg"], it.get("udf", 0))
            if "trunc_dir" in it:
                s += " trunc_direction : %d" % it["trunc_dir"]
            if "trunc_num" in it:
                s += " trunc_num : %d" % it["trunc_num"]
            items.append(s + " }")
        out.append("block_config { %s }" % " ".join(items))
    return "\n".join(out)

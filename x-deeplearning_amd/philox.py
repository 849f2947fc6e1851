"""Counter-based random numbers for the synthetic workloads: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random
numbers: as easy as 1, 2, 3", SC'11; multipliers and Weyl constants as published there).

Every value is a pure function of (seed, stream id, index), so the host and the device regenerate any element on their
own: tables of tens of gigabytes are filled on the device by csrc/synth/philox_fill.hip and a parity test recomputes
only the rows a batch touched, here, with the same integer arithmetic.  Stream ids: slot index for tables, 1000 + slot
for ids, 2000 + slot for lengths, 3000 + layer for weights, 4000 for dense features.

Host-side harness code (bench.py, the smoke check, the full-size parity tests); not part of the drop-in library.
"""
import ctypes as C
import os

import numpy as np

SEED = 20240613
_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint64(0x9E3779B9), np.uint64(0xBB67AE85)
_MASK = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Ten rounds on counters (arrays or scalars, values below 2**32) under key (k0, k1) -> four uint64 arrays holding
    the 32-bit output words."""
    c = [np.asarray(x, dtype=np.uint64) for x in (c0, c1, c2, c3)]
    k0, k1 = np.uint64(k0), np.uint64(k1)
    for r in range(10):
        if r:
            k0, k1 = (k0 + _W0) & _MASK, (k1 + _W1) & _MASK
        p0, p1 = _M0 * c[0], _M1 * c[2]  # both factors below 2**32: the 64-bit product is exact
        c = [(p1 >> _S32) ^ c[1] ^ k0, p1 & _MASK, (p0 >> _S32) ^ c[3] ^ k1, p0 & _MASK]
    return c


_quantiles = None


def normal_quantiles():
    """65 536 quantiles of N(0, 1) at (i + 0.5) / 65536, as float32: a normal draw is a lookup with the top 16 bits of a
    word, the same lookup on the host and on the device (no logarithm or cosine whose last bit could differ)."""
    global _quantiles
    if _quantiles is None:
        from scipy.special import ndtri
        _quantiles = ndtri((np.arange(65536, dtype=np.float64) + 0.5) / 65536.0).astype(np.float32)
    return _quantiles


class Stream:
    """The sequence of one (seed, stream id).  Call i of the generator has counter (i mod 2**32, i div 2**32, stream id, 0)
    and key (seed mod 2**32, seed div 2**32).  `packed` draws use all four words of a call (element e = word e % 4 of
    call e // 4); the others use one call per element."""

    def __init__(self, stream_id, seed=SEED):
        self.stream_id, self.seed = int(stream_id), int(seed)

    def calls(self, first, n):
        """-> uint64 [n, 4]: the output words of calls first .. first + n - 1"""
        i = np.uint64(first) + np.arange(n, dtype=np.uint64)
        w = philox4x32_10(i & _MASK, i >> _S32, np.uint64(self.stream_id), np.uint64(0), self.seed & 0xFFFFFFFF, self.seed >> 32)
        return np.stack(w, axis=1)

    def words(self, first, n):
        """packed: uint64 [n] holding the 32-bit words of elements first .. first + n - 1"""
        c0 = first // 4
        w = self.calls(c0, (first + n + 3) // 4 - c0).reshape(-1)
        return w[first - 4 * c0:first - 4 * c0 + n]

    def row_words(self, rows, dim):
        """packed: uint64 [len(rows), dim], the words of rows `rows` of a [*, dim] tensor filled from element 0 (only the
        calls those rows need are computed)"""
        rows = np.asarray(rows, dtype=np.uint64)
        if dim % 4 == 0:
            i = (rows[:, None] * np.uint64(dim // 4) + np.arange(dim // 4, dtype=np.uint64)[None, :]).reshape(-1)
            w = philox4x32_10(i & _MASK, i >> _S32, np.uint64(self.stream_id), np.uint64(0), self.seed & 0xFFFFFFFF, self.seed >> 32)
            return np.stack(w, axis=1).reshape(len(rows), dim)
        e = rows[:, None] * np.uint64(dim) + np.arange(dim, dtype=np.uint64)[None, :]
        i = (e >> np.uint64(2)).reshape(-1)
        w = np.stack(philox4x32_10(i & _MASK, i >> _S32, np.uint64(self.stream_id), np.uint64(0), self.seed & 0xFFFFFFFF, self.seed >> 32), axis=1)
        return w[np.arange(i.size), (e & np.uint64(3)).reshape(-1).astype(np.int64)].reshape(len(rows), dim)

    def normal(self, first, n, sigma=1.0):
        """packed: float32 [n], quantile[word >> 16] * sigma (one float32 multiplication)"""
        q = normal_quantiles()[(self.words(first, n) >> np.uint64(16)).astype(np.int64)]
        return q * np.float32(sigma)

    def int8(self, first, n):
        """packed: int8 [n] uniform over -127 .. 127: (word * 255) div 2**32 - 127"""
        return (((self.words(first, n) * np.uint64(255)) >> _S32).astype(np.int64) - 127).astype(np.int8)

    def uniform32(self, first, n, lo, hi):
        """packed: float32 [n], lo + ((word >> 8) * 2**-24) * (hi - lo): float32 product rounded, then float32 sum"""
        u = (self.words(first, n) >> np.uint64(8)).astype(np.float32) * np.float32(2.0**-24)
        return np.float32(lo) + u * (np.float32(hi) - np.float32(lo))

    def uniform(self, first, n):
        """float64 [n] in (0, 1) with 53 bits, from words 0 and 1 of one call per element (host-side draws: ids, lengths)"""
        w = self.calls(first, n)
        return (((w[:, 0] >> np.uint64(5)) * np.uint64(1 << 26) + (w[:, 1] >> np.uint64(6))).astype(np.float64) + 0.5) * 2.0**-53

    def integers(self, first, n, lo, hi):
        """int64 [n] uniform over lo .. hi - 1: lo + (word 0 * (hi - lo)) div 2**32, one call per element"""
        w = self.calls(first, n)[:, 0]
        return (w * np.uint64(hi - lo) >> _S32).astype(np.int64) + lo


def poisson_cdf(lam, kmax=256):
    k = np.arange(kmax, dtype=np.float64)
    logp = -lam + k * np.log(lam) - np.cumsum(np.log(np.maximum(k, 1.0)))
    cdf = np.cumsum(np.exp(logp))
    return cdf / cdf[-1]


# ---------------------------------------------------------------------------------------------------------------
# device side: lib/libblaze_synth.so (csrc/synth/philox_fill.hip), for tensors too large to come from the host
# ---------------------------------------------------------------------------------------------------------------
_lib = None
_quantiles_dev = {}


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libblaze_synth.so")
        if not os.path.exists(path):
            raise RuntimeError("libblaze_synth.so is missing: build it with `make -C x-deeplearning_amd/csrc` (there is no other "
                               "source of device-generated tables)")
        _lib = C.CDLL(path)
        _lib.bz_synth_fill.restype = C.c_int
        _lib.bz_synth_fill.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_uint64, C.c_uint32, C.c_float, C.c_float,
                                       C.c_void_p, C.c_void_p]
    return _lib


KIND_NORMAL_F32, KIND_NORMAL_F16, KIND_INT8, KIND_UNIFORM_F32 = 0, 1, 2, 3


def fill(t, kind, stream, first=0, a=1.0, b=0.0):
    """Fill the contiguous CUDA tensor t (element e of it = element first + e of the stream) on torch's current stream.
    kind NORMAL_*: quantile * a; INT8: -127 .. 127; UNIFORM_F32: over [a, b)."""
    import torch
    assert t.is_cuda and t.is_contiguous()
    want = {KIND_NORMAL_F32: torch.float32, KIND_NORMAL_F16: torch.float16, KIND_INT8: torch.int8, KIND_UNIFORM_F32: torch.float32}[kind]
    assert t.dtype == want, (t.dtype, want)
    dev = t.device.index or 0
    if dev not in _quantiles_dev:
        _quantiles_dev[dev] = torch.from_numpy(normal_quantiles()).to(t.device)
    rc = lib().bz_synth_fill(t.data_ptr(), kind, t.numel(), first, stream.seed, stream.stream_id, a, b,
                             _quantiles_dev[dev].data_ptr(), torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise RuntimeError("bz_synth_fill failed with %d" % rc)
    return t


def host(kind, stream, n, first=0, a=1.0, b=0.0):
    """The same elements computed here (numpy)."""
    if kind == KIND_NORMAL_F32:
        return stream.normal(first, n, a)
    if kind == KIND_NORMAL_F16:
        return stream.normal(first, n, a).astype(np.float16)
    if kind == KIND_INT8:
        return stream.int8(first, n)
    return stream.uniform32(first, n, a, b)


def host_rows(kind, stream, rows, dim, a=1.0, b=0.0):
    """Rows `rows` of the [*, dim] tensor that tensor() / fill() make from element 0 of the stream, computed here."""
    w = stream.row_words(rows, dim)
    if kind in (KIND_NORMAL_F32, KIND_NORMAL_F16):
        x = normal_quantiles()[(w >> np.uint64(16)).astype(np.int64)] * np.float32(a)
        return x.astype(np.float16) if kind == KIND_NORMAL_F16 else x
    if kind == KIND_INT8:
        return (((w * np.uint64(255)) >> _S32).astype(np.int64) - 127).astype(np.int8)
    u = (w >> np.uint64(8)).astype(np.float32) * np.float32(2.0**-24)
    return np.float32(a) + u * (np.float32(b) - np.float32(a))


def tensor(shape, kind, stream, device, a=1.0, b=0.0):
    """A tensor of that shape filled from element 0 of the stream: on the device by the fill kernel, on the CPU by numpy -
    the same bits either way."""
    import torch
    dt = {KIND_NORMAL_F32: torch.float32, KIND_NORMAL_F16: torch.float16, KIND_INT8: torch.int8, KIND_UNIFORM_F32: torch.float32}[kind]
    n = int(np.prod(shape))
    if str(device).startswith("cuda"):
        return fill(torch.empty(shape, dtype=dt, device=device), kind, stream, 0, a, b)
    out = np.empty(n, dtype=host(kind, stream, 1, 0, a, b).dtype)
    step = 1 << 22
    for s in range(0, n, step):
        out[s:s + step] = host(kind, stream, min(step, n - s), s, a, b)
    return torch.from_numpy(out.reshape(shape))

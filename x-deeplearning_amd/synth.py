"""Synthetic CTR workloads shaped like the benchmark configurations (seeded, reproducible).

Host-side harness code for bench.py, the smoke check and the full-size parity tests: it builds
device-resident tables, batches of sparse inputs (<fg>.ids / .values / .segments triples, the
reference's input layout: blaze/operator/common_helper.h:96-98) and MLP weights.

Every number comes from the counter-based generator of philox.py, keyed by (seed, stream id, index): seed = SEED +
1000003 * configuration number; stream id = slot for tables (5000 + slot for an int8 table's scales), 1000 + slot for
ids, 2000 + slot for lengths, 3000 + layer for weights, 4000 for dense features; index = position, with the batch
number in its upper 32 bits for per-batch data.  Tables are filled on the device and can be recomputed row by row on
the host with the same bits.
"""
import numpy as np

import philox
from philox import SEED, Stream


def config_seed(number):
    return SEED + 1000003 * number


class BoundedZipf:
    """Zipf(s) over ranks 1..n by inverse CDF; rank r lands on row ((r-1) * 2654435761) mod n so hot rows
    are scattered over the table instead of clustered at its head."""

    def __init__(self, n, s):
        w = np.arange(1, n + 1, dtype=np.float64)**(-s)
        self.cdf = np.cumsum(w)
        self.cdf /= self.cdf[-1]
        self.n = n

    def sample(self, u):
        """u: uniform draws in (0, 1) -> rows"""
        ranks = np.minimum(np.searchsorted(self.cdf, u, side="left"), self.n - 1).astype(np.int64)
        return (ranks * 2654435761) % self.n


class UniformIds:
    """ids uniform over the table's rows (config 5)"""

    def __init__(self, n):
        self.n = n

    def sample(self, u):
        return np.minimum((u * self.n).astype(np.int64), self.n - 1)


_POISSON = {}


def lengths(stream, first, kind, batch):
    """per-sample id counts of one slot: elements first .. first + batch - 1 of the slot's length stream"""
    if kind in ("poisson8", "poisson20"):  # config 2 (clipped to 1..64) / config 4 (0 allowed): inverse CDF
        lam = 8 if kind == "poisson8" else 20
        if lam not in _POISSON:
            _POISSON[lam] = philox.poisson_cdf(float(lam))
        k = np.searchsorted(_POISSON[lam], stream.uniform(first, batch), side="left")
        return (np.clip(k, 1, 64) if kind == "poisson8" else k).astype(np.int32)
    hi = {"u1_10": 11, "u1_4": 5, "u1_50": 51}[kind]  # configs 1, 5, 3
    return stream.integers(first, batch, 1, hi).astype(np.int32)


def sparse_batch(seed, batch_index, ids_of, slots, batch, length_kind):
    """Batch number batch_index: list over slots of (ids int64 [nnz], values float32 [nnz] == 1, segments int32 [batch]).
    ids_of: BoundedZipf or UniformIds."""
    out = []
    first = int(batch_index) << 32
    for s in range(slots):
        seg = lengths(Stream(2000 + s, seed), first, length_kind, batch)
        nnz = int(seg.sum())
        out.append((ids_of.sample(Stream(1000 + s, seed).uniform(first, nnz)), np.ones(nnz, np.float32), seg))
    return out


def normal_weights(seed, layer, k, n, device):
    """fp32 master weight [k, n] N(0, 1/sqrt(k)) and bias [n] N(0, 0.01) of a layer, as torch tensors"""
    import torch
    st = Stream(3000 + layer, seed)
    w = st.normal(0, k * n, np.float32(1.0 / np.sqrt(k))).reshape(k, n)
    b = st.normal(k * n, n, 0.01)
    return torch.from_numpy(w).to(device), torch.from_numpy(b).to(device)


def embedding_bytes(batches_nnz, batch, slots, row_bytes, scale_bytes, out_cols, out_elem):
    """Algorithmic bytes of one Embedding launch: per id one row (+scale) + 8 B id + 4 B value, per sample 4 B of
    segments per slot, plus the pooled block written once.  No cache credit."""
    return batches_nnz * (row_bytes + scale_bytes + 12) + slots * batch * 4 + batch * out_cols * out_elem


class Config2:
    """26 slots x [1M, 32] fp16, Poisson(8) lengths in [1,64], Zipf(1.1), ksum; 64 dense features;
    MLP 896-512-256-2, PReLU(0.25), softmax; fp16 MFMA with fp32 accumulate; batch 2048."""
    name = "config2: 26x[1M,32] fp16 ksum + MLP 896-512-256-2 PReLU softmax, batch 2048"
    batch, slots, rows, dim, dense = 2048, 26, 1_000_000, 32, 64
    layers = (896, 512, 256, 2)
    zipf_s, length_kind = 1.1, "poisson8"

    def __init__(self, batch=None, rows=None, slots=None):
        self.batch = batch or self.batch
        self.rows = rows or self.rows
        self.slots = slots or self.slots
        self.in_dim = self.dense + self.slots * self.dim
        self.layers = (self.in_dim, ) + tuple(self.layers[1:])

    table_dtype = "float16"
    number = 2

    @property
    def seed(self):
        return config_seed(self.number)

    def tables(self, device="cuda"):
        """[rows, dim] N(0, 0.01) per slot, rounded to the table type"""
        kind = philox.KIND_NORMAL_F16 if self.table_dtype == "float16" else philox.KIND_NORMAL_F32
        return [philox.tensor((self.rows, self.dim), kind, Stream(s, self.seed), device, 0.01) for s in range(self.slots)]

    def table_rows(self, slot, rows):
        """rows (int array) of slot's table recomputed on the host -> [len(rows), dim] of the table type"""
        kind = philox.KIND_NORMAL_F16 if self.table_dtype == "float16" else philox.KIND_NORMAL_F32
        return philox.host_rows(kind, Stream(slot, self.seed), rows, self.dim, 0.01)

    def mlp(self, device="cuda"):
        """fp32 master weights [K,N] N(0, 1/sqrt(fan_in)), bias N(0, 0.01), PReLU slope 0.25 per channel."""
        import torch
        out = []
        for li in range(len(self.layers) - 1):
            w, b = normal_weights(self.seed, li, self.layers[li], self.layers[li + 1], device)
            out.append((w, b, torch.full((self.layers[li + 1], ), 0.25).to(device)))
        return out

    def batches(self, n, seed_offset=0):
        """batches seed_offset .. seed_offset + n - 1 of the configuration's input stream"""
        zipf = BoundedZipf(self.rows, self.zipf_s)
        sparse = [sparse_batch(self.seed, seed_offset + b, zipf, self.slots, self.batch, self.length_kind) for b in range(n)]
        dense = [Stream(4000, self.seed).normal((seed_offset + b) << 32, self.batch * self.dense).reshape(self.batch, self.dense)
                 for b in range(n)]
        return sparse, dense


class Config1(Config2):
    """10 slots x [1M, 16] fp32, U{1..10} lengths, Zipf(1.1), ksum; 32 dense features; MLP 192-200-80-2, PReLU(0.25),
    softmax; everything fp32; batch 128 -- the configuration the reference's CPU path can run as is."""
    name = "config1: 10x[1M,16] fp32 ksum + MLP 192-200-80-2 PReLU softmax, batch 128"
    batch, slots, rows, dim, dense = 128, 10, 1_000_000, 16, 32
    layers = (192, 200, 80, 2)
    zipf_s, length_kind = 1.1, "u1_10"
    table_dtype = "float32"
    number = 1


class Config4:
    """50 slots x [10M, 64] int8 + one fp32 scale per row, Poisson(20) lengths (0 allowed), Zipf(1.05), kavg into an
    fp16 block [4096, 3200]; no dense part.  Tables are generated on the device (34 GB)."""
    name = "config4: 50x[10M,64] int8+scale kavg, batch 4096"
    batch, slots, rows, dim = 4096, 50, 10_000_000, 64
    zipf_s, length_kind = 1.05, "poisson20"

    def __init__(self, batch=None, rows=None, slots=None):
        self.batch, self.rows, self.slots = batch or self.batch, rows or self.rows, slots or self.slots

    seed = config_seed(4)

    def tables(self, device="cuda"):
        """-> list of (int8 [rows, dim] uniform over -127 .. 127, fp32 scale [rows] uniform over [1e-3, 1e-2)) torch tensors."""
        return [(philox.tensor((self.rows, self.dim), philox.KIND_INT8, Stream(s, self.seed), device),
                 philox.tensor((self.rows, ), philox.KIND_UNIFORM_F32, Stream(5000 + s, self.seed), device, 1e-3, 1e-2))
                for s in range(self.slots)]

    def table_rows(self, slot, rows):
        """rows (int array) of slot's table recomputed on the host -> (int8 [len(rows), dim], fp32 scale [len(rows)])"""
        return (philox.host_rows(philox.KIND_INT8, Stream(slot, self.seed), rows, self.dim),
                philox.host_rows(philox.KIND_UNIFORM_F32, Stream(5000 + slot, self.seed), rows, 1, 1e-3, 1e-2).reshape(-1))

    def batch_inputs(self, seed_offset=0):
        return sparse_batch(self.seed, seed_offset, BoundedZipf(self.rows, self.zipf_s), self.slots, self.batch, self.length_kind)


class Config5:
    """200 slots x [4M, 64] fp16, U{1..4} lengths, uniform ids, ksum into a bf16 block [8192, 12800];
    MLP 12800-1024-512-256-1 in bf16 with fp32 accumulation, bias + ReLU, sigmoid head.  Tables are
    generated on the device (102 GB)."""
    name = "config5: 200x[4M,64] fp16 ksum + MLP 12800-1024-512-256-1 bf16 ReLU sigmoid, batch 8192"
    batch, slots, rows, dim = 8192, 200, 4_000_000, 64
    layers = (12800, 1024, 512, 256, 1)
    length_kind = "u1_4"

    def __init__(self, batch=None, rows=None, slots=None):
        self.batch, self.rows, self.slots = batch or self.batch, rows or self.rows, slots or self.slots
        self.layers = (self.slots * self.dim, ) + tuple(self.layers[1:])

    seed = config_seed(5)

    def tables(self, device="cuda"):
        return [philox.tensor((self.rows, self.dim), philox.KIND_NORMAL_F16, Stream(s, self.seed), device, 0.01)
                for s in range(self.slots)]

    def table_rows(self, slot, rows):
        """rows (int array) of slot's table recomputed on the host -> fp16 [len(rows), dim]"""
        return philox.host_rows(philox.KIND_NORMAL_F16, Stream(slot, self.seed), rows, self.dim, 0.01)

    def batch_inputs(self, seed_offset=0):
        return sparse_batch(self.seed, seed_offset, UniformIds(self.rows), self.slots, self.batch, self.length_kind)

    def mlp(self, device="cuda"):
        """fp32 master weights [K,N] N(0, 1/sqrt(fan_in)), bias N(0, 0.01)."""
        return [normal_weights(self.seed, li, self.layers[li], self.layers[li + 1], device) for li in range(len(self.layers) - 1)]

"""Synthetic CTR workloads shaped like the benchmark configurations (seeded, reproducible).

Host-side harness code for bench.py, the smoke check and the full-size parity tests: it builds
device-resident tables, batches of sparse inputs (<fg>.ids / .values / .segments triples, the
reference's input layout: blaze/operator/common_helper.h:96-98) and MLP weights.
"""
import numpy as np

SEED = 20240613


class BoundedZipf:
    """Zipf(s) over ranks 1..n by inverse CDF; rank r lands on row ((r-1) * 2654435761) mod n so hot rows
    are scattered over the table instead of clustered at its head."""

    def __init__(self, n, s):
        w = np.arange(1, n + 1, dtype=np.float64)**(-s)
        self.cdf = np.cumsum(w)
        self.cdf /= self.cdf[-1]
        self.n = n

    def sample(self, rng, size):
        ranks = np.searchsorted(self.cdf, rng.random(size), side="left").astype(np.int64)
        return (ranks * 2654435761) % self.n


def lengths(rng, kind, batch):
    if kind == "poisson8":  # config 2
        return np.clip(rng.poisson(8, batch), 1, 64).astype(np.int32)
    if kind == "poisson20":  # config 4 (0 allowed)
        return rng.poisson(20, batch).astype(np.int32)
    if kind == "u1_10":  # config 1
        return rng.integers(1, 11, batch).astype(np.int32)
    if kind == "u1_4":  # config 5
        return rng.integers(1, 5, batch).astype(np.int32)
    if kind == "u1_50":  # config 3
        return rng.integers(1, 51, batch).astype(np.int32)
    raise ValueError(kind)


def sparse_batch(rng, zipf, slots, batch, length_kind):
    """One batch: list over slots of (ids int64 [nnz], values float32 [nnz] == 1, segments int32 [batch])."""
    out = []
    for _ in range(slots):
        seg = lengths(rng, length_kind, batch)
        nnz = int(seg.sum())
        out.append((zipf.sample(rng, nnz), np.ones(nnz, np.float32), seg))
    return out


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

    def tables(self, device="cuda"):
        import torch
        g = torch.Generator(device=device).manual_seed(SEED)
        return [(torch.randn((self.rows, self.dim), generator=g, device=device) * 0.01).to(getattr(torch, self.table_dtype))
                for _ in range(self.slots)]

    def mlp(self, device="cuda"):
        """fp32 master weights [K,N] N(0, 1/sqrt(fan_in)), bias N(0, 0.01), PReLU slope 0.25 per channel."""
        import torch
        g = torch.Generator(device="cpu").manual_seed(SEED + 3000)
        out = []
        for li in range(len(self.layers) - 1):
            k, n = self.layers[li], self.layers[li + 1]
            w = torch.randn((k, n), generator=g) / np.sqrt(k)
            b = torch.randn(n, generator=g) * 0.01
            slope = torch.full((n, ), 0.25)
            out.append((w.to(device), b.to(device), slope.to(device)))
        return out

    def batches(self, n, seed_offset=0):
        rng = np.random.default_rng(SEED + 1000 + seed_offset)
        zipf = BoundedZipf(self.rows, self.zipf_s)
        sparse = [sparse_batch(rng, zipf, self.slots, self.batch, self.length_kind) for _ in range(n)]
        dense = [rng.standard_normal((self.batch, self.dense)).astype(np.float32) for _ in range(n)]
        return sparse, dense


class Config1(Config2):
    """10 slots x [1M, 16] fp32, U{1..10} lengths, Zipf(1.1), ksum; 32 dense features; MLP 192-200-80-2, PReLU(0.25),
    softmax; everything fp32; batch 128 -- the configuration the reference's CPU path can run as is."""
    name = "config1: 10x[1M,16] fp32 ksum + MLP 192-200-80-2 PReLU softmax, batch 128"
    batch, slots, rows, dim, dense = 128, 10, 1_000_000, 16, 32
    layers = (192, 200, 80, 2)
    zipf_s, length_kind = 1.1, "u1_10"
    table_dtype = "float32"


class Config4:
    """50 slots x [10M, 64] int8 + one fp32 scale per row, Poisson(20) lengths (0 allowed), Zipf(1.05), kavg into an
    fp16 block [4096, 3200]; no dense part.  Tables are generated on the device (34 GB)."""
    name = "config4: 50x[10M,64] int8+scale kavg, batch 4096"
    batch, slots, rows, dim = 4096, 50, 10_000_000, 64
    zipf_s, length_kind = 1.05, "poisson20"

    def __init__(self, batch=None, rows=None, slots=None):
        self.batch, self.rows, self.slots = batch or self.batch, rows or self.rows, slots or self.slots

    def tables(self, device="cuda"):
        """-> list of (int8 [rows, dim], fp32 scale [rows]) torch tensors."""
        import torch
        g = torch.Generator(device=device).manual_seed(SEED + 4)
        out = []
        for _ in range(self.slots):
            q = torch.randint(-127, 128, (self.rows, self.dim), dtype=torch.int8, device=device, generator=g)
            sc = torch.rand(self.rows, device=device, generator=g) * 9e-3 + 1e-3
            out.append((q, sc))
        return out

    def batch_inputs(self, seed_offset=0):
        rng = np.random.default_rng(SEED + 1004 + seed_offset)
        return sparse_batch(rng, BoundedZipf(self.rows, self.zipf_s), self.slots, self.batch, self.length_kind)


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

    def tables(self, device="cuda"):
        import torch
        g = torch.Generator(device=device).manual_seed(SEED + 5)
        return [(torch.randn((self.rows, self.dim), generator=g, device=device) * 0.01).to(torch.float16)
                for _ in range(self.slots)]

    def batch_inputs(self, seed_offset=0):
        rng = np.random.default_rng(SEED + 1005 + seed_offset)
        out = []
        for _ in range(self.slots):
            seg = lengths(rng, self.length_kind, self.batch)
            nnz = int(seg.sum())
            out.append((rng.integers(0, self.rows, nnz).astype(np.int64), np.ones(nnz, np.float32), seg))
        return out

    def mlp(self, device="cuda"):
        """fp32 master weights [K,N] N(0, 1/sqrt(fan_in)), bias N(0, 0.01)."""
        import torch
        g = torch.Generator(device="cpu").manual_seed(SEED + 3005)
        out = []
        for li in range(len(self.layers) - 1):
            k, n = self.layers[li], self.layers[li + 1]
            out.append(((torch.randn((k, n), generator=g) / np.sqrt(k)).to(device), (torch.randn(n, generator=g) * 0.01).to(device)))
        return out

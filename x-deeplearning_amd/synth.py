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

    def tables(self, device="cuda"):
        import torch
        g = torch.Generator(device=device).manual_seed(SEED)
        return [(torch.randn((self.rows, self.dim), generator=g, device=device) * 0.01).to(torch.float16)
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

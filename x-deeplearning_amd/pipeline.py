"""The CTR forward pass (Embedding -> FC stack -> softmax head) as prebuilt C-ABI calls.

Harness for bench.py / smoke: every descriptor is built once, a step is four calls into
libblaze_hip.so (pool with fused scan, FC, FC, FC+softmax) on the current stream.  The sequence mirrors what
the reference's SimpleNet would run for this model: Embedding, Concat with the dense features (here
the Embedding op writes its block straight into the FC input buffer at the dense features' column
offset), then Gemm + PRelu per layer and Softmax (blaze/graph/simple_net.cc:35-46).
"""
import ctypes as C

import numpy as np

import blaze_hip as bz


class CtrForward:
    def __init__(self, cfg, tables, mlp, sparse_batches, dense_batches, dtype="f16", fused_scan=True, fused_head=True):
        """fused_head: the last (skinny) layer rides in the launch of the layer before it, as SimpleNet runs the model."""
        import torch
        self.cfg = cfg
        self.fused_scan = fused_scan
        self.fused_head = fused_head and len(mlp) >= 2
        self._launches = None
        self.lib = bz.lib()
        tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]
        bdt = {"f16": bz.F16, "bf16": bz.BF16, "f32": bz.F32}[dtype]
        self.tables = [bz.DeviceTable(t) for t in tables]
        self.weights = []
        for (w, b, slope) in mlp:
            self.weights.append((bz.pack_weight(w, False, bdt), b.float().contiguous(), slope.float().contiguous(),
                                 w.shape[0]))
        self.n_batches = len(sparse_batches)
        self.steps = []
        self.nnz = []
        B = cfg.batch
        for sp, dn in zip(sparse_batches, dense_batches):
            x = torch.zeros((B, cfg.in_dim), dtype=tdt, device="cuda")
            x[:, :cfg.dense] = torch.from_numpy(dn).cuda().to(tdt)  # the dense "Feed"
            items = []
            nnz = 0
            keep = []
            for s, (ids, vals, seg) in enumerate(sp):
                d_ids, d_vals, d_seg = (torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(),
                                        torch.from_numpy(seg).cuda())
                keep.append((d_ids, d_vals, d_seg))
                nnz += ids.size
                items.append(dict(table=self.tables[s], ids=d_ids, values=d_vals, segments=d_seg, out=x,
                                  col=cfg.dense + s * cfg.dim, udf=bz.SUM))
            plan = bz.EmbeddingPlan(items, fused_scan=fused_scan)
            acts = [x]
            descs = []
            nl = len(self.weights)
            for li, (wp, b, slope, k) in enumerate(self.weights):
                last = li == nl - 1
                y = torch.empty((B, wp.shape[0]), dtype=torch.float32 if last else tdt, device="cuda")
                d = bz.FcDesc()
                a = acts[-1]
                d.a, d.w, d.y, d.bias = a.data_ptr(), wp.data_ptr(), y.data_ptr(), b.data_ptr()
                d.lda, d.ldw, d.ldy = a.stride(0), wp.stride(0), y.stride(0)
                d.m, d.n, d.k = B, wp.shape[0], k
                d.in_dtype, d.out_dtype = bdt, bz.bz_dtype(y.dtype)
                d.bias_rows = 1
                d.alpha = d.beta = 1.0
                if last:
                    d.act = bz.ACT_SOFTMAX
                else:
                    d.act, d.act_p0, d.act_size = bz.ACT_PRELU, slope.data_ptr(), slope.numel()
                descs.append(d)
                acts.append(y)
            head_desc = None
            if self.fused_head:  # layer n-2 with layer n-1 as its head; the tensor between them is not stored
                head_desc = bz.FcDesc.from_buffer_copy(descs[-2])
                last = descs[-1]
                head_desc.y = None
                head_desc.head_w, head_desc.head_bias, head_desc.head_y = last.w, last.bias, last.y
                head_desc.head_ldw, head_desc.head_ldy, head_desc.head_n = last.ldw, last.ldy, last.n
                head_desc.head_act, head_desc.head_out_dtype = last.act, last.out_dtype
            self.steps.append(dict(plan=plan, descs=descs, acts=acts, keep=keep, x=x, head_desc=head_desc))
            self.nnz.append(nnz)

    # --- launches (current stream) ---------------------------------------------------------------
    def _stream(self):
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def scan(self, i, st=None):
        p = self.steps[i % self.n_batches]["plan"]
        bz.check(self.lib.bz_segments_to_offsets_slots(p.slots_dev.data_ptr(), p.n, st or self._stream()))

    def pool(self, i, st=None):
        p = self.steps[i % self.n_batches]["plan"]
        if p.args_eligible():  # as the Embedding operator launches it: the slot records travel as kernel arguments
            bz.check(self.lib.bz_embed_pool_args(p.host, C.byref(p.launch), st or self._stream()))
        else:
            bz.check(self.lib.bz_embed_pool(p.slots_dev.data_ptr(), C.byref(p.launch), st or self._stream()))

    def fc(self, i, layer, st=None):
        d = self.steps[i % self.n_batches]["descs"][layer]
        bz.check(self.lib.bz_fc_fused(C.byref(d), st or self._stream()))

    def fc_with_head(self, i, st=None):
        """the last two layers in one launch"""
        d = self.steps[i % self.n_batches]["head_desc"]
        bz.check(self.lib.bz_fc_fused(C.byref(d), st or self._stream()))

    def launches(self):
        """[(name, callable(i, stream))] of one step's launches after the pooling kernel"""
        if getattr(self, "_launches", None) is None:
            self._launches = self._make_launches()
        return self._launches

    def _make_launches(self):
        n = len(self.weights)
        if self.fused_head:
            return [("bz_fc[%d]" % li, (lambda i, st=None, li=li: self.fc(i, li, st))) for li in range(n - 2)] + \
                   [("bz_fc[%d+%d]" % (n - 2, n - 1), self.fc_with_head)]
        return [("bz_fc[%d]" % li, (lambda i, st=None, li=li: self.fc(i, li, st))) for li in range(n)]

    def step(self, i, st=None):
        st = st or self._stream()
        if not self.fused_scan:
            self.scan(i, st)
        self.pool(i, st)
        for _, launch in self._launches or self.launches():
            launch(i, st)

    def output(self, i):
        return self.steps[i % self.n_batches]["acts"][-1]

    def pooled(self, i):
        return self.steps[i % self.n_batches]["x"]

    # --- accounting ------------------------------------------------------------------------------
    def embedding_bytes(self, i):
        from synth import embedding_bytes
        cfg = self.cfg
        return embedding_bytes(self.nnz[i % self.n_batches], cfg.batch, cfg.slots, cfg.dim * 2, 0, cfg.slots * cfg.dim, 2)

    def fc_flops(self):
        L = self.cfg.layers
        return [2.0 * self.cfg.batch * L[i] * L[i + 1] for i in range(len(L) - 1)]

"""The entry point that allocates nothing (bz_embed_pool_static_scratch) against the two-call form it is a variant of
(bz_segments_to_offsets_slots into caller-owned offsets, then bz_embed_pool): same bits, on two calls in a row, the
second with a smaller input; and its size limit."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def bz():
    import torch
    import blaze_hip
    assert torch.cuda.is_available(), "no GPU visible"
    blaze_hip.device_check()
    return blaze_hip


def _items(bz, torch, rng, tables, batch, max_len, out, mixed):
    items, keep = [], []
    col = 0
    for s, t in enumerate(tables):
        seg = rng.integers(0, max_len + 1, batch).astype(np.int32)
        nnz = int(seg.sum())
        ids = rng.integers(-3, t.rows + 3, nnz).astype(np.int64)  # a few ids outside the table
        vals = rng.uniform(0.5, 1.5, nnz).astype(np.float32)
        d = [torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(seg).cuda()]
        keep.append(d)
        udf = (bz.SUM, bz.AVG, bz.ASSIGN)[s % 3] if mixed else (bz.SUM, bz.AVG)[s % 2]
        trunc = 3 if udf == bz.ASSIGN else 0
        items.append(dict(table=t, ids=d[0], values=d[1], segments=d[2], out=out, col=col, udf=udf, trunc_num=trunc,
                          trunc_dir=bz.ORDER if s % 2 else bz.REVERSE))
        col += t.dim * max(trunc, 1)
    return items, keep


@pytest.mark.parametrize("mixed", [False, True])
def test_static_scratch_entry_point_matches_the_two_call_form(bz, mixed):
    import torch
    import pyblaze_hip
    rng = np.random.default_rng(17 + int(mixed))
    tables = [bz.DeviceTable(torch.from_numpy((rng.standard_normal((3000, 32)) * 0.1).astype(np.float16)).cuda()) for _ in range(6)]
    width = sum(t.dim * (3 if (mixed and s % 3 == 2) else 1) for s, t in enumerate(tables))
    # two calls in a row through the same buffer: a large request, then a smaller one (fewer samples, shorter segments)
    for call, (batch, max_len) in enumerate(((700, 12), (130, 5))):
        want = torch.full((batch, width), float("nan"), dtype=torch.float32, device="cuda")
        got = torch.full((batch, width), float("nan"), dtype=torch.float32, device="cuda")
        state = rng.bit_generator.state
        items_w, keep_w = _items(bz, torch, rng, tables, batch, max_len, want, mixed)
        rng.bit_generator.state = state
        items_g, keep_g = _items(bz, torch, rng, tables, batch, max_len, got, mixed)
        ref = bz.EmbeddingPlan(items_w, fused_scan=False)   # offsets in caller-owned tensors
        ref.run()
        plan = bz.EmbeddingPlan(items_g, fused_scan=True)   # no offsets anywhere in the records
        assert all(s.offsets is None for s in plan.host) and plan.launch.max_batch == batch
        assert (plan.launch.variant == 0) == mixed
        print("static scratch call %d: mixed=%s batch=%d variant=%#x" % (call, mixed, batch, plan.launch.variant), flush=True)
        torch.cuda.synchronize()
        before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), pyblaze_hip.allocation_count())
        plan.run_static_scratch()
        torch.cuda.synchronize()
        after = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), pyblaze_hip.allocation_count())
        # no allocation by the library or through torch, and from the second call on (the first one on a device loads
        # the kernels' code and looks the buffer's address up) none by the driver either: the device's free memory stands
        assert after[1:] == before[1:]
        if call > 0:
            assert after[0] == before[0], "free device memory changed across a call that must not allocate"
        a, b = got.cpu().numpy(), want.cpu().numpy()
        assert not np.isnan(b).any()
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_static_scratch_entry_point_rejects_what_does_not_fit(bz):
    launch = bz.EmbedLaunch()
    launch.n_slots, launch.total_wg, launch.max_batch = 300, 300, 8192  # 300 x 8193 x 8 bytes > 16 MiB
    rc = bz.lib().bz_embed_pool_static_scratch(C.c_void_p(0x1000), C.byref(launch), None)
    assert rc == -22 and b"exceed" in bz.lib().bz_last_error()

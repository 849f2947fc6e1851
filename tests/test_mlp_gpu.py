"""GPU parity of bz_mlp_fused (a whole FC stack in one launch) against the CPU oracle run layer by layer.

Tolerance: 2e-3 (fp16 / bf16 tensors, fp32 accumulation) against the fp32 oracle fed the same rounded inputs,
weights and hidden activations; and against the per-layer kernel bz_fc_fused at the same bar.
"""
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


def _round(x, dt):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(dt).float().numpy()


def _stack(rng, widths, acts):
    layers = []
    for li in range(len(widths) - 1):
        k, n = widths[li], widths[li + 1]
        l = dict(w=(rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32), bias=(rng.standard_normal(n) * 0.1).astype(np.float32),
                 act=acts[li])
        if acts[li] == "prelu":
            l["params"] = ((rng.random(n) * 0.5).astype(np.float32), )
        elif acts[li] == "dice":
            l["params"] = ((rng.standard_normal(n) * 0.1).astype(np.float32), (rng.standard_normal(n) * 0.1).astype(np.float32),
                           rng.uniform(0.5, 1.5, n).astype(np.float32))
        layers.append(l)
    return layers


ACT = {"none": 0, "prelu": 1, "dice": 2, "relu": 3, "sigmoid": 4, "softmax": 5}
CASES = [
    (2048, (896, 512, 256, 2), ("prelu", "prelu", "softmax")),     # config 2
    (1000, (896, 512, 256, 2), ("prelu", "prelu", "softmax")),     # ragged last row block
    (64, (128, 128), ("none", )),                                  # one wide layer, output through LDS
    (200, (72, 384, 128, 1), ("dice", "relu", "sigmoid")),         # input width not a multiple of 64; 3 column blocks
    (130, (264, 256, 512, 128, 8), ("relu", "dice", "prelu", "none")),  # four layers, widest hidden, head of 8
    (1, (64, 128, 2), ("sigmoid", "softmax")),
    (77, (1024, 512, 256), ("prelu", "dice")),                     # last layer wide
    # from 64 workgroups of 64 rows on, the kernel takes 64 rows per workgroup (the cases above take 32)
    (4133, (896, 512, 256, 2), ("prelu", "prelu", "softmax")),
    (4096, (136, 256, 128), ("dice", "relu")),
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("m,widths,acts", CASES)
def test_fused_mlp_against_oracle(bz, oracle, dtype, m, widths, acts):
    import torch
    rng = np.random.default_rng(m + len(widths))
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    bdt = bz.F16 if dtype == "f16" else bz.BF16
    layers = _stack(rng, widths, acts)
    x = rng.standard_normal((m, widths[0])).astype(np.float32)
    print("case", dtype, m, widths, acts, flush=True)
    dev_layers = []
    for l in layers:
        dl = dict(w=torch.from_numpy(l["w"]).cuda(), bias=torch.from_numpy(l["bias"]).cuda(), act=ACT[l["act"]],
                  params=tuple(torch.from_numpy(p).cuda() for p in l.get("params", ())), act_alpha=0.0)
        dev_layers.append(dl)
    mlp = bz.FusedMlp(dev_layers, bdt)
    xd = torch.from_numpy(x).cuda().to(tdt)
    head = widths[-1] <= 8
    out = mlp(xd, out_dtype=bz.F32 if head else bdt)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    # oracle, layer by layer, rounding where the tensors are stored
    h = _round(x, tdt)
    per_layer = xd
    for li, l in enumerate(layers):
        last = li == len(layers) - 1
        w_r = _round(l["w"], tdt)
        params = l.get("params")
        h = oracle.fc(h, w_r, l["bias"], act=None if l["act"] == "none" else l["act"], act_params=params)
        if not (last and head):
            h = _round(h, tdt)
        # the same stack through the per-layer kernel
        wp = bz.pack_weight(dev_layers[li]["w"], False, bdt)
        per_layer = bz.fc_fused(per_layer, wp, widths[li], bias=dev_layers[li]["bias"], act=ACT[l["act"]],
                                act_params=dev_layers[li]["params"], act_alpha=0.0,
                                out_dtype=bz.F32 if (last and head) else bdt)
    torch.cuda.synchronize()
    assert got.shape == h.shape
    scale = max(1e-3, float(np.abs(h).max()))
    np.testing.assert_allclose(got, h, rtol=2e-3 if dtype == "f16" else 1e-2, atol=(2e-3 if dtype == "f16" else 1e-2) * scale)
    np.testing.assert_allclose(got, per_layer.float().cpu().numpy(), rtol=2e-3 if dtype == "f16" else 1e-2,
                               atol=(2e-3 if dtype == "f16" else 1e-2) * scale)


def test_fused_mlp_refuses_shapes_it_cannot_run(bz):
    import ctypes as C
    import torch
    w = torch.zeros((64, 100), device="cuda")
    with pytest.raises(AssertionError):
        bz.FusedMlp([dict(w=w, bias=None, act=0)], bz.F16)  # 100 is not a multiple of 128
    d = bz.MlpDesc()
    assert bz.lib().bz_mlp_fused(C.byref(d), None) != 0
    d.dtype, d.n_layers = bz.F32, 1
    assert bz.lib().bz_mlp_fused(C.byref(d), None) != 0 and b"fp16 and bf16 only" in bz.lib().bz_last_error()
    assert bz.lib().bz_mlp_packed_elems(896, 512) == 1024 * 512 and bz.lib().bz_mlp_packed_elems(72, 384) == 256 * 384
    assert bz.lib().bz_mlp_packed_elems(64, 100) == 0

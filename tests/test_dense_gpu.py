"""GPU parity of the dense path (bz_fc_fused, bz_fc_pack_weight, bz_gemm_strided_batched, bz_activation).

The oracle is the reference's composition Activation(Gemm(x, W, b)) in fp32 (oracle/blaze_oracle.c) plus an
fp64 product used to scale tolerances: MKL's / MFMA's summation orders differ, so the error bound is taken
relative to sum_k |a||b| (the condition of the dot product), not to the possibly cancelled result.
  fp32 path:       |got - want| <= 1e-5 * (sum|a||b| + |bias|)        (contract: rel 1e-5)
  fp16/bf16 path:  |got - want| <= 2e-3 * (sum|a||b| + |bias|) (+ out rounding)   (contract: 2e-3)
where want is computed from the same fp16/bf16-rounded inputs the kernel reads.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ACT = {"none": 0, "prelu": 1, "dice": 2, "relu": 3, "sigmoid": 4, "softmax": 5}


@pytest.fixture(scope="module")
def bz():
    import torch
    import blaze_hip
    assert torch.cuda.is_available(), "no GPU visible"
    blaze_hip.device_check()
    return blaze_hip


def _dev(x, dtype=None):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t if dtype is None else t.to(dtype)


def _tdtype(name):
    import torch
    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[name]


def _round_to(x, name):
    """numpy fp32 array rounded to the kernel's input precision (returned as fp32)."""
    import torch
    if name == "f32":
        return x.astype(np.float32)
    return torch.from_numpy(x.astype(np.float32)).to(_tdtype(name)).to(torch.float32).numpy()


def _fc_case(bz, oracle, M, N, K, in_name, out_name, act, seed, trans_b=False, lda_pad=0, full_bias=False, alpha=1.0,
             beta=1.0, bias=True):
    import torch
    rng = np.random.default_rng(seed)
    A = _round_to(rng.standard_normal((M, K)), in_name)
    Wkn = _round_to(rng.standard_normal((K, N)) / np.sqrt(K), in_name)
    b = None
    if bias:
        b = (rng.standard_normal((M, N) if full_bias else N) * 0.1).astype(np.float32)
    params_np, act_kwargs = (), {}
    if act == "prelu":
        params_np = (rng.uniform(0.1, 0.4, N).astype(np.float32),)
    elif act == "dice":
        params_np = ((rng.standard_normal(N) * 0.1).astype(np.float32), (rng.standard_normal(N) * 0.1).astype(np.float32),
                     rng.uniform(0.5, 1.5, N).astype(np.float32))
    # device inputs
    a_dev = torch.zeros((M, K + lda_pad), dtype=_tdtype(in_name), device="cuda")
    a_dev[:, :K] = _dev(A, _tdtype(in_name))
    a_view = a_dev[:, :K]
    w_src = _dev(Wkn.T.copy() if trans_b else Wkn, _tdtype(in_name) if in_name != "f32" else None)
    wp = bz.pack_weight(w_src, trans_b, {"f32": bz.F32, "f16": bz.F16, "bf16": bz.BF16}[in_name])
    out = bz.fc_fused(a_view, wp, K, bias=None if b is None else _dev(b), act=ACT[act],
                      act_params=tuple(_dev(p) for p in params_np),
                      out_dtype={"f32": bz.F32, "f16": bz.F16, "bf16": bz.BF16}[out_name], alpha=alpha, beta=beta,
                      act_alpha=0.0)
    torch.cuda.synchronize()
    got = out.to(torch.float32).cpu().numpy()
    # oracle: pre-activation in fp64 (tolerance scale) and the reference composition in fp32
    pre64 = alpha * (A.astype(np.float64) @ Wkn.astype(np.float64))
    scale = abs(alpha) * (np.abs(A).astype(np.float64) @ np.abs(Wkn).astype(np.float64))
    if b is not None:
        pre64 = pre64 + beta * b
        scale = scale + np.abs(beta * b)
    pre32 = pre64.astype(np.float32)
    if act == "none":
        want = pre32
    elif act == "prelu":
        want = oracle.prelu(pre32, params_np[0])
    elif act == "dice":
        want = oracle.dice(pre32, *params_np)
    elif act == "relu":
        want = oracle.leaky_relu(pre32, 0.0)
    elif act == "sigmoid":
        want = oracle.sigmoid(pre32)
    else:
        want = oracle.softmax(pre32, 1)
    tol = 1e-5 if in_name == "f32" else 2e-3
    out_eps = {"f32": 0.0, "f16": 2.0**-11, "bf16": 2.0**-8}[out_name]
    # activations on this path are 1-Lipschitz up to the Dice gate (|d/dx| <= 1 + |gamma-1|*0.25*|x|/den): bound by 2
    bound = 2.0 * tol * scale + out_eps * np.abs(want) + 1e-7
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    worst = np.unravel_index(np.argmax(err - bound), err.shape)
    assert np.all(err <= bound), "M=%d N=%d K=%d %s->%s act=%s: err %.3e > bound %.3e at %s (got %r want %r)" % (
        M, N, K, in_name, out_name, act, err[worst], bound[worst], worst, got[worst], want[worst])
    return got, want


def test_reference_gemm_kat_on_gpu(bz, kats):
    import torch
    from test_oracle_pins import _tensor
    c = kats["gemm_net_v1_cpu"]
    A, B, bias = (_tensor(c["tensors"][n]) for n in ("A_output", "B_output", "Bias_output"))
    wp = bz.pack_weight(_dev(B), False, bz.F32)
    out = bz.fc_fused(_dev(A), wp, 3, bias=_dev(bias))
    torch.cuda.synchronize()
    np.testing.assert_allclose(out.cpu().numpy(), np.array(c["expected"]["output"]["values"], np.float32).reshape(2, 2),
                               rtol=0, atol=1e-6)


def test_pack_weight_layout_and_rounding(bz):
    import torch
    rng = np.random.default_rng(0)
    W = rng.standard_normal((37, 21)).astype(np.float32)  # [K, N]
    for trans_b in (False, True):
        src = _dev(W.T.copy() if trans_b else W)
        for dt, tdt in ((bz.F32, torch.float32), (bz.F16, torch.float16), (bz.BF16, torch.bfloat16)):
            p = bz.pack_weight(src, trans_b, dt)
            torch.cuda.synchronize()
            assert p.shape == (21, 40)
            want = torch.from_numpy(W.T.copy()).to(tdt)
            assert torch.equal(p[:, :37].cpu(), want)
            assert not p[:, 37:].cpu().to(torch.float32).numpy().any()


@pytest.mark.parametrize("M,N,K", [(128, 200, 192), (128, 80, 200), (1, 80, 200), (33, 70, 20), (257, 129, 162),
                                   (4100, 1000, 72), (4096, 2048, 64)])
@pytest.mark.parametrize("act", ["none", "prelu", "dice", "relu", "sigmoid"])
def test_fc_fp32(bz, oracle, M, N, K, act):
    print("case fp32 M=%d N=%d K=%d act=%s" % (M, N, K, act), flush=True)
    _fc_case(bz, oracle, M, N, K, "f32", "f32", act, seed=M * 7 + N + K)


@pytest.mark.parametrize("in_name,out_name", [("f16", "f16"), ("f16", "f32"), ("bf16", "bf16"), ("bf16", "f32")])
@pytest.mark.parametrize("M,N,K,act", [(2048, 512, 896, "prelu"), (2048, 256, 512, "prelu"), (300, 80, 216, "dice"),
                                       (300, 40, 80, "dice"), (64, 200, 168, "dice"), (4096, 2048, 256, "relu"),
                                       (4100, 1000, 200, "dice"), (33000, 80, 216, "dice"), (100, 100, 104, "none"),
                                       (4000, 4104, 72, "prelu"),  # 16 x 17 tiles of 256x256, ragged in M and N
                                       # the software-pipelined K loop: 128x256 tiles (128x128 for fp32 output), ragged
                                       # in M and N, K ending inside a tile and the loop padded with absent tiles
                                       (8200, 1000, 520, "prelu"), (33000, 250, 136, "dice")])
def test_fc_half(bz, oracle, in_name, out_name, M, N, K, act):
    print("case %s->%s M=%d N=%d K=%d act=%s" % (in_name, out_name, M, N, K, act), flush=True)
    _fc_case(bz, oracle, M, N, K, in_name, out_name, act, seed=M + N * 3 + K)


# Large 2-byte layers go to the streaming kernel (256x128 tiles, loader waves, operands straight into LDS) once
# ceil(M/256) * ceil(N/128) >= 200, K is a multiple of 64 and at least 512, and the output takes 16-byte stores.
@pytest.mark.parametrize("in_name", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,act,kw", [
    (7000, 1000, 512, "prelu", {}),                 # ragged in M (88 rows in the last tile) and N (104 columns)
    (8192, 1024, 576, "dice", {}),                  # whole tiles, an odd number of K tiles
    (6500, 1032, 640, "none", {"alpha": 0.5, "beta": 2.0}),
    (6600, 1024, 512, "sigmoid", {"bias": False}),
    (6400, 1024, 1024, "relu", {"full_bias": True}),
    (51300, 128, 512, "prelu", {}),                 # one N tile; 201 M tiles: the XCD bands are uneven
])
def test_fc_streaming_kernel(bz, oracle, in_name, M, N, K, act, kw):
    print("case stream %s M=%d N=%d K=%d act=%s %r" % (in_name, M, N, K, act, kw), flush=True)
    assert -(-M // 256) * -(-N // 128) >= 200 and K % 64 == 0 and K >= 512
    _fc_case(bz, oracle, M, N, K, in_name, in_name, act, seed=M + N + K, **kw)


@pytest.mark.parametrize("in_name", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("M,K,N,N2,act,hact", [
    (2048, 512, 256, 2, "prelu", "softmax"),   # config 2's last two layers: 32x256 tile
    (300, 200, 80, 2, "dice", "softmax"),      # DIN main tower tail: 32x128 tile, ragged M
    (5000, 80, 40, 1, "dice", "none"),         # DIN attention tail: 32x64 tile
    (17000, 80, 40, 1, "dice", "none"),        # the same with enough rows for the 64x64 tile
    (513, 128, 128, 8, "relu", "sigmoid"),     # widest head
    (100, 64, 16, 3, "none", "softmax"),
])
def test_fc_with_skinny_head_in_one_launch(bz, oracle, in_name, M, K, N, N2, act, hact):
    """Layer + skinny head in one launch against the same two layers as two launches.  The one-launch form uses a tile
    that spans the whole row, so its fp32 sums run in another order: the first layer's output agrees to one rounding
    of the tensor type, the head to 1e-5 (fp32) / 2e-3 (the head reads the rounded tile as the second launch reads the
    stored tensor), also when the first layer's output is not stored.  The head against the oracle, computed from
    the first layer's own stored output: 1e-5 (fp32) / 2e-3 relative to the operand magnitudes."""
    import torch
    print("case", in_name, M, K, N, N2, act, hact, flush=True)
    rng = np.random.default_rng(M + 3 * K + N)
    tdt, bt = _tdtype(in_name), {"f32": bz.F32, "f16": bz.F16, "bf16": bz.BF16}[in_name]
    A = _round_to(rng.standard_normal((M, K)), in_name)
    W1 = _round_to(rng.standard_normal((K, N)) / np.sqrt(K), in_name)
    W2 = _round_to(rng.standard_normal((N, N2)) / np.sqrt(N), in_name)
    b1 = (rng.standard_normal(N) * 0.1).astype(np.float32)
    b2 = (rng.standard_normal(N2) * 0.1).astype(np.float32)
    params = ()
    if act == "prelu":
        params = (rng.uniform(0.1, 0.4, N).astype(np.float32), )
    elif act == "dice":
        params = ((rng.standard_normal(N) * 0.1).astype(np.float32), (rng.standard_normal(N) * 0.1).astype(np.float32),
                  rng.uniform(0.5, 1.5, N).astype(np.float32))
    a = _dev(A, tdt)
    w1 = bz.pack_weight(_dev(W1, None if in_name == "f32" else tdt), False, bt)
    w2 = bz.pack_weight(_dev(W2, None if in_name == "f32" else tdt), False, bt)
    kw = dict(bias=_dev(b1), act=ACT[act], act_params=tuple(_dev(p) for p in params), out_dtype=bt)
    y_ref = bz.fc_fused(a, w1, K, **kw)
    z_ref = bz.fc_fused(y_ref, w2, N, bias=_dev(b2), act=ACT[hact], out_dtype=bz.F32)
    z1 = torch.full((M, N2), -7.0, dtype=torch.float32, device="cuda")
    y1, _ = bz.fc_fused(a, w1, K, head=dict(w=w2, bias=_dev(b2), act=ACT[hact], out=z1), **kw)
    z2 = torch.full((M, N2), -7.0, dtype=tdt, device="cuda")
    none, _ = bz.fc_fused(a, w1, K, head=dict(w=w2, bias=_dev(b2), act=ACT[hact], out=z2), store_out=False, **kw)
    torch.cuda.synchronize()
    assert none is None
    ulp = {"f32": 1e-5, "f16": 2.0**-10, "bf16": 2.0**-7}[in_name]
    np.testing.assert_allclose(y1.float().cpu().numpy(), y_ref.float().cpu().numpy(), rtol=ulp, atol=ulp)  # sums of O(1) magnitude: absolute part for cancelled values
    tol = 1e-5 if in_name == "f32" else 2e-3
    np.testing.assert_allclose(z1.cpu().numpy(), z_ref.cpu().numpy(), rtol=tol, atol=tol)
    np.testing.assert_allclose(z2.float().cpu().numpy(), z1.cpu().numpy(), rtol=ulp, atol=1e-6)  # same head, rounded to the type
    # oracle: second layer in fp64 from the first layer's stored (rounded) output
    y = y1.float().cpu().numpy().astype(np.float64)
    pre = (y @ W2.astype(np.float64) + b2).astype(np.float32)
    want = {"none": pre, "sigmoid": oracle.sigmoid(pre), "softmax": oracle.softmax(pre, 1)}[hact]
    scale = np.abs(y) @ np.abs(W2).astype(np.float64) + np.abs(b2)
    assert np.all(np.abs(z1.cpu().numpy() - want) <= 1e-5 * scale + 1e-6)  # fp32 head from the stored tile: fp32 accuracy


def test_fc_head_limits_are_refused(bz):
    import torch
    a = torch.zeros((64, 512), dtype=torch.float16, device="cuda")
    w = torch.zeros((512, 512), dtype=torch.float16, device="cuda")
    h = torch.zeros((2, 512), dtype=torch.float16, device="cuda")
    z = torch.zeros((64, 2), dtype=torch.float32, device="cuda")
    with pytest.raises(bz.BlazeHipError, match="n <= 256"):
        bz.fc_fused(a, w, 512, head=dict(w=h, out=z))
    w = torch.zeros((128, 512), dtype=torch.float16, device="cuda")
    h = torch.zeros((9, 128), dtype=torch.float16, device="cuda")
    with pytest.raises(bz.BlazeHipError, match="head of 9 outputs"):
        bz.fc_fused(a, w, 512, head=dict(w=h, out=torch.zeros((64, 9), dtype=torch.float32, device="cuda")))


@pytest.mark.parametrize("in_name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("M,N,K,act", [(2048, 2, 256, "softmax"), (128, 2, 80, "softmax"), (5000, 1, 40, "none"),
                                       (8192, 1, 256, "sigmoid"), (7, 8, 1000, "prelu"), (3, 3, 12, "dice")])
def test_fc_skinny(bz, oracle, in_name, M, N, K, act):
    print("case skinny %s M=%d N=%d K=%d act=%s" % (in_name, M, N, K, act), flush=True)
    _fc_case(bz, oracle, M, N, K, in_name, "f32", act, seed=M + N + K)


def test_fc_variants(bz, oracle):
    """transB weights, padded lda, unaligned K with element-wise loads, full [M,N] bias, alpha/beta, no bias."""
    _fc_case(bz, oracle, 70, 90, 64, "f16", "f16", "prelu", seed=1, trans_b=True)
    _fc_case(bz, oracle, 70, 90, 162, "f16", "f32", "dice", seed=2, lda_pad=6)     # lda=168: vector loads + K tail
    _fc_case(bz, oracle, 70, 90, 162, "f16", "f32", "dice", seed=3, lda_pad=0)     # lda=162: element-wise loads
    _fc_case(bz, oracle, 70, 90, 50, "f32", "f32", "none", seed=4, lda_pad=1)      # fp32 unaligned
    _fc_case(bz, oracle, 40, 48, 32, "f32", "f32", "none", seed=5, full_bias=True, alpha=0.5, beta=-2.0)
    _fc_case(bz, oracle, 40, 48, 32, "f16", "f32", "relu", seed=6, bias=False)
    _fc_case(bz, oracle, 40, 5, 32, "f16", "f32", "none", seed=7, full_bias=True, alpha=0.5, beta=-2.0)


def test_fc_argument_errors(bz):
    import torch
    a = torch.zeros((4, 8), dtype=torch.float16, device="cuda")
    w = torch.zeros((16, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(bz.BlazeHipError, match="softmax"):
        bz.fc_fused(a, w, 8, act=ACT["softmax"])
    with pytest.raises(bz.BlazeHipError, match="PRelu"):
        bz.fc_fused(a, w, 8, act=ACT["prelu"], act_params=(torch.zeros(3, device="cuda"),))
    with pytest.raises(bz.BlazeHipError, match="unknown activation"):
        bz.fc_fused(a, w, 8, act=99)


# ------------------------------------------------------------------------------ strided batched / matmul family
def _bgemm(bz, A, B, M, N, K, batch, sa, sb, ta, tb, dtype, C0=None, alpha=1.0, beta=0.0):
    import torch
    a, b = _dev(A, dtype), _dev(B, dtype)
    c = torch.zeros((batch, M, N), dtype=dtype, device="cuda") if C0 is None else _dev(C0, dtype)
    bz.gemm_strided_batched(a, b, c, M, N, K, batch, sa, sb, M * N, ta, tb, alpha, beta)
    torch.cuda.synchronize()
    return c.to(torch.float32).cpu().numpy()


@pytest.mark.parametrize("name", ["matmul_net_v1_cpu", "fused_parallel_matmul_net_v1_cpu", "fused_parallel_matmul_net_v2_cpu",
                                  "fused_parallel_matmul_net_v3_cpu"])
def test_reference_matmul_kats_on_gpu(bz, kats, name):
    import torch
    from test_oracle_pins import _tensor
    c = kats[name]
    op = c["ops"][0]
    A, B = (_tensor(c["tensors"][n]) for n in op["inputs"])
    ta, tb = bool(op["args"].get("transA", 0)), bool(op["args"].get("transB", 0))
    P = op["args"].get("parallel_num", 1)
    M, K = A.shape[-2:]
    if ta:
        M, K = K, M
    N = B.shape[-2] if tb else B.shape[-1]
    exp = c["expected"]["output"]
    want = np.array(exp["values"], np.float32).reshape(exp["shape"])
    ab, bb = A.shape[0] // P, B.shape[0] // P
    cb = max(ab, bb)
    got = np.zeros((P * cb, M, N), np.float32)
    for p in range(P):  # BatchedBroadcastGemm: one strided-batched call per parallel slice (broadcast.h:340-378)
        Ap, Bp = A[p * ab:(p + 1) * ab], B[p * bb:(p + 1) * bb]
        got[p * cb:(p + 1) * cb] = _bgemm(bz, Ap, Bp, M, N, K, cb, 0 if ab == 1 else M * K, 0 if bb == 1 else K * N, ta, tb,
                                          torch.float32)
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=0, atol=1e-6)


@pytest.mark.parametrize("name", ["fused_parallel_gemm_net_v%d_cpu" % i for i in range(1, 6)])
def test_reference_fused_parallel_gemm_kats_on_gpu(bz, kats, name):
    """FusedParallelGemm = P FCs sharing the input: strided batched with stride_a = 0 (fused_parallel_gemm_op.h:115-129)
    after the batched bias broadcast-assign."""
    import torch
    from test_oracle_pins import _tensor
    c = kats[name]
    op = c["ops"][0]
    ins = [_tensor(c["tensors"][n]) for n in op["inputs"]]
    A, B = ins[0], ins[1]
    ta, tb = bool(op["args"].get("transA", 0)), bool(op["args"].get("transB", 0))
    P = op["args"]["parallel_num"]
    M, K = (A.shape[1], A.shape[0]) if ta else A.shape
    N = B.shape[0] // P if tb else B.shape[1]
    C0 = np.zeros((P, M, N), np.float32)
    beta = 0.0
    if len(ins) > 2:
        C0[:] = ins[2].reshape(P, 1, N)
        beta = 1.0
    got = _bgemm(bz, A, B, M, N, K, P, 0, K * N, ta, tb, torch.float32, C0=C0, alpha=1.0, beta=beta)
    exp = c["expected"]["output"]
    np.testing.assert_allclose(got.reshape(exp["shape"]), np.array(exp["values"], np.float32).reshape(exp["shape"]), rtol=0,
                               atol=1e-6)


@pytest.mark.parametrize("dtype_name", ["f32", "f16"])
def test_attention_weighted_sum(bz, oracle, dtype_name):
    """DIN batchdot: scores [B,T,1] (transA) x history [B,T,D] -> [B,1,D]; config 3 shape B=1024, T=50, D=54."""
    import torch
    rng = np.random.default_rng(3)
    Bn, T, D = 1024, 50, 54
    w = _round_to(rng.standard_normal((Bn, T, 1)), dtype_name)
    H = _round_to(rng.standard_normal((Bn, T, D)) * 0.1, dtype_name)
    got = _bgemm(bz, w, H, 1, D, T, Bn, T, T * D, True, False, _tdtype(dtype_name))
    want = oracle.matmul_op(w, H, transa=True, transb=False)
    scale = np.einsum("btk,btd->bkd", np.abs(w), np.abs(H))
    tol = 1e-5 if dtype_name == "f32" else 2e-3
    assert np.all(np.abs(got - want) <= tol * scale + 1e-7)


# ------------------------------------------------------------------------------ standalone activations
@pytest.mark.parametrize("name,act", [("prelu_net_v1_cpu", 1), ("dice_net_v1_cpu", 2), ("leaky_relu_net_v1_cpu", 3),
                                      ("sigmoid_net_v1_cpu", 4), ("softmax_net_v1_cpu", 5)])
def test_reference_activation_kats_on_gpu(bz, kats, name, act):
    import torch
    from test_oracle_pins import _tensor
    c = kats[name]
    op = c["ops"][0]
    ins = [_tensor(c["tensors"][n]) for n in op["inputs"]]
    out = bz.activation(_dev(ins[0]), act, params=tuple(_dev(p) for p in ins[1:]), act_alpha=op["args"].get("alpha", 0.0))
    torch.cuda.synchronize()
    exp = c["expected"]["output"]
    np.testing.assert_allclose(out.cpu().numpy(), np.array(exp["values"], np.float32).reshape(exp["shape"]), rtol=0,
                               atol=1e-6)


def test_activation_random_vs_oracle(bz, oracle):
    import torch
    rng = np.random.default_rng(11)
    X = (rng.standard_normal((513, 77)) * 3).astype(np.float32)
    g, mu, var = ((rng.standard_normal(77) * 0.1).astype(np.float32), (rng.standard_normal(77) * 0.1).astype(np.float32),
                  rng.uniform(0.5, 1.5, 77).astype(np.float32))
    slope = rng.uniform(0, 1, 77).astype(np.float32)
    xd = _dev(X)
    cases = [(1, (slope,), oracle.prelu(X, slope), {}), (2, (g, mu, var), oracle.dice(X, g, mu, var), {}),
             (2, (g, mu, var), oracle.dice(X, g, mu, var, True), {"dice_nosqrt": True}),
             (3, (), oracle.leaky_relu(X, 0.1), {"act_alpha": 0.1}), (4, (), oracle.sigmoid(X), {}),
             (5, (), oracle.softmax(X, 1), {})]
    for act, params, want, kw in cases:
        got = bz.activation(xd, act, params=tuple(_dev(p) for p in params), **kw)
        torch.cuda.synchronize()
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("in_name,P,M,K,N,act,full_bias", [
    ("f32", 3, 3, 2, 3, "none", False),        # the shape of the reference's fused_parallel_gemm fixtures
    ("f32", 4, 257, 72, 40, "prelu", False),   # ragged M, slices narrower than a tile
    ("f16", 3, 2048, 128, 96, "prelu", False), # tiles straddle slice boundaries (96 per slice, 64- or 128-wide tiles)
    ("f16", 5, 300, 216, 80, "dice", False),
    ("bf16", 2, 1000, 64, 256, "relu", False),
    ("f16", 2, 129, 40, 18, "none", False),    # slice width not a whole number of 16-byte chunks: element-wise stores
    ("f32", 3, 65, 30, 24, "none", True),      # a full [P*M, N] bias (fused_parallel_gemm_op.h:78-94)
    ("bf16", 8, 6400, 512, 136, "prelu", False),  # the streaming kernel (25 x 9 tiles); slices straddle its 128-wide tiles
    ("f16", 4, 13000, 512, 128, "none", True),    # the streaming kernel with a full bias
])
def test_fc_split_outputs_equal_separate_layers(bz, oracle, in_name, P, M, K, N, act, full_bias):
    """P sibling layers on one input as ONE launch (bz_fc_desc.n_split): weights [P*N, K] stacked, bias and activation
    parameters [P*N], slice p written as its own [M, N] matrix.  Against the oracle's FusedParallelGemm
    (fused_parallel_gemm_op.h:43-133) followed by the activation, and bit-equal to P separate launches."""
    import ctypes as C
    import torch
    rng = np.random.default_rng(P * 1000 + M + K + N)
    tdt = _tdtype(in_name)
    a = _round_to(rng.standard_normal((M, K)).astype(np.float32), in_name)
    w = _round_to((rng.standard_normal((P, N, K)) / np.sqrt(K)).astype(np.float32), in_name)   # slice p: [N, K] (transB form)
    bias = (rng.standard_normal((P, M, N) if full_bias else (P, N)) * 0.1).astype(np.float32)
    slope = rng.uniform(0.1, 0.4, (P, N)).astype(np.float32)
    dice = [(rng.standard_normal((P, N)) * 0.1).astype(np.float32), (rng.standard_normal((P, N)) * 0.1).astype(np.float32),
            rng.uniform(0.5, 1.5, (P, N)).astype(np.float32)]
    d_a, d_w = _dev(a).to(tdt), _dev(w.reshape(P * N, K)).to(tdt)
    ldw = (K + 7) // 8 * 8
    d_wp = torch.zeros((P * N, ldw), dtype=tdt, device="cuda")
    d_wp[:, :K] = d_w
    d_bias = _dev(bias.reshape(-1))
    params = {"none": (), "relu": (), "prelu": (_dev(slope.reshape(-1)), ), "dice": tuple(_dev(x.reshape(-1)) for x in dice)}[act]
    code = {"none": bz.ACT_NONE, "relu": bz.ACT_LEAKY_RELU, "prelu": bz.ACT_PRELU, "dice": bz.ACT_DICE}[act]
    y = torch.full((P, M, N), float("nan"), dtype=tdt, device="cuda")

    def desc(a_t, w_t, n, bias_t, ps, y_t):
        d = bz.FcDesc()
        d.a, d.w, d.y, d.bias = a_t.data_ptr(), w_t.data_ptr(), y_t.data_ptr(), bias_t.data_ptr()
        d.lda, d.ldw, d.ldy = K, ldw, N
        d.m, d.n, d.k = M, n, K
        d.in_dtype = d.out_dtype = bz.bz_dtype(tdt)
        d.bias_rows = M if full_bias else 1
        d.alpha = d.beta = 1.0
        d.act, d.act_alpha = code, 0.0
        for name, p_ in zip(("act_p0", "act_p1", "act_p2"), ps):
            setattr(d, name, p_.data_ptr())
        d.act_size = n if act == "prelu" else 0
        return d

    d = desc(d_a, d_wp, P * N, d_bias, params, y)
    d.n_split, d.y_split_stride = N, M * N
    print("split case %s P=%d M=%d K=%d N=%d act=%s full_bias=%s" % (in_name, P, M, K, N, act, full_bias), flush=True)
    bz.check(bz.lib().bz_fc_fused(C.byref(d), None))
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    # oracle: FusedParallelGemm with B stacked [P*N, K] under transB, then the activation per slice
    want = oracle.fused_parallel_gemm_op(a, w.reshape(P * N, K), bias.reshape(P * M, N) if full_bias else bias.reshape(-1), P, False, True)
    want = want.reshape(P, M, N)
    for p in range(P):
        if act == "prelu":
            want[p] = oracle.prelu(want[p], slope[p])
        elif act == "dice":
            want[p] = oracle.dice(want[p], dice[0][p], dice[1][p], dice[2][p])
        elif act == "relu":
            want[p] = oracle.leaky_relu(want[p], 0.0)
    tol = 1e-5 if in_name == "f32" else 2e-3
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol * max(1.0, float(np.abs(want).max())))
    # P separate launches of the same kernel family: the same sums tile by tile is not guaranteed (tile shapes follow N),
    # so equality is asked at the tolerance of one rounding of the tensor type
    y2 = torch.full((P, M, N), float("nan"), dtype=tdt, device="cuda")
    for p in range(P):
        ps = tuple(x[p * N:(p + 1) * N] for x in params)
        b_p = d_bias[p * M * N:(p + 1) * M * N] if full_bias else d_bias[p * N:(p + 1) * N]
        bz.check(bz.lib().bz_fc_fused(C.byref(desc(d_a, d_wp[p * N:(p + 1) * N], N, b_p, ps, y2[p])), None))
    torch.cuda.synchronize()
    np.testing.assert_allclose(got, y2.float().cpu().numpy(), rtol=tol, atol=tol * max(1.0, float(np.abs(want).max())))


def test_fc_split_argument_errors(bz):
    import ctypes as C
    import torch
    a = torch.zeros((8, 16), dtype=torch.float16, device="cuda")
    w = torch.zeros((32, 16), dtype=torch.float16, device="cuda")
    y = torch.zeros((2, 8, 16), dtype=torch.float16, device="cuda")
    d = bz.FcDesc()
    d.a, d.w, d.y = a.data_ptr(), w.data_ptr(), y.data_ptr()
    d.lda, d.ldw, d.ldy, d.m, d.n, d.k = 16, 16, 16, 8, 32, 16
    d.in_dtype = d.out_dtype = bz.F16
    d.alpha = 1.0
    d.n_split, d.y_split_stride = 12, 128   # 12 does not divide 32
    assert bz.lib().bz_fc_fused(C.byref(d), None) == -22 and b"n_split" in bz.lib().bz_last_error()
    d.n_split = 16
    d.act = bz.ACT_SOFTMAX
    assert bz.lib().bz_fc_fused(C.byref(d), None) != 0


@pytest.mark.parametrize("dtype_name", ["f32", "f16"])
@pytest.mark.parametrize("B,T,Cn", [(1024, 50, 54), (7, 1, 3), (33, 17, 130), (2, 200, 64),
                                    # fewer channels than steps (first pass or tail pass): the lanes past the last
                                    # channel still hold the weights the others read
                                    (64, 50, 16), (64, 50, 24), (19, 70, 8), (19, 40, 70), (5, 130, 1)])
def test_weighted_pool_equals_mul_matmul_reducesum(bz, oracle, dtype_name, B, T, Cn):
    """bz_weighted_pool against the three launches it replaces (Mul, strided-batched GEMM with transA, ReduceSum), bit
    for bit, and against the oracle's fp32 sums of the rounded operands."""
    import ctypes as C
    import torch
    print("weighted pool %s B=%d T=%d C=%d" % (dtype_name, B, T, Cn), flush=True)
    tdt = _tdtype(dtype_name)
    rng = np.random.default_rng(B + T + Cn)
    x = _round_to(rng.standard_normal((B, T, Cn)), dtype_name)
    w = _round_to(rng.standard_normal((B, T, 1)), dtype_name)
    lens = rng.integers(0, T + 1, B)
    mask = (np.arange(T)[None, :] < lens[:, None]).astype(np.float32).reshape(B, T, 1)
    dx, dw, dm = _dev(x).to(tdt), _dev(w).to(tdt), _dev(mask).to(tdt)
    att, tot = bz.weighted_pool(dx, dw, dm)
    # the separate launches
    aw = bz.broadcast_op(bz.EW_MUL, dw, dm)
    c = torch.empty((B, 1, Cn), dtype=tdt, device="cuda")
    bz.gemm_strided_batched(aw, dx, c, 1, Cn, T, B, T, T * Cn, Cn, trans_a=True)
    s = bz.reduce_sum(dx, 1, keepdims=False)
    torch.cuda.synchronize()
    assert torch.equal(att, c.reshape(B, Cn)) and torch.equal(tot, s)
    # without a mask, and each output alone
    att2, none = bz.weighted_pool(dx, dw, None, want_sum=False)
    bz.gemm_strided_batched(dw, dx, c, 1, Cn, T, B, T, T * Cn, Cn, trans_a=True)
    none2, tot2 = bz.weighted_pool(dx)
    torch.cuda.synchronize()
    assert none is None and none2 is None and torch.equal(att2, c.reshape(B, Cn)) and torch.equal(tot2, s)
    # both outputs as column ranges of a wider matrix, with a third piece copied alongside from a pitched source: the
    # Concat that follows the attention tail, written by the same launch; nothing else of the matrix is touched
    n_copy = 7
    wide = torch.full((B, 2 * Cn + n_copy + 5), 3.0, dtype=tdt, device="cuda")
    src = (torch.arange(B * (n_copy + 3), device="cuda").reshape(B, n_copy + 3) % 251).to(tdt)
    bz.weighted_pool(dx, dw, dm, att_out=wide[:, n_copy + Cn + 2:n_copy + 2 * Cn + 2], sum_out=wide[:, n_copy:n_copy + Cn],
                     copy=(src[:, 1:1 + n_copy], wide[:, :n_copy]))
    torch.cuda.synchronize()
    assert torch.equal(wide[:, :n_copy], src[:, 1:1 + n_copy]) and torch.equal(wide[:, n_copy:n_copy + Cn], tot)
    assert torch.equal(wide[:, n_copy + Cn + 2:n_copy + 2 * Cn + 2], att)
    assert bool((wide[:, n_copy + Cn:n_copy + Cn + 2] == 3.0).all()) and bool((wide[:, n_copy + 2 * Cn + 2:] == 3.0).all())
    bad = bz.WeightedPoolDesc()
    bad.x, bad.w, bad.att = dx.data_ptr(), dw.data_ptr(), wide.data_ptr()
    bad.batch, bad.t, bad.c, bad.dtype, bad.ld_att = B, T, Cn, bz.bz_dtype(tdt), Cn - 1
    if Cn > 1:  # (0 means "c")
        assert bz.lib().bz_weighted_pool(C.byref(bad), None) == -22 and b"ld_att" in bz.lib().bz_last_error()
    bad.ld_att, bad.copy_c = 0, 4  # a piece to copy without its pointers
    assert bz.lib().bz_weighted_pool(C.byref(bad), None) == -22 and b"copied piece" in bz.lib().bz_last_error()
    # oracle: fp32 sums in ascending t of the rounded operands
    wm = _round_to(w * mask, dtype_name)
    want_att = np.zeros((B, Cn), np.float32)
    want_sum = np.zeros((B, Cn), np.float32)
    for t in range(T):
        want_att += wm[:, t, :] * x[:, t, :]
        want_sum += x[:, t, :]
    tol = 1e-5 if dtype_name == "f32" else 2e-3
    np.testing.assert_allclose(att.float().cpu().numpy(), want_att, rtol=tol, atol=tol * max(1.0, np.abs(want_att).max()))
    np.testing.assert_allclose(tot.float().cpu().numpy(), want_sum, rtol=tol, atol=tol * max(1.0, np.abs(want_sum).max()))


def _pieces_desc(bz, pieces, r0, r1, tdt):
    return bz.pieces_desc(pieces, r0, r1, bz.bz_dtype(tdt))


@pytest.mark.parametrize("in_name,out_name", [("f16", "f16"), ("bf16", "bf16"), ("f16", "f32")])
@pytest.mark.parametrize("r0,r1,w,N,act", [(1024, 50, 54, 80, "dice"),   # DIN's attention input in front of its first layer
                                           (37, 5, 8, 96, "prelu"),     # 8 columns a lane, ragged last tile, three column blocks
                                           (300, 1, 40, 24, "none"),    # one column block, K = 160
                                           (64, 3, 56, 40, "relu")])    # K = 224, the most the kernel holds
def test_fc_on_pieces_computed_on_the_fly(bz, oracle, in_name, out_name, r0, r1, w, N, act):
    """bz_fc_fused with a_pieces = [q, k, q-k, q*k] (q broadcast over the second row coordinate) against bz_concat_ew
    followed by the stored-matrix layer, and against the oracle fed the concat's rounded values."""
    import ctypes as C
    import torch
    print("fc on pieces %s->%s r0=%d r1=%d w=%d N=%d act=%s" % (in_name, out_name, r0, r1, w, N, act), flush=True)
    tdt, odt = _tdtype(in_name), _tdtype(out_name)
    rng = np.random.default_rng(r0 + r1 + w + N)
    M, K = r0 * r1, 4 * w
    q = _dev(_round_to(rng.standard_normal((r0, 1, w)), in_name)).to(tdt)
    k = _dev(_round_to(rng.standard_normal((r0, r1, w)), in_name)).to(tdt)
    Wkn = _round_to(rng.standard_normal((K, N)) / np.sqrt(K), in_name)
    b = (rng.standard_normal(N) * 0.1).astype(np.float32)
    params_np = ()
    if act == "prelu":
        params_np = (rng.uniform(0.1, 0.4, N).astype(np.float32), )
    elif act == "dice":
        params_np = ((rng.standard_normal(N) * 0.1).astype(np.float32), (rng.standard_normal(N) * 0.1).astype(np.float32),
                     rng.uniform(0.5, 1.5, N).astype(np.float32))
    params = tuple(_dev(x) for x in params_np)
    wp = bz.pack_weight(_dev(Wkn).to(tdt), False, bz.bz_dtype(tdt))
    pieces = [(bz.EW_ASSIGN, q, None), (bz.EW_ASSIGN, k, None), (bz.EW_SUB, q, k), (bz.EW_MUL, q, k)]
    # two launches
    a_full = bz.concat_ew(pieces).reshape(M, K)
    two = bz.fc_fused(a_full, wp, K, bias=_dev(b), act=ACT[act], act_params=params, out_dtype=bz.bz_dtype(odt), act_alpha=0.0)
    # one launch
    pd = _pieces_desc(bz, pieces, r0, r1, tdt)
    one = torch.full((M, N), float("nan"), dtype=odt, device="cuda")
    d = bz.FcDesc()
    d.a_pieces = C.cast(C.pointer(pd), C.c_void_p)
    d.w, d.y, d.bias = wp.data_ptr(), one.data_ptr(), _dev(b).data_ptr()
    bias_dev = _dev(b)
    d.bias = bias_dev.data_ptr()
    d.ldw, d.ldy = wp.stride(0), N
    d.m, d.n, d.k = M, N, K
    d.in_dtype, d.out_dtype = bz.bz_dtype(tdt), bz.bz_dtype(odt)
    d.bias_rows, d.alpha, d.beta = 1, 1.0, 1.0
    d.act, d.act_alpha = ACT[act], 0.0
    for name, p_ in zip(("act_p0", "act_p1", "act_p2"), params):
        setattr(d, name, p_.data_ptr())
    d.act_size = N if act in ("prelu", "dice") else 0
    bz.check(bz.lib().bz_fc_fused(C.byref(d), None))
    torch.cuda.synchronize()
    got, ref = one.float().cpu().numpy(), two.float().cpu().numpy()
    assert not np.isnan(got).any()
    # oracle on the concat's values (each an fp32 operation rounded once to the tensor type)
    A = a_full.float().cpu().numpy()
    pre = (A.astype(np.float64) @ Wkn.astype(np.float64) + b).astype(np.float32)
    scale = np.abs(A).astype(np.float64) @ np.abs(Wkn).astype(np.float64) + np.abs(b)
    want = {"none": lambda x: x, "relu": lambda x: oracle.leaky_relu(x, 0.0), "prelu": lambda x: oracle.prelu(x, params_np[0]),
            "dice": lambda x: oracle.dice(x, *params_np)}[act](pre)
    out_eps = {"f32": 0.0, "f16": 2.0**-11, "bf16": 2.0**-8}[out_name]
    bound = 2.0 * 2e-3 * scale + out_eps * np.abs(want) + 1e-7
    assert np.all(np.abs(got - want) <= bound)
    assert np.all(np.abs(got - ref) <= bound)


def test_fc_on_pieces_limits_are_refused(bz):
    """outside the kernel's model bz_fc_fused answers BZ_ENOTSUP and launches nothing (the caller runs the concat instead)"""
    import ctypes as C
    import torch
    q = torch.zeros((4, 1, 64), dtype=torch.float16, device="cuda")
    k = torch.zeros((4, 3, 64), dtype=torch.float16, device="cuda")
    wp = torch.zeros((16, 256), dtype=torch.float16, device="cuda")
    y = torch.zeros((12, 16), dtype=torch.float16, device="cuda")
    pieces = [(bz.EW_ASSIGN, q, None), (bz.EW_ASSIGN, k, None), (bz.EW_SUB, q, k), (bz.EW_MUL, q, k)]
    pd = _pieces_desc(bz, pieces, 4, 3, torch.float16)
    d = bz.FcDesc()
    d.a_pieces = C.cast(C.pointer(pd), C.c_void_p)
    d.w, d.y, d.ldw, d.ldy, d.m, d.n, d.k = wp.data_ptr(), y.data_ptr(), 256, 16, 12, 16, 256
    d.in_dtype = d.out_dtype = bz.F16
    d.alpha = 1.0
    assert bz.lib().bz_fc_fused(C.byref(d), None) == bz.ENOTSUP and b"a_pieces" in bz.lib().bz_last_error()  # k = 256 > 224
    pd.op[3] = bz.EW_DIV
    pd.width[0] = pd.width[1] = pd.width[2] = pd.width[3] = 40
    d.k, d.ldw = 160, 160
    assert bz.lib().bz_fc_fused(C.byref(d), None) == bz.ENOTSUP  # a piece that divides


@pytest.mark.parametrize("in_name", ["f16", "bf16"])
@pytest.mark.parametrize("r0,r1,w,N,N2,N3,act2,head_act", [
    (1024, 50, 54, 80, 40, 1, "dice", "none"),     # DIN's attention MLP 216 -> 80 -> 40 -> 1
    (37, 5, 24, 96, 64, 2, "prelu", "softmax"),    # widest second layer, a softmax head, ragged last tile
    (300, 3, 40, 24, 16, 0, "relu", "none"),       # no third layer: the second layer's output is stored
])
def test_attention_mlp_as_one_launch(bz, oracle, in_name, r0, r1, w, N, N2, N3, act2, head_act):
    """bz_fc_fused with a_pieces + next (+ head): the layers after the first run in its launch from rows that never leave
    the chip.  Against the separate launches (concat, layer, layer with its head), which round and store what this one
    only rounds."""
    import ctypes as C
    import torch
    print("attention mlp %s r0=%d r1=%d w=%d %d->%d->%d %s %s" % (in_name, r0, r1, w, N, N2, N3, act2, head_act), flush=True)
    tdt = _tdtype(in_name)
    dt = bz.bz_dtype(tdt)
    rng = np.random.default_rng(r0 + w + N + N2)
    M, K = r0 * r1, 4 * w
    q = _dev(_round_to(rng.standard_normal((r0, 1, w)), in_name)).to(tdt)
    k = _dev(_round_to(rng.standard_normal((r0, r1, w)), in_name)).to(tdt)
    W1 = _dev(_round_to(rng.standard_normal((K, N)) / np.sqrt(K), in_name)).to(tdt)
    W2 = _dev(_round_to(rng.standard_normal((N, N2)) / np.sqrt(N), in_name)).to(tdt)
    b1, b2 = _dev((rng.standard_normal(N) * 0.1).astype(np.float32)), _dev((rng.standard_normal(N2) * 0.1).astype(np.float32))
    dice1 = tuple(_dev(x) for x in ((rng.standard_normal(N) * 0.1).astype(np.float32), (rng.standard_normal(N) * 0.1).astype(np.float32),
                                    rng.uniform(0.5, 1.5, N).astype(np.float32)))
    p2 = {"dice": tuple(_dev(x) for x in ((rng.standard_normal(N2) * 0.1).astype(np.float32), (rng.standard_normal(N2) * 0.1).astype(np.float32),
                                          rng.uniform(0.5, 1.5, N2).astype(np.float32))),
          "prelu": (_dev(rng.uniform(0.1, 0.4, N2).astype(np.float32)), ), "relu": ()}[act2]
    wp1, wp2 = bz.pack_weight(W1, False, dt), bz.pack_weight(W2, False, dt)
    head = None
    if N3:
        W3 = _dev(_round_to(rng.standard_normal((N2, N3)) / np.sqrt(N2), in_name)).to(tdt)
        b3 = _dev((rng.standard_normal(N3) * 0.1).astype(np.float32))
        wp3 = bz.pack_weight(W3, False, dt)
    pieces = [(bz.EW_ASSIGN, q, None), (bz.EW_ASSIGN, k, None), (bz.EW_SUB, q, k), (bz.EW_MUL, q, k)]
    # separate launches
    a_full = bz.concat_ew(pieces).reshape(M, K)
    y1 = bz.fc_fused(a_full, wp1, K, bias=b1, act=bz.ACT_DICE, act_params=dice1)
    if N3:
        z_ref = torch.empty((M, N3), dtype=torch.float32, device="cuda")
        bz.fc_fused(y1, wp2, N, bias=b2, act=ACT[act2], act_params=p2, act_alpha=0.0,
                    head=dict(w=wp3, bias=b3, act=ACT[head_act], out=z_ref), store_out=False)
    else:
        y2_ref = bz.fc_fused(y1, wp2, N, bias=b2, act=ACT[act2], act_params=p2, act_alpha=0.0)
    # one launch
    pd = _pieces_desc(bz, pieces, r0, r1, tdt)
    nx = bz.FcNext()
    nx.w, nx.ldw, nx.n, nx.bias = wp2.data_ptr(), wp2.stride(0), N2, b2.data_ptr()
    nx.alpha = nx.beta = 1.0
    nx.act, nx.act_alpha = ACT[act2], 0.0
    for name, p_ in zip(("act_p0", "act_p1", "act_p2"), p2):
        setattr(nx, name, p_.data_ptr())
    nx.act_size = N2 if act2 in ("prelu", "dice") else 0
    d = bz.FcDesc()
    d.a_pieces = C.cast(C.pointer(pd), C.c_void_p)
    d.next = C.cast(C.pointer(nx), C.c_void_p)
    d.w, d.ldw, d.bias = wp1.data_ptr(), wp1.stride(0), b1.data_ptr()
    d.m, d.n, d.k, d.ldy = M, N, K, N
    d.in_dtype = d.out_dtype = dt
    d.bias_rows, d.alpha, d.beta = 1, 1.0, 1.0
    d.act, d.act_size = bz.ACT_DICE, N
    d.act_p0, d.act_p1, d.act_p2 = (t.data_ptr() for t in dice1)
    if N3:
        z = torch.full((M, N3), float("nan"), dtype=torch.float32, device="cuda")
        d.head_w, d.head_ldw, d.head_bias, d.head_y, d.head_ldy = wp3.data_ptr(), wp3.stride(0), b3.data_ptr(), z.data_ptr(), N3
        d.head_n, d.head_act, d.head_out_dtype = N3, ACT[head_act], bz.F32
    else:
        y2 = torch.full((M, N2), float("nan"), dtype=tdt, device="cuda")
        nx.y, nx.ldy = y2.data_ptr(), N2
    bz.check(bz.lib().bz_fc_fused(C.byref(d), None))
    torch.cuda.synchronize()
    got = (z if N3 else y2).float().cpu().numpy()
    ref = (z_ref if N3 else y2_ref).float().cpu().numpy()
    assert not np.isnan(got).any()
    eps = 2.0**-8 if in_name == "bf16" else 2.0**-11
    # three roundings of the tensor type on the way, each amplified by at most the next layer's row sums (weights ~ 1/sqrt(K))
    np.testing.assert_allclose(got, ref, rtol=0, atol=(8 * eps) * max(1.0, float(np.abs(ref).max())) + 2e-3)
    # also with the first layer's own output stored
    y1_one = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    d.y = y1_one.data_ptr()
    bz.check(bz.lib().bz_fc_fused(C.byref(d), None))
    torch.cuda.synchronize()
    np.testing.assert_allclose(y1_one.float().cpu().numpy(), y1.float().cpu().numpy(), rtol=0,
                               atol=4 * eps * max(1.0, float(y1.float().abs().max())))
    np.testing.assert_allclose((z if N3 else y2).float().cpu().numpy(), got, rtol=0, atol=0)

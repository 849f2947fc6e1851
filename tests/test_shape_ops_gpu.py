"""GPU parity of the shape / elementwise kernels around the attention unit (bz_broadcast_op, bz_reduce_sum,
bz_batch_norm, bz_softmax_axis, bz_concat_cols with a repeated row) against the CPU oracle.

Bars: Add/Sub/Mul/Div/BroadcastTo/Where/ReduceSum on fp32 tensors are single IEEE operations
(or sums in the reference's order): bit-exact.  BatchNormalization and Softmax rel 1e-5.  fp16 tensors: the fp32 result rounded once,
compared at 2e-3.
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


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


SHAPES = [
    ((1024, 1, 54), (1024, 50, 54)),      # DIN: target item against the behaviour history
    ((1, 50, 36), (7, 1, 36)),            # the example graph: one user's history against 7 candidate ads
    ((6, 5, 4, 3), (4, 1)),               # lower rank on the right
    ((3, ), (2, 5, 3)),
    ((2, 3, 1, 5, 1, 7), (1, 3, 4, 1, 6, 7)),  # rank 6, nothing merges
    ((4096, 64), (4096, 64)),             # same shape: merges to one dim
    ((1, ), (33, 17)),                    # scalar-like
    ((5, 1), (1, 9)),
]


@pytest.mark.parametrize("sa,sb", SHAPES)
@pytest.mark.parametrize("op", ["Add", "Sub", "Mul", "Div"])
def test_elementwise_broadcast_fp32_bit_exact(bz, oracle, op, sa, sb):
    import torch
    rng = np.random.default_rng(len(sa) * 100 + len(sb))
    a = rng.standard_normal(sa).astype(np.float32)
    b = (rng.standard_normal(sb) + 2.5).astype(np.float32)
    print("case", op, sa, sb, flush=True)
    code = {"Add": bz.EW_ADD, "Sub": bz.EW_SUB, "Mul": bz.EW_MUL, "Div": bz.EW_DIV}[op]
    got = bz.broadcast_op(code, _dev(a), _dev(b))
    torch.cuda.synchronize()
    want = oracle.elementwise(op, a, b)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("sa,sb", SHAPES[:4])
def test_elementwise_fp16_rounds_once(bz, oracle, sa, sb):
    import torch
    rng = np.random.default_rng(3)
    a = rng.standard_normal(sa).astype(np.float16)
    b = rng.standard_normal(sb).astype(np.float16)
    got = bz.broadcast_op(bz.EW_MUL, _dev(a), _dev(b))
    torch.cuda.synchronize()
    want = oracle.elementwise("Mul", a.astype(np.float32), b.astype(np.float32))
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want.astype(np.float16).view(np.uint16))
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("sa,target", [((1024, 1, 54), (1024, 50, 54)), ((1, 3), (4, 3)), ((2, 1, 2), (2, 2, 2)), ((5, ), (3, 4, 5))])
def test_broadcast_to(bz, oracle, sa, target):
    import torch
    a = np.random.default_rng(1).standard_normal(sa).astype(np.float32)
    got = bz.broadcast_op(bz.EW_ASSIGN, _dev(a), out_shape=target)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), oracle.broadcast_to(a, like=np.empty(target)))


@pytest.mark.parametrize("cdt", [np.int32, np.int64])
@pytest.mark.parametrize("sc,sx,sy", [((1, 100, 1), (64, 100, 1), (1, 100, 1)), ((2, 2), (2, 2), (2, 2)), ((8, 1, 3), (1, 5, 3), (3, ))])
def test_where(bz, oracle, cdt, sc, sx, sy):
    import torch
    rng = np.random.default_rng(9)
    cond = rng.integers(0, 2, sc).astype(cdt) * rng.integers(1, 5, sc).astype(cdt)  # any nonzero value is true
    x = rng.standard_normal(sx).astype(np.float32)
    y = np.full(sy, -4294967295.0, np.float32)  # the padding constant of the example graph
    got = bz.broadcast_op(bz.EW_WHERE, _dev(cond), _dev(x), _dev(y))
    torch.cuda.synchronize()
    want = oracle.where(cond, x, y)
    assert tuple(got.shape) == want.shape and np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape,axis", [((1024, 50, 54), 1), ((2, 3, 2), 1), ((7, 9), 0), ((7, 9), 1), ((3, 1, 5), 1), ((4, 6, 5, 3), 2),
                                        ((100003, ), 0)])
@pytest.mark.parametrize("keepdims", [0, 1])
def test_reduce_sum_bit_exact(bz, oracle, shape, axis, keepdims):
    import torch
    x = np.random.default_rng(axis).standard_normal(shape).astype(np.float32)
    print("case reduce_sum", shape, axis, flush=True)
    got = bz.reduce_sum(_dev(x), axis, bool(keepdims))
    torch.cuda.synchronize()
    want = oracle.reduce_sum(x, axis, keepdims)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape,c", [((2, 3), 3), ((1024, 162), 162), ((4, 5, 6), 6), ((4, 5, 6), 30)])
@pytest.mark.parametrize("nosqrt", [False, True])
def test_batch_norm(bz, oracle, shape, c, nosqrt):
    import torch
    rng = np.random.default_rng(c)
    x = rng.standard_normal(shape).astype(np.float32)
    gamma, beta, mean = (rng.standard_normal(c).astype(np.float32) for _ in range(3))
    var = (rng.random(c) + 0.5).astype(np.float32)
    got = bz.batch_norm(_dev(x), _dev(gamma), _dev(beta), _dev(mean), _dev(var), 0.001, nosqrt)
    torch.cuda.synchronize()
    want = oracle.batch_norm(x, gamma, beta, mean, var, 0.001, nosqrt)
    g = got.cpu().numpy()
    # fp32 bar of the path: rel 1e-5 (abs 1e-6 where gamma*xn and beta cancel)
    np.testing.assert_allclose(g, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape,axis", [((1024, 50, 1), 1), ((64, 100, 1), 1), ((3, 4, 5), 1), ((3, 4, 5), 0), ((6, 7), 1), ((2, 3, 2, 2), 2)])
def test_softmax_axis(bz, oracle, shape, axis):
    import torch
    x = (np.random.default_rng(5).standard_normal(shape) * 3).astype(np.float32)
    got = bz.softmax_axis(_dev(x), axis)
    torch.cuda.synchronize()
    want = oracle.softmax(x, axis)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-7)


def test_fuse_repeats_the_single_row(bz, oracle):
    """bz_concat_cols with src_pitch 0 = the Fuse operator (fuse_op.cc:11-33)."""
    import ctypes as C
    import torch
    rng = np.random.default_rng(2)
    for comm, (s1, s2) in ((0, ((1, 36), (200, 72))), (1, ((200, 18), (1, 90)))):
        x1, x2 = rng.standard_normal(s1).astype(np.float32), rng.standard_normal(s2).astype(np.float32)
        d1, d2 = _dev(x1), _dev(x2)
        m, n1, n2 = max(s1[0], s2[0]), s1[1], s2[1]
        out = torch.full((m, n1 + n2), float("nan"), device="cuda")
        d = bz.ConcatDesc()
        d.n = 2
        d.src[0], d.src[1] = d1.data_ptr(), d2.data_ptr()
        d.width[0], d.width[1] = n1 * 4, n2 * 4
        d.src_pitch[0], d.src_pitch[1] = (0 if s1[0] == 1 else n1 * 4), (0 if s1[0] != 1 else n2 * 4)
        d.dst, d.dst_pitch, d.rows = out.data_ptr(), (n1 + n2) * 4, m
        bz.check(bz.lib().bz_concat_cols(C.byref(d), None))
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), oracle.fuse(x1, x2, comm))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("r0,r1,w,kshape", [(64, 50, 54, "q"),     # DIN: [q, k, q-k, q*k], q broadcast over the history
                                            (7, 50, 36, "k"),      # the example graph: one history, 7 candidate ads
                                            (33, 1, 8, "q"),       # 2-D after merging, widths a multiple of 8
                                            (5, 3, 7, "q")])       # odd width: one column per thread
def test_concat_of_pieces_computed_on_the_fly_equals_the_separate_operators(bz, oracle, dtype, r0, r1, w, kshape):
    """bz_concat_ew against the oracle's BroadcastTo / Sub / Mul / Add / Div followed by Concat: bit-identical
    (every element is one fp32 operation on the widened operands, rounded once)."""
    import torch
    rng = np.random.default_rng(r0 * 1000 + r1 * 10 + w)
    qs, ks = ((r0, 1, w), (r0, r1, w)) if kshape == "q" else ((r0, 1, w), (1, r1, w))
    q = rng.standard_normal(qs).astype(dtype)
    k = (rng.standard_normal(ks) + 2.5).astype(dtype)
    print("case", dtype.__name__, r0, r1, w, kshape, flush=True)
    qd, kd = _dev(q), _dev(k)
    got = bz.concat_ew([(bz.EW_ASSIGN, qd, None), (bz.EW_ASSIGN, kd, None), (bz.EW_SUB, qd, kd), (bz.EW_MUL, qd, kd),
                        (bz.EW_ADD, kd, qd), (bz.EW_DIV, qd, kd)])
    torch.cuda.synchronize()
    rnd = (lambda x: x.astype(dtype).astype(np.float32))
    qf, kf = q.astype(np.float32), k.astype(np.float32)
    full = (r0, r1, w)
    want = oracle.concat([rnd(oracle.broadcast_to(qf, shape=full)), rnd(oracle.broadcast_to(kf, shape=full)),
                          rnd(oracle.elementwise("Sub", qf, kf)), rnd(oracle.elementwise("Mul", qf, kf)),
                          rnd(oracle.elementwise("Add", kf, qf)), rnd(oracle.elementwise("Div", qf, kf))], 2).astype(dtype)
    assert tuple(got.shape) == want.shape
    view = np.uint32 if dtype == np.float32 else np.uint16
    assert np.array_equal(got.cpu().numpy().view(view), want.view(view))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("r0,r1,widths", [(40, 50, (54, 18, 8)),    # pieces of different widths: a lane looks its piece up
                                          (9, 3, (130, 130)),        # one width, but more than 64 lanes' worth of a row
                                          (300, 7, (64, 64, 64, 64))])
def test_concat_of_pieces_of_mixed_widths(bz, oracle, dtype, r0, r1, widths):
    """bz_concat_ew's general kernel (the pieces' widths differ, or a piece is wider than a wave covers): piece i is
    q_i - k_i for even i and a copy of k_i for odd i, q_i broadcast over the second row coordinate."""
    import torch
    rng = np.random.default_rng(r0 + r1 + sum(widths))
    pieces, want = [], []
    for i, w in enumerate(widths):
        q = rng.standard_normal((r0, 1, w)).astype(dtype)
        k = rng.standard_normal((r0, r1, w)).astype(dtype)
        if i % 2 == 0:
            pieces.append((bz.EW_SUB, _dev(q), _dev(k)))
            want.append(oracle.elementwise("Sub", q.astype(np.float32), k.astype(np.float32)).astype(dtype))
        else:
            pieces.append((bz.EW_ASSIGN, _dev(k), None))
            want.append(k)
    print("case", dtype.__name__, r0, r1, widths, flush=True)
    got = bz.concat_ew(pieces)
    torch.cuda.synchronize()
    want = np.concatenate(want, axis=2)
    view = np.uint32 if dtype == np.float32 else np.uint16
    assert tuple(got.shape) == want.shape and np.array_equal(got.cpu().numpy().view(view), want.view(view))


def test_bad_descriptors_are_refused(bz):
    import ctypes as C
    d = bz.BcastDesc()
    assert bz.lib().bz_broadcast_op(C.byref(d), None) != 0  # rank 0
    d.rank = 7
    assert bz.lib().bz_broadcast_op(C.byref(d), None) != 0
    assert b"rank" in bz.lib().bz_last_error()
    assert bz.lib().bz_reduce_sum(None, None, 1, 1, 1, bz.F32, None) != 0
    assert bz.lib().bz_softmax_axis(None, None, 1, 1, 1, bz.F32, None) != 0
    e = bz.ConcatEwDesc()
    assert bz.lib().bz_concat_ew(C.byref(e), None) != 0  # no pieces
    assert b"pieces" in bz.lib().bz_last_error()

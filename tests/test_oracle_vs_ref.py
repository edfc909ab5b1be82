"""The CPU oracle against the real reference library, live, bit for bit.  Runs only where
oracle/_ref/libctorch_ref.so has been built (the reference sources are mounted); elsewhere the
golden vectors written from the same library stand in (test_oracle_golden.py)."""
import numpy as np
import pytest

from support import (ADD, CE, COS, DIV, DOT, MAE, MATMUL, MSE, MUL, NEG, RELU, SIGMOID, SIN, SUB, TANH,
                     same_bits)

UNARY = [(NEG, "neg"), (RELU, "relu"), (SIN, "sin"), (COS, "cos"), (TANH, "tanh"), (SIGMOID, "sigmoid")]


def eq(a, b, what=""):
    assert same_bits(a, b), what


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_elementwise_forward(oracle, ref, seed):
    x = oracle.normal((3001,), 10 + seed, 0, 3)
    y = oracle.normal((3001,), 20 + seed, 0, 3)
    for code in (ADD, SUB, MUL, DIV):
        rc, out = ref.binary(code, x, y, x.shape)
        eq(oracle.binary(code, x, y), out, code)
    for code, name in UNARY:
        eq(oracle.unary(code, x), ref.unary(code, x), name)
    for which, s in [(0, 5.0), (1, -2.5), (2, 3.0)]:
        eq(oracle.scalar(which, x, s), ref.scalar(which, x, s)[1], which)


@pytest.mark.parametrize("n", list(range(1, 41)) + [53, 100, 1003, 65537])
def test_contiguous_reductions_every_tail_length(oracle, ref, n):
    """Dot / MSE / row-wise softmax gradient share one compiled loop shape whose bits depend on
    n mod 8; every residue is checked, several draws each."""
    for seed in range(6):
        a = oracle.normal((n,), 1000 + 7 * seed + n)
        b = oracle.normal((n,), 5000 + 11 * seed + n)
        eq(oracle.dot(a, b), ref.binary(DOT, a, b, ())[1], ("dot", n, seed))
        eq(oracle.mse(a, b), ref.binary(MSE, a, b, ())[1], ("mse", n, seed))
        eq(oracle.mae(a, b), ref.binary(MAE, a, b, ())[1], ("mae", n, seed))
        eq(oracle.sum(a), ref.sum(a), ("sum", n, seed))
    if n <= 100:
        x = oracle.normal((5, n), 77 + n, 0, 2)
        w = oracle.normal((5, n), 78 + n)
        up = oracle.accumulate0(w)
        eq(oracle.accumulate0(oracle.softmax_bwd(oracle.softmax(x, 1), up, 1)), ref.grad_softmax(x, 1, w), n)
        eq(oracle.accumulate0(oracle.softmax_bwd(oracle.softmax(x, 0), up, 0)), ref.grad_softmax(x, 0, w), n)


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (33, 47), (64, 130)])
def test_softmax_ce(oracle, ref, shape):
    x = oracle.normal(shape, 31, 0, 2.5)
    eq(oracle.softmax(x, 1), ref.softmax(x, 1))
    eq(oracle.softmax(x, 0), ref.softmax(x, 0))
    idx = oracle.ints((shape[0],), 32, shape[1])
    oh = np.zeros(shape, np.float32)
    oh[np.arange(shape[0]), idx.astype(int)] = 1
    eq(oracle.ce_onehot(x, oh), ref.binary(CE, x, oh, ())[1])
    if shape[1] != shape[0]:   # equal extents make the reference take the one-hot branch
        eq(oracle.ce_index(x, idx), ref.binary(CE, x, idx, ())[1])
    soft = oracle.softmax(oracle.normal(shape, 33), 1)   # soft targets
    eq(oracle.ce_onehot(x, soft), ref.binary(CE, x, soft, ())[1])
    rc, loss, dp = ref.grad_loss(CE, x, oh, -1.25)
    eq(oracle.accumulate0(oracle.ce_bwd_onehot(x, oh, np.float32(-1.25))), dp)
    eq(loss, oracle.ce_onehot(x, oh))


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (5, 3, 9), (33, 29, 47), (16, 64, 128)])
def test_matmul_layouts_and_gradients(oracle, ref, m, n, k):
    A = oracle.normal((m, k), 41)
    B = oracle.normal((k, n), 42)
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    eq(oracle.matmul(A, B), ref.matmul_t(A, 0, B, 0))
    eq(oracle.matmul(A, Bt.T), ref.matmul_t(A, 0, Bt, 1))
    eq(oracle.matmul(At.T, B), ref.matmul_t(At, 1, B, 0))
    eq(oracle.matmul(At.T, Bt.T), ref.matmul_t(At, 1, Bt, 1))
    W = oracle.normal((m, n), 43)
    rc, da, db = ref.grad_binary(MATMUL, A, B, W)
    up = oracle.accumulate0(W)
    eq(oracle.accumulate0(oracle.matmul(up, B.T)), da)
    eq(oracle.accumulate0(oracle.matmul(A.T, up)), db)


def test_elementwise_gradients(oracle, ref):
    x = oracle.normal((23, 31), 51, 0, 2)
    y = oracle.normal((23, 31), 52, 0, 2)
    w = oracle.normal((23, 31), 53)
    acc = oracle.accumulate0
    up = acc(w)
    for code, name in UNARY:
        eq(acc(oracle.unary_bwd(code, x, up)), ref.grad_unary(code, x, w), name)
    for code, fn in [(MSE, oracle.mse_bwd), (MAE, oracle.mae_bwd)]:
        for scale in (1.0, 0.37):
            eq(acc(fn(x, y, np.float32(scale))), ref.grad_loss(code, x, y, scale)[2], (code, scale))
    yb = (y + np.float32(4.0) * np.sign(y)).astype(np.float32)
    rc, da, db = ref.grad_binary(DIV, x, yb, w)
    eq(acc(oracle.div_bwd_a(up, yb)), da)
    eq(acc(oracle.div_bwd_b(x, yb, up)), db)
    rc, da, db = ref.grad_binary(MUL, x, y, w)
    eq(acc(oracle.mul(y, up)), da)
    eq(acc(oracle.mul(x, up)), db)
    rc, da, db = ref.grad_binary(SUB, x, y, w)
    eq(acc(up), da)
    eq(acc(oracle.neg(up)), db)
    b = oracle.uniform((31,), 54, -1, 1)
    rc, da, db = ref.grad_binary(ADD, x, b, w)
    eq(acc(up), da)
    eq(acc(oracle.adjust_row0(up)), db)


def test_configurations(oracle, ref):
    a = oracle.uniform((10007,), 101, -1, 1)
    b = oracle.uniform((10007,), 102, -1, 1)
    for got, want in zip(oracle.chain(a, b), ref.chain(a, b)):
        eq(got, want)
    Bn, I, H, Cn = 24, 50, 32, 10
    x = (oracle.ints((Bn, I), 301, 256) / np.float32(255.0)).astype(np.float32)
    lab = oracle.ints((Bn,), 302, Cn).astype(int)
    oh = np.zeros((Bn, Cn), np.float32)
    oh[np.arange(Bn), lab] = 1
    k1, k2 = 1 / np.sqrt(I), 1 / np.sqrt(H)
    W1, b1 = oracle.uniform((I, H), 311, -k1, k1), oracle.uniform((H,), 312, -k1, k1)
    W2, b2 = oracle.uniform((H, Cn), 313, -k2, k2), oracle.uniform((Cn,), 314, -k2, k2)
    for got, want in zip(oracle.mlp_step(x, W1, b1, W2, b2, oh, True), ref.mlp_step(x, W1, b1, W2, b2, oh)):
        eq(got, want)
    X = oracle.uniform((16, 24), 501, -2, 2)
    rv = oracle.uniform((24,), 502, 0.5, 2)
    T = oracle.normal((16, 24), 503)
    R = np.broadcast_to(rv, X.shape).copy()
    for got, want in zip(oracle.expr(X, R, T), ref.expr(X, R, T)):
        eq(got, want)


def test_tensors_that_are_not_fp32(oracle, ref):
    """The typed cases live against the reference (the committed vectors are these results), and the
    fact the front-end relies on: backward() through a double / int tensor throws in the reference."""
    from support import typed_cases
    for name, a, dt, steps in typed_cases(oracle):
        rc, want = ref.typed(a, dt, steps)
        assert rc == a.size, name
        got = oracle.typed(a, dt, steps)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name
    x = oracle.normal((2, 3), 5, 0, 10)
    for dt in (1, 2, 3):
        for steps in ([(0, 5.0)], [(1, 3.0)], [(1, 3.0), (0, 5.0)], [(2, 4.0)]):
            assert ref.typed_grad(x, dt, steps)[0] == -1, (dt, steps)
    rc, code, raw = ref.typed_grad(x, 0, [(1, 3.0), (0, 5.0)])
    assert rc == 6 and code == 0 and np.array_equal(raw.view(np.float32)[:6], np.full(6, 3.0, np.float32))


# shape pairs (gradient, target) that keep the reference's index arithmetic inside the gradient's
# buffer, one or more for every branch of check_and_adjust_grad_shape (src/AutoDiff.cpp:562-1049)
ADJUST_CASES = [
    ((2, 3), (2, 3)),        # :565-567  equal
    ((), (2, 3)), ((), (5,)),                      # :579-627  0-D gradient
    ((3,), (1, 3)), ((4,), (4, 1)), ((6,), (1, 1, 6)), ((2, 3), (1, 2, 3)),   # :633-687 rank(g) < rank(target)
    ((1,), (2, 3)),          # :633-687 then the broadcast branch from a one-element gradient
    ((2, 3), (3,)), ((4, 5), (5,)), ((2, 3, 4), (4,)), ((2, 3, 4), (3, 4)),   # :690-757 slice with leading index 0
    ((2, 3), (1,)), ((2, 3), ()), ((3, 1), (3, 1)), ((5, 1), (1,)), ((4, 1), (2,)),   # one-element / last dim 1
    ((2, 6), (3,)), ((6,), (2, 2)), ((3, 5), (2,)), ((7,), (3,)), ((2, 3), (4, 3)),   # :968-1046 modulo fold
]


@pytest.mark.parametrize("gshape, tshape", ADJUST_CASES)
def test_gradient_shape_adjustment_every_branch(oracle, ref, gshape, tshape):
    for seed in range(3):
        g = oracle.normal(gshape if gshape else (1,), 900 + seed, 0, 2).reshape(gshape)
        if seed == 1:
            g.reshape(-1)[0] = -0.0                  # the broadcast branch adds to +0: -0 must come out +0
        want = ref.adjust_grad_shape(g, tshape)
        assert want is not None
        got = oracle.adjust_grad_shape(g, tshape)
        assert got is not None
        eq(got, want, (gshape, tshape, seed))


def test_gradient_shape_adjustment_flags_the_reads_beyond_the_buffer(oracle):
    # [3] -> [2, 3] and [1, 3] -> [2, 3]: the reference indexes the gradient with the flat result
    # index (0..5) and reads past its three elements; the restatement reports that instead
    g = oracle.normal((3,), 1)
    assert oracle.adjust_grad_shape(g, (2, 3)) is None
    assert oracle.adjust_grad_shape(g.reshape(1, 3), (2, 3)) is None

"""Pins the CPU oracle without the reference binary: the known answers of the reference's own
tests (src/tests/test.cpp, test_tensor_grad.cpp, test_activation_loss.cpp) and what the
mathematics fixes (exact integer products, fp64 recomputation, identities that a transposed
operand, a dropped term or a wrong sign would break)."""
import numpy as np

from support import ADD, DIV, MUL, SUB, same_bits, ulp_diff

F = np.float32


def test_scalar_gradients_of_reference_unit_test(oracle):
    # src/tests/test.cpp:6-155: a=2, b=3 -> d(a+b)=(1,1), d(a*b)=(3,2), d(a-b)=(1,-1), d(-a)=-1;
    # a=6, b=2... the test's division case expects (0.5, -1.5) for a=3, b=2.
    one = np.ones(1, F)
    a, b = np.array([2.0], F), np.array([3.0], F)
    assert oracle.mul(b, one)[0] == 3.0 and oracle.mul(a, one)[0] == 2.0
    assert oracle.neg(one)[0] == -1.0
    a, b = np.array([3.0], F), np.array([2.0], F)
    assert abs(oracle.div_bwd_a(one, b)[0] - 0.5) < 1e-6
    assert abs(oracle.div_bwd_b(a, b, one)[0] - (-0.75)) < 1e-6   # -a/b^2 = -3/4
    a, b = np.array([6.0], F), np.array([2.0], F)
    assert abs(oracle.div_bwd_b(a, b, one)[0] - (-1.5)) < 1e-6


def test_tensor_gradients_of_reference_unit_test(oracle):
    # src/tests/test_tensor_grad.cpp:7-73: d = 2*(a+b) -> both gradients all 2
    up = oracle.scalar(1, np.ones((2, 3), F), 2.0)       # Mul backward: other(=2) * ones
    assert np.all(oracle.accumulate0(up) == 2.0)
    # :76-149: c = a[2,3] + b[3], backward(c): the reference expects db == 1 (row 0, not the sum 2)
    g = np.ones((2, 3), F)
    assert np.all(oracle.adjust_row0(g) == 1.0)
    assert np.all(oracle.colsum_f64(g) == 2.0)
    # :152-224: z = x*y + x -> dx = y + 1, dy = x
    x = np.arange(6, dtype=F).reshape(2, 3)
    y = (np.arange(6, dtype=F).reshape(2, 3) + 1)
    ones = np.ones_like(x)
    dx = oracle.accumulate0(ones)              # Add branch edge to x
    dx = dx + oracle.mul(y, ones)              # Mul branch edge to x
    assert np.array_equal(dx, y + 1) and np.array_equal(oracle.mul(x, ones), x)


def test_activation_loss_properties_of_reference_unit_test(oracle):
    # src/tests/test_activation_loss.cpp:57-65, 94-112: softmax rows / columns sum to 1
    x = oracle.normal((7, 11), 5, 0, 2)
    assert np.allclose(oracle.softmax(x, 1).sum(1), 1, atol=1e-6)
    assert np.allclose(oracle.softmax(x, 0).sum(0), 1, atol=1e-6)
    assert abs(oracle.softmax(x[0]).sum() - 1) < 1e-6
    # :114-126: d(sum(softmax(x)))/dx ~ 0
    y = oracle.softmax(x, 1)
    assert np.abs(oracle.softmax_bwd(y, np.ones_like(y), 1)).max() < 1e-4
    # :156-170: CE(1-D one-hot) == -log(softmax[true]); :172-189: dCE/dz == softmax - target
    z = x[0]
    t = np.zeros_like(z)
    t[4] = 1
    assert abs(oracle.ce_onehot(z, t) - (-np.log(oracle.softmax(z)[4]))) < 1e-4
    assert np.abs(oracle.ce_bwd_onehot(z, t, F(1.0)) - (oracle.softmax(z) - t)).max() < 1e-4


def test_ieee_special_values(oracle):
    x = np.array([0.0, -0.0, np.nan, -np.inf, np.inf, -1e-45, 1e-45], F)
    r = oracle.relu(x)
    assert same_bits(r, np.array([0.0, 0.0, 0.0, 0.0, np.inf, 0.0, 1e-45], F))   # -0 -> +0, NaN -> +0
    n = oracle.neg(x)
    assert same_bits(n[:2], np.array([-0.0, 0.0], F)) and np.isnan(n[2])
    assert np.signbit(oracle.neg(np.array([np.nan], F)))[0] != np.signbit(np.array([np.nan], F))[0]
    # relu gradient is a multiply by the 0/1 mask: g*0 keeps g's sign and propagates NaN/inf
    g = np.array([-3.0, np.inf, np.nan, 2.0], F)
    xm = np.array([-1.0, -1.0, -1.0, 1.0], F)
    d = oracle.relu_bwd(xm, g)
    assert same_bits(d[:1], np.array([-0.0], F)) and np.isnan(d[1]) and np.isnan(d[2]) and d[3] == 2.0
    # tanh is NaN (inf/inf) once exp overflows: Tanh_BASIC_kernel.cpp:25-27
    assert np.isnan(oracle.tanh(np.array([89.0], F))[0]) and oracle.tanh(np.array([80.0], F))[0] == 1.0
    # division by zero yields the IEEE quotient
    q = oracle.div(np.array([1.0, -1.0, 0.0], F), np.zeros(3, F))
    assert q[0] == np.inf and q[1] == -np.inf and np.isnan(q[2])


def test_binary_ops_are_the_correctly_rounded_ieee_ops(oracle):
    a = oracle.normal((5000,), 1, 0, 100)
    b = oracle.normal((5000,), 2, 0, 1e-3)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert same_bits(oracle.binary(ADD, a, b), (a64 + b64).astype(F))
    assert same_bits(oracle.binary(SUB, a, b), (a64 - b64).astype(F))
    assert same_bits(oracle.binary(MUL, a, b), (a64 * b64).astype(F))   # exact in fp64, one rounding
    assert same_bits(oracle.binary(DIV, a, b), a / b)


def test_transcendentals_against_fp64(oracle):
    x = np.concatenate([oracle.uniform((20000,), 3, -8, 8), oracle.uniform((5000,), 4, -100, 100)])
    x64 = x.astype(np.float64)
    assert ulp_diff(oracle.sin(x), np.sin(x64).astype(F)).max() <= 1
    assert ulp_diff(oracle.cos(x), np.cos(x64).astype(F)).max() <= 1
    xs = x[np.abs(x) < 80]
    assert ulp_diff(oracle.sigmoid(xs), (1 / (1 + np.exp(-xs.astype(np.float64)))).astype(F)).max() <= 2
    xt = xs[np.abs(xs) > 0.5]   # away from the cancellation region of the two-exp formula
    assert ulp_diff(oracle.tanh(xt), np.tanh(xt.astype(np.float64)).astype(F)).max() <= 4


def test_matmul_exact_on_small_integers_and_layout_identities(oracle):
    rng = np.random.default_rng(7)
    A = rng.integers(-8, 9, (17, 23)).astype(F)
    B = rng.integers(-8, 9, (23, 13)).astype(F)
    C = oracle.matmul(A, B)
    assert np.array_equal(C.astype(np.int64), A.astype(np.int64) @ B.astype(np.int64))   # exact in fp32
    # non-square, asymmetric operands: a transposed or swapped operand cannot pass
    A = oracle.normal((9, 31), 8)
    B = oracle.normal((31, 5), 9)
    C = oracle.matmul(A, B)
    C64 = A.astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert np.all(np.abs(C - C64) <= bound)
    # (A B)^T = B^T A^T with identical bits: same products, same order of accumulation
    assert same_bits(oracle.matmul(B.T, A.T), np.ascontiguousarray(C.T))


def test_reductions_against_fp64(oracle):
    a = oracle.uniform((20003,), 11, -1, 1)   # sequential fp32 sums lose ~n*2^-25 relative
    b = oracle.uniform((20003,), 12, -1, 1)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    assert abs(oracle.dot(a, b) - a64 @ b64) <= 1e-5 * np.abs(a64 * b64).sum()
    assert abs(oracle.sum(a) - a64.sum()) <= 1e-5 * np.abs(a64).sum()
    assert abs(oracle.mse(a, b) - ((a64 - b64) ** 2).mean()) <= 1e-5 * ((a64 - b64) ** 2).mean()
    assert abs(oracle.mae(a, b) - np.abs(a64 - b64).mean()) <= 1e-5 * np.abs(a64 - b64).mean()
    # MSE of a constant offset is the square of the offset; MAE its magnitude
    assert oracle.mse(a, a + F(0.5)) == F(0.25) and oracle.mae(a + F(0.5), a) == F(0.5)


def test_cross_entropy_closed_forms(oracle):
    x = oracle.normal((13, 37), 21, 0, 2)
    idx = oracle.ints((13,), 22, 37)
    oh = np.zeros_like(x)
    oh[np.arange(13), idx.astype(int)] = 1
    x64 = x.astype(np.float64)
    lse = np.log(np.exp(x64 - x64.max(1, keepdims=True)).sum(1)) + x64.max(1)
    want = (lse - x64[np.arange(13), idx.astype(int)]).sum()      # SUM over rows, not the mean
    assert abs(oracle.ce_onehot(x, oh) - want) <= 1e-5 * abs(want)
    assert abs(oracle.ce_index(x, idx) - want) <= 1e-5 * abs(want)
    # uniform logits: loss = rows * log(classes)
    u = np.zeros((4, 10), F)
    assert abs(oracle.ce_index(u, np.zeros(4, F)) - 4 * np.log(10)) < 1e-5
    # the 1e-10 clamp: a class 60 below the maximum has p ~ 8.8e-27 -> -log(1e-10)
    s = np.zeros((1, 2), F)
    s[0, 0] = 60.0
    assert abs(oracle.ce_index(s, np.array([1.0], F)) - (-np.log(1e-10))) < 1e-4
    # gradient rows sum to ~0 and equal softmax - onehot
    d = oracle.ce_bwd_index(x, idx, F(1.0))
    assert np.abs(d.sum(1)).max() < 1e-5
    assert same_bits(d, oracle.ce_bwd_onehot(x, oh, F(1.0)))
    sm = np.exp(x64 - lse[:, None])
    assert np.abs(d - (sm - oh)).max() < 1e-6


def test_expression_gradients_against_fp64_closed_form(oracle):
    rows, cols = 24, 16
    X = oracle.uniform((rows, cols), 501, -2, 2)
    r = oracle.uniform((cols,), 502, 0.5, 2)
    T = oracle.normal((rows, cols), 503)
    R = np.broadcast_to(r, X.shape).copy()
    Y, mse, mae, gX, gR = oracle.expr(X, R, T)
    x, rr, t = X.astype(np.float64), R.astype(np.float64), T.astype(np.float64)
    sig = 1 / (1 + np.exp(-x / rr))
    y = sig - np.tanh(x) * np.sin(x) + np.cos(-x)
    n = x.size
    gy = 2 * (y - t) / n + np.sign(y - t) / n
    dsig = sig * (1 - sig)
    gx = gy * (dsig / rr - (1 - np.tanh(x) ** 2) * np.sin(x) - np.tanh(x) * np.cos(x) - np.sin(x))
    gr = gy * dsig * (-x / rr ** 2)
    assert np.abs(Y - y).max() < 1e-6
    assert abs(mse - ((y - t) ** 2).mean()) < 1e-6 and abs(mae - np.abs(y - t).mean()) < 1e-6
    assert np.abs(gX - gx).max() < 1e-8 and np.abs(gR - gr).max() < 1e-8
    # the complete gradient of the row vector is the column sum of gR
    assert np.abs(oracle.colsum_f64(gR) - gr.sum(0)).max() < 1e-7


def test_mlp_gradients_against_fp64(oracle):
    Bn, I, H, C = 12, 20, 16, 10
    x = (oracle.ints((Bn, I), 301, 256) / F(255.0)).astype(F)
    lab = oracle.ints((Bn,), 302, C).astype(int)
    oh = np.zeros((Bn, C), F)
    oh[np.arange(Bn), lab] = 1
    k1, k2 = 1 / np.sqrt(I), 1 / np.sqrt(H)
    W1, b1 = oracle.uniform((I, H), 311, -k1, k1), oracle.uniform((H,), 312, -k1, k1)
    W2, b2 = oracle.uniform((H, C), 313, -k2, k2), oracle.uniform((C,), 314, -k2, k2)
    loss, logits, gW1, gb1, gW2, gb2 = oracle.mlp_step(x, W1, b1, W2, b2, oh, False)
    d = np.float64
    a1 = x.astype(d) @ W1.astype(d) + b1.astype(d)
    h = np.maximum(a1, 0)
    lg = h @ W2.astype(d) + b2.astype(d)
    p = np.exp(lg - lg.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    assert abs(loss - (-np.log(p[np.arange(Bn), lab])).sum()) < 1e-4
    gl = p - oh
    assert np.abs(gW2 - h.T @ gl).max() < 1e-5 and np.abs(gb2 - gl.sum(0)).max() < 1e-5
    ga1 = (gl @ W2.astype(d).T) * (a1 > 0)
    assert np.abs(gW1 - x.astype(d).T @ ga1).max() < 1e-5 and np.abs(gb1 - ga1.sum(0)).max() < 1e-5
    # strict mode reproduces the reference's bias gradient: row 0 of the upstream gradient
    _, _, _, gb1s, _, gb2s = oracle.mlp_step(x, W1, b1, W2, b2, oh, True)
    assert np.abs(gb2s - gl[0]).max() < 1e-6 and np.abs(gb1s - ga1[0]).max() < 1e-6


def test_input_generator_is_stable(oracle):
    u = oracle.uniform((4,), 101, -1, 1)
    assert np.all((u >= -1) & (u < 1))
    assert same_bits(u, oracle.uniform((8,), 101, -1, 1)[:4])        # counter based: prefix-stable
    z = oracle.normal((200000,), 7)
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1) < 0.01
    k = oracle.ints((100000,), 9, 10)
    assert k.min() == 0 and k.max() == 9 and abs(k.mean() - 4.5) < 0.05

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


# --------------------------------------------------------------------------------------------
# The methods the reference declares on Tensor and never defines (include/Tensor.h:719, 824-1072):
# no reference run can pin their oracle functions, so the mathematics does - numpy in double,
# closed forms, brute force on tiny inputs, and central differences for the gradients.  Each check is
# chosen so that a plausible slip (wrong ddof, wrong sign, axis mix-up, last instead of first
# extreme, dropped factor 2) fails it.

def _numeric_gradient(f, x, eps=1e-6):
    """Central differences of a scalar function of a float64 array."""
    g = np.zeros_like(x)
    flat, gf = x.reshape(-1), g.reshape(-1)
    for i in range(flat.size):
        keep = flat[i]
        flat[i] = keep + eps
        up = f(x)
        flat[i] = keep - eps
        down = f(x)
        flat[i] = keep
        gf[i] = (up - down) / (2 * eps)
    return g


def test_extension_unary_operators_against_double_precision(oracle):
    x = np.concatenate([oracle.normal((4000,), 41, 0, 3), np.array([0.0, -0.0, 1.0, -1.0, 0.5, 88.0, -88.0, 1e-30, 3e38], F)])
    pos = np.abs(x) + F(1e-3)
    x64, pos64 = x.astype(np.float64), pos.astype(np.float64)
    assert same_bits(oracle.unary_ext("abs", x), np.abs(x))
    with np.errstate(over="ignore"):
        assert same_bits(oracle.unary_ext("square", x), x * x)
    assert same_bits(oracle.unary_ext("sqrt", pos), np.sqrt(pos))                 # IEEE: correctly rounded
    assert same_bits(oracle.unary_ext("sub_scalar", x, 1.25), x - F(1.25))
    lr = oracle.unary_ext("leaky_relu", x, 0.01)
    assert same_bits(lr, np.where(x > 0, x, x * F(0.01)))
    assert lr[np.where(x == -1.0)[0][0]] == F(-0.01)
    with np.errstate(over="ignore"):
        assert ulp_diff(oracle.unary_ext("exp", x), np.exp(x64).astype(F)).max() <= 1
    assert ulp_diff(oracle.unary_ext("log", pos), np.log(pos64).astype(F)).max() <= 1
    small = x[np.abs(x) < 50]
    assert ulp_diff(oracle.unary_ext("tan", small), np.tan(small.astype(np.float64)).astype(F)).max() <= 1
    # identities: exp(log(x)) = x, tan = sin / cos, sqrt(x)^2 = x
    assert np.allclose(oracle.unary_ext("exp", oracle.unary_ext("log", pos)), pos, rtol=5e-6)
    assert np.allclose(oracle.unary_ext("tan", small), oracle.sin(small) / oracle.cos(small), rtol=1e-5, atol=1e-6)
    # special values of the library calls
    assert np.isneginf(oracle.unary_ext("log", np.zeros(1, F))[0]) and np.isnan(oracle.unary_ext("log", np.array([-1.0], F))[0])
    assert np.isnan(oracle.unary_ext("sqrt", np.array([-4.0], F))[0]) and oracle.unary_ext("sqrt", np.array([-0.0], F)).view(np.uint32)[0] == 0x80000000


def test_extension_unary_gradients_against_central_differences(oracle):
    x = oracle.uniform((24,), 43, 0.3, 1.4)        # positive, inside (0, pi/2): every operator is smooth there
    x[::3] *= F(-1.0)
    w = oracle.normal((24,), 44)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    fns = {
        "abs": (np.abs, x), "exp": (np.exp, x), "square": (np.square, x), "tan": (np.tan, x),
        "log": (np.log, np.abs(x)), "sqrt": (np.sqrt, np.abs(x)),
        "leaky_relu": (lambda t: np.where(t > 0, t, 0.2 * t), x), "sub_scalar": (lambda t: t - 0.5, x),
    }
    for name, (fn, at) in fns.items():
        at64 = at.astype(np.float64)
        want = _numeric_gradient(lambda t: float(np.sum(w64 * fn(t))), at64.copy())
        v = at if name in ("abs", "log", "square", "leaky_relu", "sub_scalar") else oracle.unary_ext(name, at)
        got = oracle.unary_ext_bwd(name, v, w, 0.2 if name == "leaky_relu" else 0.5)
        assert np.allclose(got, want, rtol=2e-5, atol=2e-6), name
    # sign conventions at zero: d|x|/dx = 0 there, and the leaky slope applies to x <= 0
    z = np.array([0.0, -0.0], F)
    assert np.all(oracle.unary_ext_bwd("abs", z, np.ones(2, F)) == 0)
    assert np.all(oracle.unary_ext_bwd("leaky_relu", z, np.ones(2, F), 0.3) == F(0.3))


def _as3(x, outer, length, inner):
    return np.asarray(x, np.float64).reshape(outer, length, inner)


def test_reductions_along_an_axis_against_numpy_in_double(oracle):
    for (outer, length, inner), seed in [((1, 37, 1), 1), ((5, 9, 1), 2), ((1, 11, 6), 3), ((3, 7, 4), 4), ((2, 1, 3), 5)]:
        x = oracle.normal((outer, length, inner), 60 + seed, 3.0, 2.0)
        x3 = _as3(x, outer, length, inner)
        for kind, fn in [("sum", np.sum), ("mean", np.mean), ("max", np.max), ("min", np.min)]:
            out, index, _ = oracle.reduce_dim(kind, x, outer, length, inner)
            assert np.allclose(out, fn(x3, axis=1), rtol=1e-6, atol=1e-6), (kind, outer, length, inner)
            if kind in ("max", "min"):
                assert same_bits(out, fn(x3, axis=1).astype(F))
                want = np.argmax(x3, axis=1) if kind == "max" else np.argmin(x3, axis=1)
                assert np.array_equal(index, want)
        if length > 1:
            for ddof in (0, 1):
                out, _, mean = oracle.reduce_dim("var", x, outer, length, inner, ddof)
                assert np.allclose(out, np.var(x3, axis=1, ddof=ddof), rtol=1e-6), (ddof, outer, length, inner)
                assert np.allclose(mean, np.mean(x3, axis=1), rtol=1e-6)
                out, _, _ = oracle.reduce_dim("std", x, outer, length, inner, ddof)
                assert np.allclose(out, np.std(x3, axis=1, ddof=ddof), rtol=1e-6)


def test_reductions_closed_forms_and_first_occurrence(oracle):
    n = 101
    x = np.arange(1, n + 1, dtype=F)
    assert oracle.reduce_dim("sum", x, 1, n, 1)[0][0, 0] == n * (n + 1) / 2
    assert oracle.reduce_dim("mean", x, 1, n, 1)[0][0, 0] == (n + 1) / 2
    assert oracle.reduce_dim("var", x, 1, n, 1, 0)[0][0, 0] == F((n * n - 1) / 12)      # variance of 1..n
    assert oracle.reduce_dim("var", x, 1, n, 1, 1)[0][0, 0] == F(n * (n + 1) / 12)      # with Bessel's correction
    assert abs(oracle.reduce_dim("std", x + F(1e4), 1, n, 1, 0)[0][0, 0] - np.sqrt((n * n - 1) / 12)) < 1e-4   # shift invariant
    assert oracle.reduce_dim("var", np.full(50, 7.25, F), 1, 50, 1)[0][0, 0] == 0
    # ties: the first occurrence; NaN: only a leading one stays (a loop `if (v > m)` from element 0)
    t = np.array([1, 5, 2, 5, -3, -3], F)
    out, idx, _ = oracle.reduce_dim("max", t, 1, 6, 1)
    assert out[0, 0] == 5 and idx[0, 0] == 1
    out, idx, _ = oracle.reduce_dim("min", t, 1, 6, 1)
    assert out[0, 0] == -3 and idx[0, 0] == 4
    out, idx, _ = oracle.reduce_dim("max", np.array([1, np.nan, 3], F), 1, 3, 1)
    assert out[0, 0] == 3 and idx[0, 0] == 2
    out, idx, _ = oracle.reduce_dim("max", np.array([np.nan, 1, 3], F), 1, 3, 1)
    assert np.isnan(out[0, 0]) and idx[0, 0] == 0
    # columns of a matrix: axis 0 of [3, 2]
    m = np.array([[1, 9], [4, 2], [4, 9]], F)
    out, idx, _ = oracle.reduce_dim("max", m, 1, 3, 2)
    assert out.tolist() == [[4, 9]] and idx.tolist() == [[1, 0]]


def test_reduction_gradients_against_central_differences(oracle):
    outer, length, inner = 2, 5, 3
    x = oracle.normal((outer, length, inner), 71, 1.0, 2.0)
    w = oracle.normal((outer, inner), 72)
    w64 = w.astype(np.float64)
    fns = {"sum": lambda t: t.sum(1), "mean": lambda t: t.mean(1), "max": lambda t: t.max(1), "min": lambda t: t.min(1),
           "var": lambda t: t.var(1, ddof=1), "std": lambda t: t.std(1, ddof=1)}
    for kind, fn in fns.items():
        y, index, mean = oracle.reduce_dim(kind, x, outer, length, inner, 1)
        got = oracle.reduce_dim_bwd(kind, x, y, index, mean, w, outer, length, inner, 1)
        want = _numeric_gradient(lambda t: float(np.sum(w64 * fn(t))), x.astype(np.float64).copy())
        assert np.allclose(got, want, rtol=3e-5, atol=3e-6), kind
    # population variance (ddof 0) as well: the divisor is len - ddof
    y, index, mean = oracle.reduce_dim("var", x, outer, length, inner, 0)
    got = oracle.reduce_dim_bwd("var", x, y, index, mean, w, outer, length, inner, 0)
    want = _numeric_gradient(lambda t: float(np.sum(w64 * t.var(1, ddof=0))), x.astype(np.float64).copy())
    assert np.allclose(got, want, rtol=3e-5, atol=3e-6)


def test_log_softmax_against_double_precision_and_its_identities(oracle):
    for shape, seed in [((7, 13), 1), ((1, 50), 2), ((33, 4), 3)]:
        x = oracle.normal(shape, 80 + seed, 0, 3)
        x64 = x.astype(np.float64)
        for dim in (0, 1):
            y = oracle.log_softmax(x, dim)
            sh = x64 - x64.max(axis=dim, keepdims=True)
            want = sh - np.log(np.exp(sh).sum(axis=dim, keepdims=True))
            assert np.allclose(y, want, rtol=2e-6, atol=2e-6)
            assert np.allclose(np.exp(y.astype(np.float64)).sum(axis=dim), 1, atol=1e-5)       # exp(y) is a distribution
            assert np.allclose(np.exp(y.astype(np.float64)), oracle.softmax(x, dim), rtol=1e-5, atol=1e-8)
            # shift invariance along the axis
            assert np.allclose(oracle.log_softmax(x + F(5), dim), y, atol=3e-6)
    v = oracle.normal((9,), 90)
    assert np.allclose(oracle.log_softmax(v), oracle.log_softmax(v.reshape(1, 9), 1).reshape(9))
    x = oracle.normal((4, 6), 91)
    w = oracle.normal((4, 6), 92)
    w64 = w.astype(np.float64)
    for dim in (0, 1):
        def f(t):
            sh = t - t.max(axis=dim, keepdims=True)
            return float(np.sum(w64 * (sh - np.log(np.exp(sh).sum(axis=dim, keepdims=True)))))
        got = oracle.log_softmax_bwd(oracle.log_softmax(x, dim), w, dim)
        assert np.allclose(got, _numeric_gradient(f, x.astype(np.float64).copy()), rtol=3e-5, atol=3e-6), dim
        assert np.allclose(got.sum(axis=dim), 0, atol=2e-6)        # gradients of a normalised quantity sum to zero... times sum(w)
    

def test_broadcast_reduce_is_the_sum_over_broadcast_dimensions(oracle):
    cases = [((4, 5), (5,)), ((4, 5), (4, 1)), ((4, 5), (1,)), ((4, 5), ()), ((2, 3, 4), (3, 1)), ((2, 3, 4), (4,)),
             ((2, 3, 4), (2, 1, 4)), ((1, 5), (3, 5)), ((5,), (2, 5)), ((3, 1), (3, 4)), ((2, 1, 4), (3, 4))]
    for gshape, tshape in cases:
        g = oracle.normal(gshape, 95, 0, 2)
        if len(tshape) > g.ndim:                    # the caller reshapes a lower-rank gradient to [1, .., 1, dims] first
            g = g.reshape((1,) * (len(tshape) - g.ndim) + g.shape)
        got = oracle.broadcast_reduce(g, tshape)
        assert got is not None, (gshape, tshape)
        g64 = g.astype(np.float64)
        pad = (1,) * (g.ndim - len(tshape)) + tuple(tshape)
        axes = tuple(d for d in range(g.ndim) if pad[d] == 1 and g.shape[d] > 1)
        want = np.broadcast_to(g64.sum(axis=axes, keepdims=True), pad).reshape(tshape)
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6), (gshape, tshape)
    assert oracle.broadcast_reduce(oracle.normal((2, 6), 1), (3,)) is None

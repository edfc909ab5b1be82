"""The Tensor methods that the reference declares and never defines (include/Tensor.h:719, :824-1072),
the LReLU kernel it registers without a function (include/Ctorch_Scheduler.h:51-52) and the complete
gradient shape adjustment (src/AutoDiff.cpp:562-1049), through the C++ front-end on the device:
Tensor method -> scheduler / shim -> C ABI -> kernel, and back through the tape.  Checked against the
oracle functions (pinned by mathematics, or - the shape adjustment - against the reference)."""
import numpy as np
import pytest

from support import HostLayer, ulp_diff

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def host():
    return HostLayer()


def bits_equal(got, want, what=""):
    assert got is not None, what
    got, want = np.asarray(got, F), np.asarray(want, F)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    nan_both = np.isnan(got) & np.isnan(want)
    bad = (got.view(np.uint32) != want.view(np.uint32)) & ~nan_both
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} differ"


def test_declared_unary_methods_and_their_tape_gradients(oracle, host):
    print("case host declared unary", flush=True)
    x = oracle.normal((37, 53), 10, 0, 2)
    pos = np.abs(x) + F(0.05)
    w = oracle.normal((37, 53), 11)
    up = oracle.accumulate0(w)            # the upstream gradient the tape hands to f: 0 + 1 * w
    for name, at, p in [("abs", x, 0.0), ("exp", x, 0.0), ("log", pos, 0.0), ("sqrt", pos, 0.0), ("square", x, 0.0),
                        ("leaky_relu", x, 0.01), ("leaky_relu", x, 0.2), ("sub_scalar", x, 1.5)]:
        bits_equal(host.declared_unary(name, at, p), oracle.unary_ext(name, at, p), name)
        v = at if name in ("abs", "log", "square", "leaky_relu", "sub_scalar") else oracle.unary_ext(name, at, p)
        want = oracle.accumulate0(oracle.unary_ext_bwd(name, v, oracle.mul(np.ones_like(w), w) if False else up, p))
        bits_equal(host.grad_declared_unary(name, at, w, p), want, name + " gradient")
    got, want = host.declared_unary("tan", x), oracle.unary_ext("tan", x)
    assert ulp_diff(got, want).max() <= 2
    g = host.grad_declared_unary("tan", x, w)
    y64 = np.tan(x.astype(np.float64))
    assert np.allclose(g, (1 + y64 * y64) * w, rtol=2e-5, atol=1e-6)
    # the scheduler's LReLU column: registered (the reference registers the op without a function)
    bits_equal(host.declared_unary("lrelu_dispatch", x), oracle.unary_ext("leaky_relu", x, 0.01), "Ctorch_Scheduler::dispatch(op::LReLU)")


CASES = [((6, 7), (), False), ((6, 7), (0,), False), ((6, 7), (1,), False), ((6, 7), (1,), True), ((6, 7), (-1,), False),
         ((6, 7), (0, 1), False), ((6, 7), (0, 1), True), ((40,), (0,), False), ((40,), (), False), ((3, 4, 5), (1,), False),
         ((3, 4, 5), (1, 2), False), ((3, 4, 5), (0, 1), True), ((3, 4, 5), (0, 2), False), ((3, 4, 5), (0, 2), True),
         ((300, 130), (0,), False), ((300, 130), (1,), False), ((), (), False)]


@pytest.mark.parametrize("shape, dims, keepdim", CASES)
def test_reductions_over_dimensions(oracle, host, shape, dims, keepdim):
    print("case host reduce", shape, dims, keepdim, flush=True)
    x = oracle.normal(shape if shape else (1,), 20, 1.0, 2.0).reshape(shape)
    x64 = x.astype(np.float64)
    rank = len(shape)
    axes = tuple(sorted(d % rank for d in dims)) if dims else tuple(range(rank))
    separated = any(b != a + 1 for a, b in zip(axes, axes[1:]))
    fns = {"sum": np.sum, "mean": np.mean, "max": np.max, "min": np.min,
           "var": lambda t, axis, keepdims: np.var(t, axis=axis, keepdims=keepdims, ddof=1),
           "std": lambda t, axis, keepdims: np.std(t, axis=axis, keepdims=keepdims, ddof=1)}
    count = int(np.prod([shape[a] for a in axes])) if rank else 1
    for kind, fn in fns.items():
        if kind == "sum" and not dims and not keepdim:
            continue                                     # Tensor::sum() is the reference's own method, tested elsewhere
        got = host.reduce(kind, x, dims, keepdim)
        if kind in ("var", "std") and separated:
            assert got is None                           # refused: the dimensions must be adjacent
            continue
        if kind in ("var", "std") and count < 2:
            continue
        want = fn(x64, axis=axes if rank else None, keepdims=keepdim) if rank else fn(x64.reshape(1), axis=0, keepdims=False)
        assert got is not None, kind
        assert got.shape == np.shape(want), (kind, got.shape, np.shape(want))
        if kind in ("max", "min"):
            bits_equal(got, np.asarray(want, F), kind)
        else:
            scale = np.abs(x64).sum(axis=axes if rank else None, keepdims=keepdim) / (1 if kind == "sum" else count) if kind in ("sum", "mean") \
                else np.abs(want)
            assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30), kind
        # the tape's gradient against the oracle's arithmetic for one block of adjacent dimensions
        w = oracle.normal(np.shape(want) if np.shape(want) else (1,), 21).reshape(np.shape(want))
        g = host.grad_reduce(kind, x, w, dims, keepdim)
        assert g is not None and g.shape == x.shape
        if not separated:
            outer = int(np.prod(shape[:axes[0]])) if rank else 1
            inner = int(np.prod(shape[axes[-1] + 1:])) if rank else 1
            y, index, mean = oracle.reduce_dim(kind, x, outer, count, inner, 1)
            up = oracle.accumulate0(w)
            want_g = oracle.accumulate0(oracle.reduce_dim_bwd(kind, x, y, index, mean, up, outer, count, inner, 1)).reshape(x.shape)
            if kind in ("sum", "mean", "max", "min"):
                bits_equal(g, want_g, kind + " gradient")
            else:   # the device's mean / result differ from the oracle's in the last bits
                assert np.all(np.abs(g - want_g) <= 2e-5 * np.abs(want_g) + 1e-7 * np.abs(w).max()), kind
        else:
            def f(t, kind=kind, fn=fn):
                return float(np.sum(w.astype(np.float64) * fn(t, axis=axes, keepdims=keepdim)))
            eps = 1e-6
            num = np.zeros_like(x64)
            flat = x64.reshape(-1)
            for i in range(flat.size):
                keep = flat[i]
                flat[i] = keep + eps
                up_ = f(x64)
                flat[i] = keep - eps
                down = f(x64)
                flat[i] = keep
                num.reshape(-1)[i] = (up_ - down) / (2 * eps)
            assert np.allclose(g, num, rtol=3e-5, atol=3e-6), kind


def test_var_with_an_explicit_correction_and_error_cases(oracle, host):
    print("case host var ddof", flush=True)
    x = oracle.normal((9, 11), 30, 3.0, 1.5)
    for ddof in (0, 1, 2):
        got = host.reduce("var", x, (1,), False, ddof)
        assert np.allclose(got, x.astype(np.float64).var(axis=1, ddof=ddof), rtol=1e-5)
        got = host.reduce("std", x, (0,), True, ddof)
        assert got.shape == (1, 11) and np.allclose(got, x.astype(np.float64).std(axis=0, ddof=ddof, keepdims=True), rtol=1e-5)
    assert host.reduce("mean", x, (2,)) is None            # dim out of range: throws
    assert host.reduce("max", x, (-3,)) is None
    assert host.log_softmax(x, 2) is None


def test_log_softmax_method_and_gradient(oracle, host):
    print("case host log_softmax", flush=True)
    for shape in [(19, 31), (3, 300), (200, 12), (50,)]:
        x = oracle.normal(shape, 40, 0, 2)
        w = oracle.normal(shape, 41)
        for dim in ((0, 1, -1) if len(shape) == 2 else (0,)):
            d = dim % len(shape) if len(shape) == 2 else 1
            want = oracle.log_softmax(x, d)
            got = host.log_softmax(x, dim)
            assert got is not None and np.abs(got - want).max() <= 4e-6 * (1 + np.abs(want).max()), (shape, dim)
            gw = oracle.accumulate0(oracle.log_softmax_bwd(want, oracle.accumulate0(w), d))
            g = host.grad_log_softmax(x, dim, w)
            assert g is not None and np.abs(g - gw).max() <= 2e-5 * (np.abs(w).max() + np.abs(w).sum(axis=d if len(shape) == 2 else 0).max() * 1e-2 + 1), (shape, dim)


ADJUST = [((2, 3), (2, 3)), ((), (2, 3)), ((3,), (1, 3)), ((4,), (4, 1)), ((6,), (1, 1, 6)), ((2, 3), (1, 2, 3)), ((1,), (2, 3)),
          ((2, 3), (3,)), ((4, 5), (5,)), ((2, 3, 4), (4,)), ((2, 3, 4), (3, 4)), ((2, 3), (1,)), ((2, 3), ()), ((5, 1), (1,)),
          ((4, 1), (2,)), ((2, 6), (3,)), ((6,), (2, 2)), ((3, 5), (2,)), ((7,), (3,)), ((2, 3), (4, 3))]


@pytest.mark.parametrize("gshape, tshape", ADJUST)
def test_gradient_shape_adjustment_in_the_reference_mode(oracle, host, gshape, tshape):
    """Every branch of check_and_adjust_grad_shape, bit for bit with the oracle's restatement, which
    is pinned against the reference on exactly these shape pairs."""
    print("case host adjust (reference mode)", gshape, tshape, flush=True)
    host.set_reference_row0(True)
    try:
        for seed in range(2):
            g = oracle.normal(gshape if gshape else (1,), 900 + seed, 0, 2).reshape(gshape)
            if seed == 1:
                g.reshape(-1)[0] = -0.0
            want = oracle.adjust_grad_shape(g, tshape)
            got = host.adjust_grad_shape(g, tshape)
            bits_equal(got, want, (gshape, tshape, seed))
    finally:
        host.set_reference_row0(False)


def test_gradient_shape_adjustment_where_the_reference_leaves_its_buffer(oracle, host):
    print("case host adjust out of bounds", flush=True)
    host.set_reference_row0(True)
    try:
        g = oracle.normal((3,), 1)
        assert oracle.adjust_grad_shape(g, (2, 3)) is None
        assert host.adjust_grad_shape(g, (2, 3)) is None          # refused with an exception, nothing is read
    finally:
        host.set_reference_row0(False)
    # by default that shape pair means what the mathematics says: the gradient repeated along the new dimension
    got = host.adjust_grad_shape(g, (2, 3))
    bits_equal(got, np.stack([g, g]) + F(0), "[3] -> [2, 3]")


@pytest.mark.parametrize("gshape, tshape", [((4, 5), (5,)), ((4, 5), (4, 1)), ((4, 5), (1, 5)), ((2, 3, 4), (3, 1)), ((2, 3, 4), (4,)),
                                            ((2, 3, 4), (3, 4)), ((2, 3, 4), (2, 1, 4)), ((1, 5), (3, 5)), ((5,), (2, 5)), ((3, 1), (3, 4)),
                                            ((300, 40, 6), (40, 6)), ((4, 5), ()), ((2, 6), (3,))])
def test_gradient_shape_adjustment_by_default_is_the_sum_over_broadcast_dimensions(oracle, host, gshape, tshape):
    print("case host adjust (sum mode)", gshape, tshape, flush=True)
    g = oracle.normal(gshape, 95, 0, 2)
    got = host.adjust_grad_shape(g, tshape)
    assert got is not None
    if (gshape, tshape) == ((2, 6), (3,)):
        bits_equal(got, oracle.adjust_grad_shape(g, tshape), "shapes that do not broadcast: the reference's fold in both modes")
        return
    g64 = g.astype(np.float64)
    gp = g64.reshape((1,) * max(0, len(tshape) - g.ndim) + g.shape)
    pad = (1,) * (gp.ndim - len(tshape)) + tuple(tshape)
    axes = tuple(d for d in range(gp.ndim) if pad[d] == 1 and gp.shape[d] > 1)
    want = np.broadcast_to(gp.sum(axis=axes, keepdims=True), pad).reshape(tshape)
    scale = np.broadcast_to(np.abs(gp).sum(axis=axes, keepdims=True), pad).reshape(tshape)
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-30)


def test_dot_gradient_extension(oracle, host):
    """The reference has no gradient for Dot (src/AutoDiff.cpp:1856-1862: both operands stay 0); this
    tape has the closed form d(a.b)/da = g * b, d/db = g * a, each product rounded once."""
    print("case host dot gradient", flush=True)
    a = oracle.normal((1003,), 50)
    b = oracle.normal((1003,), 51)
    for scale in (1.0, -2.5):
        value, da, db = host.grad_dot(a, b, scale)
        assert abs(value - np.dot(a.astype(np.float64), b.astype(np.float64))) <= 1e-5 * np.abs(a * b).sum()
        g = F(scale)                                        # upstream gradient of the dot product: d(y * s)/dy = s
        bits_equal(da, oracle.accumulate0(b * g), "d/da")
        bits_equal(db, oracle.accumulate0(a * g), "d/db")

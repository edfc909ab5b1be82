"""GPU parity, through the C ABI, of the operators the reference declares on Tensor and never defines
(include/Tensor.h:719, :824-1072; LReLU of include/Ctorch_Scheduler.h:51-52) and of the complete
gradient shape adjustment (src/AutoDiff.cpp:562-1049).  The oracle functions behind them are pinned
by mathematics (tests/test_oracle_math.py) or against the reference (tests/test_oracle_vs_ref.py).

Bars: bit-exact for abs / square / sqrt / leaky_relu / a - s / exp / log (the device returns glibc's
floats) and for every gradient given the same inputs; <= 2 ulp for tan; max / min values and
positions exact; |x - y| <= 1e-5 * sum|terms| (fp64 arbiter) for sum / mean / var / std /
log_softmax."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_support as G
from support import same_bits, ulp_diff

pytestmark = pytest.mark.gpu
F = np.float32

SPECIAL = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 1e-38, 88.8, -88.8, 104.0, -104.0,
                    1.0, -1.0, 0.5, 1e-3, 1e-6, 20.0, 1.57079637, 3.14159274, 1e4, 1e7, 1e22, 119.9, 120.0, 120.1, 2.4e-4, 1.2e-4], F)


def bits_equal(got, want, what=""):
    got, want = np.asarray(got, F), np.asarray(want, F)
    nan_both = np.isnan(got) & np.isnan(want)
    bad = (got.view(np.uint32) != want.view(np.uint32)) & ~nan_both
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} differ, first at {np.argmax(bad)}: {got.reshape(-1)[np.argmax(bad)]} vs {want.reshape(-1)[np.argmax(bad)]}"


def unary(name, a, p=None):
    r = torch.empty_like(a)
    if p is None:
        G.call("ctamd_%s_f32" % name, G.ptr(a), G.ptr(r), a.numel(), G.stream())
    else:
        G.call("ctamd_%s_f32" % name, G.ptr(a), C.c_float(p), G.ptr(r), a.numel(), G.stream())
    return r


def unary_bwd(name, v, g, p=None):
    r = torch.empty_like(v)
    if p is None:
        G.call("ctamd_%s_backward_f32" % name, G.ptr(v), G.ptr(g), G.ptr(r), v.numel(), G.stream())
    else:
        G.call("ctamd_%s_backward_f32" % name, G.ptr(v), G.ptr(g), C.c_float(p), G.ptr(r), v.numel(), G.stream())
    return r


@pytest.mark.parametrize("n", [0, 1, 5, 4099, (1 << 20) + 3])
def test_declared_unary_operators(oracle, n):
    print("case declared unary n", n, flush=True)
    a = oracle.normal((n,), 11, 0, 3)
    if n >= SPECIAL.size:
        a[:SPECIAL.size] = SPECIAL
    da = G.dev(a)
    for name in ("abs", "exp", "log", "sqrt", "square"):
        bits_equal(G.host(unary(name, da)), oracle.unary_ext(name, a), name)
    bits_equal(G.host(unary("leaky_relu", da, 0.01)), oracle.unary_ext("leaky_relu", a, 0.01), "leaky_relu")
    bits_equal(G.host(unary("leaky_relu", da, -0.3)), oracle.unary_ext("leaky_relu", a, -0.3), "leaky_relu, negative slope")
    bits_equal(G.host(unary("sub_scalar", da, 1.7)), oracle.unary_ext("sub_scalar", a, 1.7), "a - s")
    got, want = G.host(unary("tan", da)), oracle.unary_ext("tan", a)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    if ok.any():
        d = ulp_diff(got[ok], want[ok])
        print(f"tan: max ulp {d.max()}, exact {float((d == 0).mean()):.4f}")
        assert d.max() <= 2
        assert np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))


def test_log_and_exp_bit_identical_over_a_sweep_of_all_floats(oracle):
    print("case log exp sweep", flush=True)
    u = np.arange(0, 1 << 32, 509, dtype=np.uint64).astype(np.uint32)
    a = u.view(F)
    da = G.dev(a)
    with np.errstate(all="ignore"):
        bits_equal(G.host(unary("log", da)), oracle.unary_ext("log", a), "log")
        bits_equal(G.host(unary("exp", da)), oracle.unary_ext("exp", a), "exp")
        bits_equal(G.host(unary("sqrt", da)), oracle.unary_ext("sqrt", a), "sqrt")
        got, want = G.host(unary("tan", da)), oracle.unary_ext("tan", a)
    ok = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    d = ulp_diff(got[ok], want[ok])
    print(f"tan over {ok.sum()} floats: max ulp {d.max()}, exact {float((d == 0).mean()):.4f}")
    assert d.max() <= 2


def test_declared_unary_gradients_bit_exact(oracle):
    print("case declared unary gradients", flush=True)
    x = np.concatenate([oracle.normal((70001,), 12, 0, 2), SPECIAL])
    g = np.concatenate([oracle.normal((70001,), 13, 0, 1), SPECIAL[::-1]])
    dx, dg = G.dev(x), G.dev(g)
    for name in ("abs", "sqrt", "square", "tan"):
        bits_equal(G.host(unary_bwd(name, dx, dg)), oracle.unary_ext_bwd(name, x, g), name)
    for slope in (0.01, 0.25):
        bits_equal(G.host(unary_bwd("leaky_relu", dx, dg, slope)), oracle.unary_ext_bwd("leaky_relu", x, g, slope), "leaky_relu")
    # exp: y * g and log: g / x are the Mul and Div kernels
    bits_equal(G.host(G.binary("mul", dx, dg)), oracle.unary_ext_bwd("exp", x, g), "exp gradient")
    bits_equal(G.host(G.binary("div", dg, dx)), oracle.unary_ext_bwd("log", x, g), "log gradient")


# ------------------------------------------------------------------------- reductions along an axis
KINDS = ["sum", "mean", "max", "min", "var", "std"]
CODE = {k: i for i, k in enumerate(KINDS)}


def reduce_dim(kind, x, outer, length, inner, ddof=1):
    out = torch.full((outer, inner), float("nan"), device=G.DEV)
    index = torch.full((outer, inner), -7, dtype=torch.int32, device=G.DEV)
    mean = torch.full((outer, inner), float("nan"), device=G.DEV)
    G.call("ctamd_reduce_dim_f32", CODE[kind], G.ptr(x), G.ptr(out), G.ptr(index), G.ptr(mean), outer, length, inner, ddof, G.stream())
    return G.host(out), index.cpu().numpy(), G.host(mean)


def reduce_dim_bwd(kind, x, y, index, mean, g, outer, length, inner, ddof=1):
    dx = torch.full((outer * length * inner,), float("nan"), device=G.DEV)
    G.call("ctamd_reduce_dim_backward_f32", CODE[kind], G.ptr(x), G.ptr(y), G.ptr(index), G.ptr(mean), G.ptr(g), G.ptr(dx),
           outer, length, inner, ddof, G.stream())
    return G.host(dx)


SHAPES = [(1, 1, 1), (1, 37, 1), (1, 4099, 1), (1, (1 << 20) + 5, 1), (7, 33, 1), (300, 1000, 1), (5, 8192, 1), (2048, 64, 1),
          (1, 9, 6), (1, 700, 10), (1, 4096, 256), (1, 130, 4100), (3, 17, 5), (2, 300, 64), (1, 1, 9), (4, 1, 1),
          (70000, 6, 8), (66000, 7, 3)]          # more slabs than a launch grid's third dimension holds


@pytest.mark.parametrize("shape", SHAPES)
def test_reductions_along_an_axis(oracle, shape):
    outer, length, inner = shape
    print("case reduce_dim", shape, flush=True)
    x = oracle.normal((outer, length, inner), 21, 2.0, 3.0)
    if length > 5:
        x[0, 3, 0] = x[0, 1, 0] = x.max() + 1          # a tie for the maximum: the first one counts
        x[-1, 2, -1] = x[-1, 4, -1] = x.min() - 1
    dx = G.dev(x)
    x64 = x.astype(np.float64)
    for kind in KINDS:
        for ddof in ((0, 1) if kind in ("var", "std") else (1,)):
            if kind in ("var", "std") and length - ddof <= 0:
                continue
            got, gi, gm = reduce_dim(kind, dx, outer, length, inner, ddof)
            want, wi, wm = oracle.reduce_dim(kind, x, outer, length, inner, ddof)
            if kind in ("max", "min"):
                bits_equal(got, want, kind)
                assert np.array_equal(gi, wi), kind
            elif kind in ("sum", "mean"):
                scale = np.abs(x64).sum(axis=1) / (1 if kind == "sum" else length)
                exact = x64.sum(axis=1) / (1 if kind == "sum" else length)
                assert np.all(np.abs(got - exact) <= 1e-5 * scale + 1e-30), kind
                assert np.all(np.abs(got - want) <= 2e-5 * scale + 1e-30), kind
            else:
                exact = x64.var(axis=1, ddof=ddof)
                exact = exact if kind == "var" else np.sqrt(exact)
                assert np.all(np.abs(got - exact) <= 1e-5 * np.abs(exact) + 1e-30), (kind, ddof)
                assert np.all(np.abs(got - want) <= 2e-5 * np.abs(exact) + 1e-30), (kind, ddof)
                assert np.all(np.abs(gm - x64.mean(axis=1)) <= 1e-6 * np.abs(x64).mean(axis=1) + 1e-30)


@pytest.mark.parametrize("shape", [(1, 37, 1), (7, 33, 1), (3, 5000, 1), (1, 9, 6), (1, 700, 10), (1, 130, 4100), (3, 17, 5), (2, 300, 64), (1, 70001, 1),
                                   (70000, 6, 8)])
def test_reduction_gradients_bit_exact(oracle, shape):
    outer, length, inner = shape
    print("case reduce_dim backward", shape, flush=True)
    x = oracle.normal((outer, length, inner), 22, 1.0, 2.0)
    g = oracle.normal((outer, inner), 23)
    for kind in KINDS:
        y, index, mean = oracle.reduce_dim(kind, x, outer, length, inner, 1)
        want = oracle.reduce_dim_bwd(kind, x, y, index, mean, g, outer, length, inner, 1)
        got = reduce_dim_bwd(kind, G.dev(x), G.dev(y), torch.from_numpy(index).to(G.DEV), G.dev(mean), G.dev(g), outer, length, inner, 1)
        bits_equal(got.reshape(want.shape), want, kind)


def test_reductions_edge_cases(oracle):
    print("case reduce_dim edges", flush=True)
    l = G.lib()
    # NaN stays only in front; all -inf keeps element 0
    for row, val, pos in [([1, np.nan, 3], 3, 2), ([np.nan, 1, 3], np.nan, 0), ([-np.inf] * 3, -np.inf, 0), ([2, 2, 2], 2, 0)]:
        got, gi, _ = reduce_dim("max", G.dev(np.array(row, F)), 1, 3, 1)
        assert (np.isnan(val) and np.isnan(got[0, 0])) or got[0, 0] == val
        assert gi[0, 0] == pos, row
    got, gi, _ = reduce_dim("min", G.dev(np.array([np.inf, np.inf], F)), 1, 2, 1)
    assert got[0, 0] == np.inf and gi[0, 0] == 0
    # a constant run has variance exactly 0, also far from the origin
    got, _, gm = reduce_dim("var", G.dev(np.full(5000, 1234.5, F)), 1, 5000, 1)
    assert got[0, 0] == 0 and gm[0, 0] == F(1234.5)
    # data far from the origin: the shift keeps the variance accurate
    x = (oracle.normal((1, 100000, 1), 31, 0, 1).astype(np.float64) + 1e4).astype(F)
    got, _, _ = reduce_dim("std", G.dev(x), 1, 100000, 1, 0)
    assert abs(got[0, 0] - x.astype(np.float64).std()) <= 1e-5 * x.astype(np.float64).std()
    # unaligned input (a view one element off a 16-byte boundary) and a row length that is no multiple of four
    base = G.dev(oracle.normal((7 * 33 + 1,), 32))
    got, gi, _ = reduce_dim("max", base[1:], 7, 33, 1)
    want, wi, _ = oracle.reduce_dim("max", G.host(base)[1:], 7, 33, 1)
    bits_equal(got, want)
    assert np.array_equal(gi, wi)
    # argument checks: nothing is launched
    out = torch.zeros(1, device=G.DEV)
    assert l.ctamd_reduce_dim_f32(9, G.ptr(base), G.ptr(out), None, None, 1, 4, 1, 1, G.stream()) == -1
    assert l.ctamd_reduce_dim_f32(0, G.ptr(base), G.ptr(out), None, None, 1, 0, 1, 1, G.stream()) == -1      # empty axis
    assert l.ctamd_reduce_dim_f32(0, None, None, None, None, 0, 4, 1, 1, G.stream()) == 0                        # no results
    assert l.ctamd_reduce_dim_backward_f32(2, G.ptr(base), G.ptr(out), None, None, G.ptr(out), G.ptr(base), 1, 4, 1, 1, G.stream()) == -1


# -------------------------------------------------------------------------------------- log_softmax
def log_softmax(x, dim):
    y = torch.empty_like(x)
    rows, cols = (1, x.numel()) if x.dim() == 1 else x.shape
    name = "ctamd_log_softmax_rows_f32" if (x.dim() == 1 or dim == 1) else "ctamd_log_softmax_cols_f32"
    G.call(name, G.ptr(x), G.ptr(y), rows, cols, G.stream())
    return y


def log_softmax_bwd(y, g, dim):
    dx = torch.empty_like(y)
    rows, cols = (1, y.numel()) if y.dim() == 1 else y.shape
    name = "ctamd_log_softmax_backward_rows_f32" if (y.dim() == 1 or dim == 1) else "ctamd_log_softmax_backward_cols_f32"
    G.call(name, G.ptr(y), G.ptr(g), G.ptr(dx), rows, cols, G.stream())
    return dx


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (33, 47), (64, 130), (5, 1000), (256, 10), (7, 2048), (3, 4099), (9, 32000), (2, 40000),
                                   (2, 70001), (300, 64), (1000, 260), (3, 65536), (2, 49156)])
def test_log_softmax_and_its_gradient(oracle, shape):
    print("case log_softmax", shape, flush=True)
    x = oracle.normal(shape, 41, 0, 2.5)
    w = oracle.normal(shape, 42)
    x64 = x.astype(np.float64)
    for dim in (1, 0):
        if dim == 0 and shape[1] > 5000:
            continue
        y = G.host(log_softmax(G.dev(x), dim))
        sh = x64 - x64.max(axis=dim, keepdims=True)
        lse = np.log(np.exp(sh).sum(axis=dim, keepdims=True))
        exact = sh - lse
        # each element is a difference of two terms: the bar is relative to their sizes, plus the
        # rounding of the fp32 sum itself (a sum of 1 + 1e-9 is 1 in fp32, and its logarithm 0)
        bound = 1e-5 * (np.abs(sh) + np.abs(lse)) + 2e-7
        assert np.all(np.abs(y - exact) <= bound), dim
        want = oracle.log_softmax(x, dim)
        assert np.all(np.abs(y - want) <= 2 * bound), dim
        if shape[1 if dim == 1 else 0] < 128 or (dim == 1 and shape[1] < 2048):
            # short runs use the bit-exact exponential; only the order of the sum differs from the oracle's
            assert np.abs(y - want).max() <= 4e-7 * (1 + np.abs(want).max()), dim
        # gradient, from the oracle's y so that both sides see the same inputs
        got = G.host(log_softmax_bwd(G.dev(want), G.dev(w), dim))
        dwant = oracle.log_softmax_bwd(want, w, dim)
        w64 = w.astype(np.float64)
        d64 = w64 - np.exp(want.astype(np.float64)) * w64.sum(axis=dim, keepdims=True)
        gb = 1e-5 * (np.abs(w64) + np.exp(want.astype(np.float64)) * np.abs(w64).sum(axis=dim, keepdims=True)) + 1e-30
        assert np.all(np.abs(got - d64) <= gb), dim
        assert np.all(np.abs(got - dwant) <= 2 * gb), dim


# -------------------------------------------------------------------- gradient shape adjustment
def test_fold_of_a_gradient_that_does_not_broadcast(oracle):
    print("case fold_mod", flush=True)
    for gn, tn in [(12, 3), (6, 4), (15, 2), (7, 3), (6, 12), (100003, 17), (5, 5)]:
        g = oracle.normal((gn,), 51, 0, 2)
        out = torch.full((tn,), float("nan"), device=G.DEV)
        G.call("ctamd_fold_mod_f32", G.ptr(G.dev(g)), G.ptr(out), gn, tn, G.stream())
        # out[i] = g[i] + g[i + tn] + ... in that order, from 0, every step rounded to fp32
        want = np.zeros(tn, F)
        for i in range(tn):
            s = F(0)
            for v in g[i::tn]:
                s = F(s + v)
            want[i] = s
        bits_equal(G.host(out), want, (gn, tn))
    g = oracle.normal((2, 6), 52)
    want = oracle.adjust_grad_shape(g, (3,))            # takes the modulo branch (6 vs 3 do not broadcast)
    out = torch.empty(3, device=G.DEV)
    G.call("ctamd_fold_mod_f32", G.ptr(G.dev(g)), G.ptr(out), 12, 3, G.stream())
    bits_equal(G.host(out), want)


def test_broadcast_reduce_general_shapes(oracle):
    print("case broadcast_reduce", flush=True)
    cases = [((4, 5), (1, 5)), ((4, 5), (4, 1)), ((4, 5), (1, 1)), ((2, 3, 4), (1, 3, 1)), ((2, 3, 4), (1, 1, 4)), ((2, 3, 4), (2, 1, 4)),
             ((1, 5), (3, 5)), ((3, 1), (3, 4)), ((2, 1, 4), (1, 3, 4)), ((300, 7, 9), (1, 7, 1)), ((6,), (6,)), ((), ())]
    for gshape, tshape in cases:
        g = oracle.normal(gshape if gshape else (1,), 61, 0, 2).reshape(gshape)
        want = oracle.broadcast_reduce(g, tshape)
        out = torch.full(tshape if tshape else (1,), float("nan"), device=G.DEV)
        rank = len(gshape)
        gs = (C.c_size_t * max(1, rank))(*gshape)
        ts = (C.c_size_t * max(1, rank))(*tshape)
        G.call("ctamd_broadcast_reduce_f32", G.ptr(G.dev(g.reshape(-1) if gshape else g.reshape(1))), gs, ts, rank, G.ptr(out), G.stream())
        g64 = g.astype(np.float64)
        axes = tuple(d for d in range(rank) if tshape[d] == 1 and gshape[d] > 1)
        exact = np.broadcast_to(g64.sum(axis=axes, keepdims=True), tshape) if rank else g64
        scale = np.broadcast_to(np.abs(g64).sum(axis=axes, keepdims=True), tshape) if rank else np.abs(g64)
        got = G.host(out).reshape(tshape)
        assert np.all(np.abs(got - exact) <= 1e-6 * scale + 1e-30), (gshape, tshape)
        assert np.all(np.abs(got - want.reshape(tshape)) <= 2e-6 * scale + 1e-30)
    l = G.lib()
    bad_g, bad_t = (C.c_size_t * 2)(2, 6), (C.c_size_t * 2)(1, 3)
    assert l.ctamd_broadcast_reduce_f32(G.ptr(G.dev(np.zeros(12, F))), bad_g, bad_t, 2, G.ptr(torch.zeros(3, device=G.DEV)), G.stream()) == -1

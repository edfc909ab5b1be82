"""Tensors that are not fp32 (double, int32, int64, bool) through the C ABI: conversion from fp32,
fill, tensor (+ * /) float and the gradient accumulation byte for byte against the CPU oracle and the
reference's golden vectors.  The double softmax (its exponential is glibc's bit for bit - cta_exp64, checked on the
host in tests/native/exp64_check.c; its sums are trees of sequential partial sums, and the column form
scales chunk sums to the column maximum): within 4 + sqrt(len) units in the last place of an extended-
precision arbiter and within 4 + 2 sqrt(len) of the reference, a sequential sum of len terms carrying
about sqrt(len) roundings; through its invariants at a large size."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_support as G
from support import NP_DTYPE, typed_cases

pytestmark = pytest.mark.gpu

SOFTMAX_ULP = 4


def dev_typed(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, NP_DTYPE[dtype])).to(G.DEV)


def same_bytes(t, want):
    got = G.host(t)
    return got.shape == want.shape and np.array_equal(got.view(np.uint8), np.ascontiguousarray(want).view(np.uint8))


def run_steps(a, dtype, steps):
    """The device counterpart of Oracle.typed: conversion, then each step through its entry point."""
    t = G.cast_from_f32(G.dev(a), dtype)
    for what, s in steps:
        if what <= 2:
            t = G.scalar_op_typed(t, dtype, what, s)
        elif what in (3, 4):
            t = G.fill_typed(dtype, float(what == 4), t.numel()).reshape(t.shape)
        else:
            t = G.softmax_f64(t, int(s))
    return t


def close_in_ulp(got, want, ulp):
    return np.all(np.abs(got - want) <= ulp * np.spacing(np.abs(want)))


def softmax_arbiter(x, axis):
    """exp, sum and quotient in extended precision, of the differences x - max rounded to double as every
    implementation rounds them (that rounding alone moves exp by |x - max| / 2 units in the last place)."""
    d = np.asarray(x - x.max(axis, keepdims=True), np.longdouble)
    e = np.exp(d)
    return (e / e.sum(axis, keepdims=True)).astype(np.float64)


def check_softmax(got, want, x, axis):
    assert close_in_ulp(got, softmax_arbiter(x, axis), SOFTMAX_ULP + np.sqrt(x.shape[axis]))   # partial sums are sequential
    assert close_in_ulp(got, want, SOFTMAX_ULP + 2 * np.sqrt(x.shape[axis]))


def test_against_the_reference_vectors(oracle, golden):
    g = golden("typed")
    for name, a, dt, steps in typed_cases(oracle):
        print("case typed", name, flush=True)
        got = run_steps(a, dt, steps)
        if name.startswith("softmax"):
            x = oracle.typed(a, dt, steps[:-1])
            check_softmax(G.host(got), g[name], x, 0 if x.ndim == 1 else int(steps[-1][1]))
        else:
            assert same_bytes(got, g[name]), name


@pytest.mark.parametrize("n", [0, 1, 3, 5, 1023, 4099, (1 << 20) + 7])
def test_sizes_with_tails(oracle, n):
    """Every size class of the 16-byte vector loop: nothing, less than a vector, whole blocks plus a tail."""
    print("case typed sizes", n, flush=True)
    x = oracle.normal((n,), 81, 0, 5000) if n else np.zeros(0, np.float32)
    for dt in (1, 2, 3, 4):
        c = G.cast_from_f32(G.dev(x), dt)
        want = oracle.cast_from_f32(x, dt)
        assert same_bytes(c, want), (dt, "cast")
        assert same_bytes(G.fill_typed(dt, 1.0, n), np.ones(n, NP_DTYPE[dt])), (dt, "ones")
        assert same_bytes(G.fill_typed(dt, 0.0, n), np.zeros(n, NP_DTYPE[dt])), (dt, "zero")
        if dt == 4:
            continue
        for op, s in ((0, -12345.6), (1, 77777.7), (2, -3.5)):
            assert same_bytes(G.scalar_op_typed(c, dt, op, s), oracle.scalar_op_typed(want, dt, op, s)), (dt, op)
        other = oracle.cast_from_f32(oracle.normal((n,), 82, 0, 2e9) if n else x, dt)
        acc = G.accumulate_typed(c.clone(), dev_typed(other, dt), dt)
        assert same_bytes(acc, oracle.accumulate_typed(want, other, dt)), (dt, "accumulate")


def test_full_range_integers(oracle):
    """Sums and products that wrap, the most negative integer over -1."""
    rng = np.random.default_rng(9)
    for dt, t in ((2, np.int32), (3, np.int64)):
        info = np.iinfo(t)
        x = rng.integers(info.min, info.max, 100003, dtype=t)
        x[:3] = (info.min, info.max, -1)
        y = rng.integers(info.min, info.max, 100003, dtype=t)
        dx = dev_typed(x, dt)
        for op, s in ((0, 2e9), (1, 65537.0), (1, -3.0), (2, -1.0), (2, 7.0), (2, -2e9)):
            assert same_bytes(G.scalar_op_typed(dx, dt, op, s), oracle.scalar_op_typed(x, dt, op, s)), (dt, op, s)
        assert same_bytes(G.accumulate_typed(dx.clone(), dev_typed(y, dt), dt), oracle.accumulate_typed(x, y, dt)), dt


def test_refusals():
    x = torch.zeros(8, dtype=torch.int32, device=G.DEV)
    r = torch.empty_like(x)
    lib = G.lib()
    s = G.stream()
    assert lib.ctamd_scalar_op_typed(G.ptr(x), G.ptr(r), G.DT_I32, 2, C.c_float(0.5), 8, s) < 0     # integer 0 divisor
    assert lib.ctamd_scalar_op_typed(G.ptr(x), G.ptr(r), G.DT_I64, 2, C.c_float(-0.9), 8, s) < 0
    assert lib.ctamd_scalar_op_typed(G.ptr(x), G.ptr(r), G.DT_BOOL, 0, C.c_float(1), 8, s) < 0       # no arithmetic on bool
    assert lib.ctamd_scalar_op_typed(G.ptr(x), G.ptr(r), G.DT_I32, 3, C.c_float(1), 8, s) < 0        # bad op
    assert lib.ctamd_cast_from_f32(G.ptr(x), G.ptr(r), 7, 8, s) < 0
    assert lib.ctamd_fill_typed(G.ptr(r), 9, C.c_double(0), 8, s) < 0
    assert lib.ctamd_accumulate_typed(G.ptr(r), G.ptr(x), G.DT_BOOL, 8, s) < 0
    d = torch.zeros(8, dtype=torch.float64, device=G.DEV)
    assert lib.ctamd_softmax_f64(G.ptr(d), G.ptr(d), 2, 4, 2, s) < 0
    assert lib.ctamd_scalar_op_typed(G.ptr(d), G.ptr(d), G.DT_F64, 2, C.c_float(0.5), 8, s) == 0     # doubles divide by 0.5


@pytest.mark.parametrize("shape,dim", [((1, 1), 1), ((3, 7), 0), ((3, 7), 1), ((300, 64), 1), ((64, 300), 0), ((17, 5000), 1),
                                        ((2000, 33), 0), ((4096,), 0),
                                        # every register-resident row shape, the streaming one past it, odd lengths
                                        ((9, 66), 1), ((8, 400), 1), ((8, 1000), 1), ((5, 2000), 1), ((4, 4000), 1), ((3, 8192), 1),
                                        ((2, 8194), 1), ((3, 1001), 1),
                                        # column chunks: several chunks, two columns per lane and one
                                        ((1000, 64), 0), ((8192, 130), 0), ((8192, 131), 0), ((100000, 2), 0)])
def test_double_softmax(oracle, shape, dim):
    print("case softmax f64", shape, dim, flush=True)
    rng = np.random.default_rng(shape[0] * 7 + dim)
    x = rng.standard_normal(shape) * 4.0 + 720.0    # exp(x) itself would overflow
    got = G.host(G.softmax_f64(dev_typed(x, 1), dim))
    axis = 0 if len(shape) == 1 else dim
    check_softmax(got, oracle.softmax_f64(x, dim), x, axis)
    assert np.all(np.abs(got.sum(axis) - 1.0) <= 1e-13)


def test_double_softmax_large_rows_by_its_invariants():
    rows, cols = 4096, 8192
    x = torch.randn(rows, cols, dtype=torch.float64, device=G.DEV, generator=torch.Generator(G.DEV).manual_seed(3))
    y = G.softmax_f64(x, 1)
    assert torch.all((y.sum(1) - 1.0).abs() <= 1e-12)
    # softmax(x + c) = softmax(x); log y - x is constant along a row
    shifted = G.softmax_f64(x + 3.0, 1)
    assert torch.all((shifted - y).abs() <= 1e-14 + 1e-13 * y)
    spread = (y.log() - x)
    assert torch.all((spread - spread[:, :1]).abs() <= 1e-10)

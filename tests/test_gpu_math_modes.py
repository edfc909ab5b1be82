"""The two ways the softmax family evaluates exp(x - max) / sum (ctamd_set_math_mode): single
precision within 2 ulp of expf with a multiplication by 1 / sum (the default), or glibc's expf bit for
bit with the exactly rounded quotient (what the reference computes, src/Tensor.cpp:1713-1727,
src/AutoDiff.cpp:1546-1574).  Bars: the exponential itself <= 2 ulp against the oracle's expf over a
sweep of its whole argument range (histogram printed); every softmax output and every cross-entropy
gradient element RELATIVE to its own size (not to the row), 1e-5; row sums 1e-5."""
import numpy as np
import pytest
import torch

import gpu_support as G
from support import ulp_diff

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(params=["fast", "exact"])
def mode(request):
    prev = G.set_math_mode(G.MATH_FAST if request.param == "fast" else G.MATH_EXACT)
    yield request.param
    G.set_math_mode(prev)


def histogram(d):
    return {int(k): int((d == k).sum()) for k in np.unique(d)}


def test_the_single_precision_exponential_alone_is_within_2_ulp(oracle):
    """ctamd_cross_entropy_backward_index_stats_f32 with statistics (max 0, sum 1), upstream gradient 1
    and the class index on a column that is not looked at returns 0 + exp(x) for every other column:
    the exponential of the fast mode, bare."""
    print("case fast exponential sweep", flush=True)
    prev = G.set_math_mode(G.MATH_FAST)
    try:
        # every 97th float of [-104, -2^-20] plus the neighbourhood of zero, 2048 columns per row
        lo, hi = np.array([-104.0, -2.0 ** -20], F).view(np.uint32)
        u = np.arange(int(hi), int(lo), 97, dtype=np.uint32)
        x = np.concatenate([u.view(F), -np.logspace(-30, -6, 4001).astype(F), np.zeros(3, F)])
        cols = 2048
        rows = x.size // cols
        x = x[:rows * cols].reshape(rows, cols)
        x[:, 0] = 0.0                                   # the class column: excluded below
        stats = np.tile(np.array([0.0, 1.0], F), (rows, 1))
        dx = torch.empty((rows, cols), device=G.DEV)
        tx, ti, ts, tg = G.dev(x), G.dev(np.zeros(rows, F)), G.dev(stats), G.dev(np.ones(1, F))    # (kept alive across the call)
        G.call("ctamd_cross_entropy_backward_index_stats_f32", G.ptr(tx), G.ptr(ti), G.ptr(ts), G.ptr(tg), G.ptr(dx), rows, cols, G.stream())
        got = G.host(dx)[:, 1:].reshape(-1)
        arg = x[:, 1:].reshape(-1)
        want = oracle.unary_ext("exp", arg)
        normal = want >= F(2.0 ** -126)
        d = ulp_diff(got[normal], want[normal])
        print(f"exp, {normal.sum()} arguments with normal results: ulp histogram {histogram(d)}")
        assert d.max() <= 2
        # results below the normal range: flushed towards zero, never above the true value's neighbourhood
        assert np.all(got[~normal] >= 0) and np.all(got[~normal] <= want[~normal] * F(1.0001) + F(1e-45))
    finally:
        G.set_math_mode(prev)


@pytest.mark.parametrize("shape", [(7, 13), (64, 1000), (33, 2048), (16, 32000), (5, 40000), (3, 70004), (300, 64), (2000, 96), (3, 65536), (2, 49156)])
def test_softmax_elements_relative_to_their_own_size(oracle, mode, shape):
    print("case softmax relative", mode, shape, flush=True)
    x = oracle.normal(shape, 61, 0, 4.0)
    x64 = x.astype(np.float64)
    for dim in (1, 0):
        if dim == 0 and shape[1] > 5000:
            continue
        # x - max is an fp32 subtraction in the reference's formula (src/Tensor.cpp:1722) and here: it is part
        # of the definition (for x - max ~ -20 it rounds by 1e-6, i.e. 16 ulp of the exponential), everything
        # after it in double
        e = np.exp((x - x.max(axis=dim, keepdims=True)).astype(np.float64))
        exact = e / e.sum(axis=dim, keepdims=True)
        got = G.host(G.softmax(G.dev(x), dim))
        seen = exact >= 1e-36                           # below: subnormal results, flushed in the fast mode
        rel = np.abs(got[seen] - exact[seen]) / exact[seen]
        # in units in the last place of the correctly rounded result (the double-precision one, rounded)
        d = ulp_diff(got[seen], exact[seen].astype(F))
        print(f"  dim {dim}: max relative error {rel.max():.2e}; ulp histogram against the rounded fp64 softmax {histogram(np.minimum(d, 9))} (9 = more)")
        assert rel.max() <= 1e-5, (mode, dim)
        assert np.all(np.abs(got.astype(np.float64).sum(axis=dim) - 1) <= 1e-5)
        # exp within 0.5 / 2 ulp, the quotient within 0.5 / 1.5, the tree sum of the row within a few more
        # (a matrix of fewer than 128 rows has its columns summed one row after the other, as the reference
        # does, in both modes: that order's own rounding is allowed for)
        slack = np.sqrt(shape[0]) if dim == 0 and shape[0] < 128 else 0
        assert d.max() <= (6 if mode == "exact" else 10) + slack, (mode, dim, d.max())
        assert np.all(got[~seen] <= 2e-36)
        # the oracle (the reference's arithmetic: a sequential fp32 row sum) is itself further from the
        # exact result than either mode; both stay inside the reduction bar around it
        want = oracle.softmax(x, dim)
        assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) * max(1.0, np.sqrt(shape[dim]) / 8) + 1e-37), (mode, dim)


@pytest.mark.parametrize("shape", [(19, 31), (64, 2048), (16, 32000), (4, 50000), (200, 1000), (2, 65536), (2, 49156)])
def test_cross_entropy_gradient_elements_relative_to_their_own_size(oracle, mode, shape):
    """dlogits = softmax - onehot for class-index targets: every element off the class column is a
    probability, possibly tiny, and is held to 1e-5 of ITSELF; the class column (p - 1) to 1e-5 of
    p + 1.  All four ways the gradient is formed."""
    print("case cross entropy gradient relative", mode, shape, flush=True)
    rows, cols = shape
    x = oracle.normal(shape, 71, 0, 2.0)
    idx = oracle.ints((rows,), 72, cols)
    e = np.exp((x - x.max(axis=1, keepdims=True)).astype(np.float64))      # the fp32 subtraction is part of the formula
    p = e / e.sum(axis=1, keepdims=True)
    onehot = np.zeros(shape)
    onehot[np.arange(rows), idx.astype(int)] = 1
    exact = p - onehot
    bound = 1e-5 * (p + onehot) + 1e-37
    dx, di, g1 = G.dev(x), G.dev(idx), G.dev(np.ones(1, F))
    results = {"recomputing": G.host(G.ce_bwd(dx, di, g1, True))}
    oh = G.dev(onehot.astype(F))
    results["one-hot targets"] = G.host(G.ce_bwd(dx, oh, g1, False))
    if cols <= 32768:
        loss, status, fused = G.ce_index_fused(dx, di)
        assert status == 0
        results["one pass"] = G.host(fused)
    out = torch.empty(1, device=G.DEV)
    status = torch.zeros(1, dtype=torch.int32, device=G.DEV)
    stats = torch.empty((rows, 2), device=G.DEV)
    G.call("ctamd_cross_entropy_index_stats_f32", G.ptr(dx), G.ptr(di), G.ptr(out), G.ptr(status), G.ptr(stats), rows, cols, G.stream())
    r = torch.empty_like(dx)
    G.call("ctamd_cross_entropy_backward_index_stats_f32", G.ptr(dx), G.ptr(di), G.ptr(stats), G.ptr(g1), G.ptr(r), rows, cols, G.stream())
    results["from forward statistics"] = G.host(r)
    for name, got in results.items():
        err = np.abs(got - exact)
        worst = (err / (p + onehot + 1e-300)).max()
        print(f"  {name}: max error relative to the element {worst:.2e}")
        assert np.all(err <= bound), (mode, name, worst)
    want_loss = float(-np.log(p[np.arange(rows), idx.astype(int)]).sum())
    assert abs(float(G.host(out)[0]) - want_loss) <= 1e-5 * want_loss


def test_mode_switch_is_checked_and_restored():
    l = G.lib()
    assert l.ctamd_math_mode() == G.MATH_FAST
    assert l.ctamd_set_math_mode(7) == -1 and l.ctamd_math_mode() == G.MATH_FAST
    assert G.set_math_mode(G.MATH_EXACT) == G.MATH_FAST and l.ctamd_math_mode() == G.MATH_EXACT
    G.set_math_mode(G.MATH_FAST)

"""Parity of the HIP path with the CPU oracle, through the C ABI, on the same seeded inputs.

Bars: bit-exact for Add/Sub/Mul/Div/Neg/ReLU, their broadcast and scalar forms and the
gradient multiplies; <= 2 ulp for Sin/Cos/Tanh/Sigmoid and their gradients (the device routines
are built to return glibc's floats, so the golden vectors written from the real reference are
also required to match to <= 2 ulp, and the fraction of exact matches is printed);
|x - y| <= 1e-5 * sum|terms| for reductions, MatMul, softmax and cross entropy, with fp64 as the
arbiter."""
import ctypes as C

import numpy as np
import pytest
import torch

import gpu_support as G
from support import (ADD, COS, DIV, EX, MUL, NEG, RELU, SIGMOID, SIN, SUB, TANH, f32, same_bits, ulp_diff)

pytestmark = pytest.mark.gpu

F = np.float32
BIN = [("add", ADD), ("sub", SUB), ("mul", MUL), ("div", DIV)]
SPECIAL = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 1e-38, -1e-38,
                    88.8, -88.8, 100.0, -100.0, 1.0, -1.0, 0.5, -0.5, 1e-3, -1e-3, 1e-6, 20.0, -20.0,
                    3.14159274, 1.57079637, 6.28318548, 1e4, -1e4, 1e7, 1e22, 87.3, -87.3, 103.9, 200.0, -200.0,
                    119.9, 120.0, 120.1, 0.74, 0.75, 0.76, 2.4e-4, 2.5e-4], F)


def bits_equal(got, want, what=""):
    got, want = np.asarray(got, F), np.asarray(want, F)
    nan_both = np.isnan(got) & np.isnan(want)
    bad = (got.view(np.uint32) != want.view(np.uint32)) & ~nan_both
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} elements differ, first at {np.argmax(bad)}"


def ulp_close(got, want, max_ulp, what=""):
    got, want = np.asarray(got, F), np.asarray(want, F)
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{what}: NaN pattern differs"
    ok = ~np.isnan(want)
    d = ulp_diff(got[ok], want[ok])
    exact = float((d == 0).mean()) if d.size else 1.0
    print(f"{what}: max ulp {d.max() if d.size else 0}, exact {exact:.6f}")
    assert d.size == 0 or d.max() <= max_ulp, f"{what}: max ulp {d.max()}"


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 1023, 4099, (1 << 20) + 3])
def test_binary_same_shape_bit_exact(oracle, n):
    print("case binary n", n, flush=True)
    a = np.concatenate([oracle.normal((n,), 1, 0, 3)])
    b = np.concatenate([oracle.normal((n,), 2, 0, 3)])
    if n >= SPECIAL.size:
        a[:SPECIAL.size] = SPECIAL
        b[:SPECIAL.size] = SPECIAL[::-1]
    da, db = G.dev(a), G.dev(b)
    for name, code in BIN:
        bits_equal(G.host(G.binary(name, da, db)), oracle.binary(code, a, b), name)


@pytest.mark.parametrize("n", [(6 << 20) + 8, (1 << 24) - 4, (1 << 24) + 4])
def test_large_streams_take_every_access_hint_variant_bit_exact(oracle, n):
    """Above 64 MiB of operands + result the loads carry the streaming hint, and above 64 MiB of
    result the stores do too: one size per variant of the plain kernels and the row-broadcast
    kernel, and the fused-expression kernel on the same sizes (two results)."""
    print("case access hints n", n, flush=True)
    a = oracle.normal((n,), 11, 0, 3)
    b = oracle.normal((n,), 12, 0, 3)
    da, db = G.dev(a), G.dev(b)
    bits_equal(G.host(G.binary("add", da, db)), oracle.binary(dict(BIN)["add"], a, b), "add")
    bits_equal(G.host(G.unary("relu", da)), np.where(a > 0, a, np.float32(0)).astype(np.float32), "relu")
    cols = 4
    r = oracle.uniform((cols,), 13, 0.5, 2)
    got = G.host(G.rowbcast("mul", da.view(n // cols, cols), G.dev(r)))
    bits_equal(got.reshape(-1), (a.reshape(-1, cols) * r).astype(np.float32).reshape(-1), "row-broadcast mul")
    E = EX
    prog = [(E["LOAD_FULL"], 0, 0, 0, 0.0), (E["LOAD_FULL"], 1, 1, 0, 0.0), (E["MUL"], 2, 0, 1, 0.0), (E["ADDS"], 3, 2, 0, 5.0),
            (E["RELU"], 4, 3, 0, 0.0), (E["STORE"], 0, 4, 0, 0.0), (E["STORE"], 1, 2, 0, 0.0)]
    (y, p), _ = G.expr_run(prog, [da.view(n // cols, cols), db.view(n // cols, cols)], 2, n // cols, cols)
    ab = (a * b).astype(np.float32)
    t = (ab + np.float32(5.0)).astype(np.float32)
    bits_equal(G.host(y).reshape(-1), np.where(t > 0, t, np.float32(0)).astype(np.float32), "fused relu(a*b+5)")
    bits_equal(G.host(p).reshape(-1), ab, "fused a*b (second result)")


def test_binary_unaligned_views_bit_exact(oracle):
    print("case binary unaligned", flush=True)
    a = oracle.normal((5003,), 3, 0, 2)
    b = oracle.normal((5003,), 4, 0, 2)
    da, db = G.dev(a), G.dev(b)
    for off in (1, 2, 3):
        got = G.binary("mul", da[off:], db[off:].clone())   # first operand off the 16-byte grid
        bits_equal(G.host(got), oracle.mul(a[off:], b[off:]), f"offset {off}")


@pytest.mark.parametrize("shape", [(37, 53), (8, 256), (5, 10), (64, 4096), (1, 7), (300, 1)])
def test_row_broadcast_bit_exact(oracle, shape):
    print("case rowbcast", shape, flush=True)
    a = oracle.normal(shape, 5, 0, 2)
    b = oracle.uniform((shape[1],), 6, 0.5, 2)
    da, db = G.dev(a), G.dev(b)
    for name, code in BIN:
        bits_equal(G.host(G.rowbcast(name, da, db)), oracle.binary_rowbcast(code, a, b), name)


def test_scalar_forms_bit_exact(oracle):
    print("case scalar forms", flush=True)
    a = np.concatenate([oracle.normal((4099,), 7, 0, 3), SPECIAL])
    da = G.dev(a)
    s = F(1.7)
    ds = G.dev(np.array([s]))
    full = np.full_like(a, s)
    for name, code in BIN:
        bits_equal(G.host(G.bscalar(name, da, ds)), oracle.binary(code, a, full), "bscalar " + name)
    bits_equal(G.host(G.rsub(ds, da)), oracle.sub(full, a), "rsub")
    bits_equal(G.host(G.scalar("add", da, 5.0)), oracle.scalar(0, a, 5.0), "scalar add")
    bits_equal(G.host(G.scalar("mul", da, -2.5)), oracle.scalar(1, a, -2.5), "scalar mul")
    bits_equal(G.host(G.scalar("div", da, 3.0)), oracle.scalar(2, a, 3.0), "scalar div")


def test_division_by_a_shared_divisor_on_subnormal_midpoints(oracle):
    """a = M * B * 2^-149 (M odd), b = 2 * B: the exact quotient lies halfway between two subnormal
    floats, where IEEE division rounds to even.  Tensor / float and tensor / one-element tensor go
    through the divisor's double reciprocal and must break those ties the same way."""
    print("case division ties", flush=True)
    for B in (1, 3, 49, 98, 405, 1023):
        M = np.arange(1, min(1 << 18, (1 << 24) // B), 2, dtype=np.int64)
        a = np.ldexp((M * B).astype(np.float64), -149).astype(F)
        a[1::2] *= F(-1.0)
        b = F(2 * B)
        want = a / b
        assert want.view(np.uint32).tolist() == oracle.scalar(2, a, float(b)).view(np.uint32).tolist()
        da = G.dev(a)
        bits_equal(G.host(G.scalar("div", da, float(b))), want, f"tensor / float, B={B}")
        bits_equal(G.host(G.bscalar("div", da, G.dev(np.array([b])))), want, f"tensor / 0-D tensor, B={B}")


def test_neg_relu_fill_accumulate_bit_exact(oracle):
    print("case neg relu fill accumulate", flush=True)
    a = np.concatenate([oracle.normal((70001,), 8, 0, 3), SPECIAL])
    da = G.dev(a)
    bits_equal(G.host(G.unary("neg", da)), oracle.neg(a), "neg")
    r = G.host(G.unary("relu", da))
    want = oracle.relu(a)
    assert same_bits(r, want), "relu"          # NaN -> +0 here, so plain bit equality
    assert np.all(G.host(G.fill(1001, 2.5)) == F(2.5))
    assert np.all(G.host(G.fill_from(1001, G.dev(np.array([-0.75])))) == F(-0.75))
    g = oracle.normal((70001,), 9)
    v = oracle.normal((70001,), 10)
    want = g.copy()
    oracle.lib.co_accumulate(want.ctypes.data_as(G.C.POINTER(G.C.c_float)),
                             v.ctypes.data_as(G.C.POINTER(G.C.c_float)), G.C.c_long(g.size))
    bits_equal(G.host(G.accumulate(G.dev(g), G.dev(v))), want, "accumulate")


def test_transcendentals_within_2ulp(oracle):
    print("case transcendentals", flush=True)
    x = np.concatenate([oracle.uniform((200000,), 11, -2, 2), oracle.uniform((50000,), 12, -0.02, 0.02),
                        oracle.uniform((50000,), 13, -90, 90), oracle.uniform((50000,), 14, -1000, 1000),
                        oracle.normal((50000,), 15, 0, 1e6), SPECIAL])
    dx = G.dev(x)
    for name, code in [("sin", SIN), ("cos", COS), ("tanh", TANH), ("sigmoid", SIGMOID)]:
        ulp_close(G.host(G.unary(name, dx)), oracle.unary(code, x), 2, name)


def test_transcendentals_bit_identical_over_a_sweep_of_all_floats(oracle):
    """Every 509th fp32 bit pattern (8.4 million values: all exponents, both signs, subnormals,
    infinities, NaNs): Sin, Cos, Tanh and Sigmoid on the device have the oracle's bits - the restated
    glibc algorithms run in IEEE double on both sides.  (The stated bar is 2 ulp; this is what holds.)"""
    print("case transcendental sweep", flush=True)
    x = np.arange(0, 1 << 32, 509, dtype=np.uint64).astype(np.uint32).view(F)
    dx = G.dev(x)
    for name, code in [("sin", SIN), ("cos", COS), ("tanh", TANH), ("sigmoid", SIGMOID)]:
        got, want = G.host(G.unary(name, dx)), oracle.unary(code, x)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan), name
        assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32)), name


def test_tanh_over_every_float_against_its_formula_through_the_operator_kernels():
    """All 2^32 bit patterns: the tanh kernel against (e^x - e^-x) / (e^x + e^-x) formed by the exp, neg,
    sub, add and div kernels (the exponential's bits are glibc's - sweep above, native check - and the
    others are single IEEE operations).  tanh forms its quotient without the scaling and fix-up steps of
    the division the compiler writes: this is the check that those never mattered.  The gradient kernel
    recomputes tanh by the same routine: checked through 1 - tanh^2 on every 64th chunk."""
    import torch
    print("case tanh, every float", flush=True)
    chunk = 1 << 26
    base = torch.arange(chunk, dtype=torch.int64, device=G.DEV)
    ones = torch.ones(chunk, device=G.DEV)
    for c in range((1 << 32) // chunk):
        x = (base + c * chunk).to(torch.int32).view(torch.float32)
        ep, en = G.unary("exp", x), G.unary("exp", G.unary("neg", x))
        want = G.binary("div", G.binary("sub", ep, en), G.binary("add", ep, en))
        got = G.unary("tanh", x)
        nan = torch.isnan(want)
        assert bool((torch.isnan(got) == nan).all()), c
        assert bool((got.view(torch.int32)[~nan] == want.view(torch.int32)[~nan]).all()), c
        if c % 16 == 0:
            gb = G.unary_bwd("tanh", x, ones)
            wb = (1.0 - want * want) * ones          # three single operations, as the gradient kernel's
            ok = ~torch.isnan(wb)
            assert bool((torch.isnan(gb) == ~ok).all()), c
            assert bool((gb.view(torch.int32)[ok] == wb.view(torch.int32)[ok]).all()), c
        if c % 16 == 15:
            print("  chunk", c, flush=True)


def test_transcendentals_against_golden_reference_vectors(golden):
    print("case transcendentals golden", flush=True)
    g = golden("elementwise")
    for key_in, names in (("x", ["sin", "cos", "tanh", "sigmoid"]), ("t", ["t_sin", "t_cos", "t_tanh", "t_sigmoid"])):
        dx = G.dev(g[key_in])
        for nm in names:
            ulp_close(G.host(G.unary(nm.replace("t_", ""), dx)), g[nm], 2, "golden " + nm)
    x, y = G.dev(g["x"]), G.dev(g["y"])
    for name in ("add", "sub", "mul", "div"):
        bits_equal(G.host(G.binary(name, x, y)), g[name], "golden " + name)
    bits_equal(G.host(G.unary("neg", x)), g["neg"], "golden neg")
    assert same_bits(G.host(G.unary("relu", x)), g["relu"])


def test_elementwise_gradients(oracle):
    print("case elementwise gradients", flush=True)
    x = np.concatenate([oracle.normal((50001,), 16, 0, 2), SPECIAL[:32]])
    g = np.concatenate([oracle.normal((50001,), 17), SPECIAL[:32][::-1]])
    dx, dg = G.dev(x), G.dev(g)
    bits_equal(G.host(G.unary_bwd("relu", dx, dg)), oracle.relu_bwd(x, g), "relu bwd")
    for name, code in [("sigmoid", SIGMOID), ("tanh", TANH), ("sin", SIN), ("cos", COS)]:
        ulp_close(G.host(G.unary_bwd(name, dx, dg)), oracle.unary_bwd(code, x, g), 2, name + " bwd")
    # the same gradients added to a gradient gathered so far: bit for bit the separate kernel, then "+"
    gathered = np.concatenate([oracle.normal((50001,), 21, 0, 1), SPECIAL[:32]])
    gathered[:64] = F(-0.0)
    dacc = G.dev(gathered)
    with np.errstate(invalid="ignore", over="ignore"):
        for name in ("relu", "sigmoid", "tanh", "sin", "cos"):
            sep = G.host(G.unary_bwd(name, dx, dg))
            got = G.host(G.unary_bwd_acc(name, dx, dg, dacc))
            want = (gathered + sep).astype(F)
            both_nan = np.isnan(got) & np.isnan(want)
            assert np.array_equal(np.where(both_nan, 0, got.view(np.uint32)), np.where(both_nan, 0, want.view(np.uint32))), name
        out = torch.empty_like(dx)
        G.call("ctamd_mul_acc_f32", G.ptr(dx), G.ptr(dg), G.ptr(dacc), G.ptr(out), dx.numel(), G.stream())
        want = (gathered + (x * g).astype(F)).astype(F)
        both_nan = np.isnan(G.host(out)) & np.isnan(want)
        assert np.array_equal(np.where(both_nan, 0, G.host(out).view(np.uint32)), np.where(both_nan, 0, want.view(np.uint32))), "mul + gathered"
        G.call("ctamd_div_acc_f32", G.ptr(dx), G.ptr(dg), G.ptr(dacc), G.ptr(out), dx.numel(), G.stream())
        want = (gathered + (x / g).astype(F)).astype(F)
        both_nan = np.isnan(G.host(out)) & np.isnan(want)
        assert np.array_equal(np.where(both_nan, 0, G.host(out).view(np.uint32)), np.where(both_nan, 0, want.view(np.uint32))), "div + gathered"
    for rows, cols in ((37, 53), (129, 1024)):
        a2, acc2 = oracle.normal((rows, cols), 83, 0, 2), oracle.normal((rows, cols), 84)
        rv = oracle.uniform((cols,), 85, 0.5, 2)
        out2 = torch.empty(rows, cols, device=G.DEV)
        da2, drv, dacc2 = G.dev(a2), G.dev(rv), G.dev(acc2)        # held: a pointer does not keep a tensor alive
        G.call("ctamd_div_rowbcast_acc_f32", G.ptr(da2), G.ptr(drv), G.ptr(dacc2), G.ptr(out2), rows, cols, G.stream())
        bits_equal(G.host(out2), (acc2 + (a2 / rv).astype(F)).astype(F), "row-vector div + gathered")
    p = oracle.normal((50001,), 18, 0, 2)
    t = oracle.normal((50001,), 19, 0, 2)
    t[:100] = p[:100]           # exact ties: sign(0) = 0
    g1 = G.dev(np.array([0.37]))
    bits_equal(G.host(G.loss_bwd("mse", G.dev(p), G.dev(t), g1)), oracle.mse_bwd(p, t, F(0.37)), "mse bwd")
    bits_equal(G.host(G.loss_bwd("mae", G.dev(p), G.dev(t), g1)), oracle.mae_bwd(p, t, F(0.37)), "mae bwd")
    # the term added to a gradient gathered so far in the same pass: gathered + term, the term rounded first
    acc = oracle.normal((50001,), 20, 0, 1e-5)
    acc[:50] = F(-0.0)
    for name, want in (("mse", oracle.mse_bwd(p, t, F(0.37))), ("mae", oracle.mae_bwd(p, t, F(0.37)))):
        bits_equal(G.host(G.loss_bwd_acc(name, G.dev(p), G.dev(t), g1, G.dev(acc))), (acc + want).astype(F), name + " bwd + gathered")
    b = (t + F(4.0) * np.sign(t) + F(0.5)).astype(F)
    bits_equal(G.host(G.div_bwd_b(G.dev(p), G.dev(b), G.dev(g[:50001]))), oracle.div_bwd_b(p, b, g[:50001]), "div bwd b")
    # row-vector divisor: the same arithmetic on the divisor repeated down the rows
    for rows, cols in ((37, 53), (129, 1024), (5, 4100)):
        a2 = oracle.normal((rows, cols), 81, 0, 2)
        g2 = oracle.normal((rows, cols), 82)
        bv = oracle.uniform((cols,), 83, 0.5, 2)
        d_a, d_b, d_g = G.dev(a2), G.dev(bv), G.dev(g2)
        bits_equal(G.host(G.div_bwd_b_rowbcast(d_a, d_b, d_g)),
                   oracle.div_bwd_b(a2, np.ascontiguousarray(np.broadcast_to(bv, (rows, cols))), g2), "div bwd b rowbcast")
    assert G.any_tiny(G.dev(b)) == 0
    b[777] = 1e-8
    assert G.any_tiny(G.dev(b)) == 1 and oracle.any_abs_lt_eps(b)


@pytest.mark.parametrize("n", [0, 1, 5, 1000, 65537, (1 << 22) + 1])
def test_reductions_normwise(oracle, n):
    print("case reductions n", n, flush=True)
    a = oracle.uniform((n,), 21, -1, 1)
    b = oracle.uniform((n,), 22, -1, 1)
    da, db = G.dev(a), G.dev(b)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    cases = [("sum", G.host(G.reduce1("sum", da))[0], a64.sum(), np.abs(a64).sum()),
             ("dot", G.host(G.reduce2("dot", da, db))[0], a64 @ b64, np.abs(a64 * b64).sum())]
    if n:
        cases += [("mse", G.host(G.reduce2("mse", da, db))[0], ((a64 - b64) ** 2).mean(), ((a64 - b64) ** 2).mean()),
                  ("mae", G.host(G.reduce2("mae", da, db))[0], np.abs(a64 - b64).mean(), np.abs(a64 - b64).mean())]
    for name, got, want, scale in cases:
        assert abs(got - want) <= 1e-5 * scale + 1e-30, (name, got, want)
    if 0 < n <= 70000:   # the oracle's sequential sums agree to the same bound
        assert abs(G.host(G.reduce2("dot", da, db))[0] - oracle.dot(a, b)) <= 1e-5 * np.abs(a64 * b64).sum()
        assert abs(G.host(G.reduce2("mse", da, db))[0] - oracle.mse(a, b)) <= 1e-5 * oracle.mse(a, b)


@pytest.mark.parametrize("shape", [(1, 1), (2, 3), (37, 53), (8192, 256), (1000, 10), (4096, 4096), (33, 4100), (70000, 3), (128, 10),
                                   (256, 256), (1024, 512), (1025, 16), (1024, 513), (8192, 10), (100000, 128), (5000, 512), (3001, 129),
                                   (2049, 1)])
def test_column_sum(oracle, shape):
    print("case colsum", shape, flush=True)
    g = oracle.normal(shape, 23)
    got = G.host(G.colsum(G.dev(g)))
    want = g.astype(np.float64).sum(0)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(g).astype(np.float64).sum(0))
    if shape[0] * shape[1] < 1 << 16:
        assert np.all(np.abs(got - oracle.colsum_f64(g)) <= 1e-5 * np.abs(g).astype(np.float64).sum(0))


SOFTMAX_SHAPES = [(1, 1), (3, 7), (19, 301), (64, 10), (5, 1000), (7, 1024), (4, 2052), (3, 8192), (2, 8200),
                  (2, 32000), (2, 32768), (2, 33000), (3, 40001), (2, 131076),
                  (3, 65536), (2, 49156), (2, 65540)]      # rows kept on the chip between the two sweeps: full, partly, one word too long


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
def test_softmax_and_cross_entropy_rows(oracle, shape):
    print("case softmax/ce", shape, flush=True)
    rows, cols = shape
    x = oracle.normal(shape, 24, 0, 2)
    dx = G.dev(x)
    y = G.host(G.softmax(dx, 1))
    want = oracle.softmax(x, 1)
    # same exp() bits; only the order of the row sum differs (tree here, sequential fp32 in the
    # reference), which scales a whole row by 1 + O(cols * 2^-24): 1e-5 relative, fp64 as arbiter
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(1, keepdims=True))
    y64 = e64 / e64.sum(1, keepdims=True)
    assert np.all(np.abs(y - y64) <= 1e-5 * y64 + 1e-45)
    # (beyond 65536 columns the reference's own sequential fp32 sum has drifted from the true sum by
    # more than 1e-5: ~sqrt(cols) roundings of 2^-24 each; the fp64 arbiter above keeps the 1e-5 bar)
    ref_tol = 1e-5 if cols <= 65536 else 4 * np.sqrt(cols) * 2.0 ** -24
    assert np.all(np.abs(y - want) <= ref_tol * want + 1e-45)
    assert np.allclose(y.astype(np.float64).sum(1), 1, atol=1e-5)
    idx = oracle.ints((rows,), 25, cols)
    oh = np.zeros(shape, F)
    oh[np.arange(rows), idx.astype(int)] = 1
    loss_i, status = G.ce_index(dx, G.dev(idx))
    assert status == 0
    loss_o = G.ce_onehot(dx, G.dev(oh))
    want_loss = oracle.ce_index(x, idx) if rows != cols else oracle.ce_onehot(x, oh)
    for got in (G.host(loss_i)[0], G.host(loss_o)[0]):
        assert abs(got - want_loss) <= 1e-5 * abs(want_loss) + 1e-6
    soft = oracle.softmax(oracle.normal(shape, 26), 1)
    got = G.host(G.ce_onehot(dx, G.dev(soft)))[0]
    assert abs(got - oracle.ce_onehot(x, soft)) <= 1e-5 * abs(oracle.ce_onehot(x, soft)) + 1e-6
    g1 = G.dev(np.array([-1.25]))
    want_d = oracle.ce_bwd_onehot(x, oh, F(-1.25))
    for got in (G.host(G.ce_bwd(dx, G.dev(oh), g1, False)), G.host(G.ce_bwd(dx, G.dev(idx), g1, True))):
        assert np.abs(got - want_d).max() <= 1e-6
    w = oracle.normal(shape, 27)
    got = G.host(G.softmax_bwd(G.dev(want), G.dev(w), 1))
    want_b = oracle.softmax_bwd(want, w, 1)
    scale = (np.abs(want) * (np.abs(w) + np.abs(w * want).sum(1, keepdims=True))).astype(np.float64)
    assert np.all(np.abs(got - want_b) <= 1e-5 * scale + 1e-12)


@pytest.mark.parametrize("shape", [(64, 10), (19, 301), (4, 2052), (3, 8192), (2, 33000), (3, 40001)])
def test_cross_entropy_backward_from_forward_statistics(oracle, shape):
    """The class-index forward pass leaves (max, sum) per row; the backward pass that uses them
    agrees with the oracle's dlogits and with the backward pass that recomputes them."""
    print("case ce stats", shape, flush=True)
    rows, cols = shape
    x = oracle.normal(shape, 90, 0, 2)
    idx = oracle.ints((rows,), 91, cols)
    dx, didx = G.dev(x), G.dev(idx)
    loss = torch.empty(1, device=G.DEV)
    status = torch.zeros(1, dtype=torch.int32, device=G.DEV)
    stats = torch.empty(rows, 2, device=G.DEV)
    G.call("ctamd_cross_entropy_index_stats_f32", G.ptr(dx), G.ptr(didx), G.ptr(loss), G.ptr(status), G.ptr(stats), rows,
           cols, G.stream())
    st = G.host(stats)
    x64 = x.astype(np.float64)
    assert int(status.item()) == 0 and np.array_equal(st[:, 0], x.max(1))
    s64 = np.exp(x64 - x64.max(1, keepdims=True)).sum(1)
    assert np.all(np.abs(st[:, 1] - s64) <= 1e-5 * s64)
    want_loss = oracle.ce_index(x, idx)
    assert abs(G.host(loss)[0] - want_loss) <= 1e-5 * abs(want_loss)
    g1 = G.dev(np.array([0.75]))
    out = torch.empty_like(dx)
    G.call("ctamd_cross_entropy_backward_index_stats_f32", G.ptr(dx), G.ptr(didx), G.ptr(stats), G.ptr(g1), G.ptr(out),
           rows, cols, G.stream())
    oh = np.zeros(shape, F)
    oh[np.arange(rows), idx.astype(int)] = 1
    want = oracle.ce_bwd_onehot(x, oh, F(0.75))
    assert np.abs(G.host(out) - want).max() <= 1e-6
    assert np.abs(G.host(out) - G.host(G.ce_bwd(dx, didx, g1, True))).max() <= (5e-7 if cols >= 2048 else 2e-7)


@pytest.mark.parametrize("shape", [(1, 1), (64, 10), (19, 301), (33, 1000), (4, 2052), (3, 8192), (5, 32768), (2, 8191)])
def test_cross_entropy_loss_and_gradient_in_one_pass(oracle, shape):
    """ctamd_cross_entropy_index_fused_f32: the loss of the forward entry point and the gradient the
    backward entry point gives for an upstream gradient of 1 - bit for bit against the recomputing
    backward for rows under 2048 columns (same exponential, same sums), to the reduction bar against
    the oracle everywhere."""
    print("case ce fused", shape, flush=True)
    rows, cols = shape
    x = oracle.normal(shape, 92, 0, 2)
    idx = oracle.ints((rows,), 93, cols)
    dx, didx = G.dev(x), G.dev(idx)
    loss, status, grad = G.ce_index_fused(dx, didx)
    want_loss = oracle.ce_index(x, idx)
    assert status == 0 and abs(G.host(loss)[0] - want_loss) <= 1e-5 * abs(want_loss) + 1e-6
    oh = np.zeros(shape, F)
    oh[np.arange(rows), idx.astype(int)] = 1
    assert np.abs(G.host(grad) - oracle.ce_bwd_onehot(x, oh, F(1.0))).max() <= 1e-6
    one = G.dev(np.array([1.0]))
    if cols < 2048:
        bits_equal(G.host(grad), G.host(G.ce_bwd(dx, didx, one, True)), "fused gradient vs the backward entry point")
    else:   # long rows use the hardware exponential, as the forward / backward-from-statistics pair does
        assert np.abs(G.host(grad) - G.host(G.ce_bwd(dx, didx, one, True))).max() <= 5e-7
    assert np.all(np.abs(G.host(grad).astype(np.float64).sum(1)) <= 1e-5)
    # a bad index: status and a NaN loss as the forward entry point; the row's gradient is its softmax
    if cols > 1:
        bad = idx.copy()
        bad[rows // 2] = cols
        loss, status, grad_bad = G.ce_index_fused(dx, G.dev(bad))
        assert status == 1 and np.isnan(G.host(loss)[0])
        keep = np.arange(rows) != rows // 2
        bits_equal(G.host(grad_bad)[keep], G.host(grad)[keep], "rows with good indices")


def test_cross_entropy_in_one_pass_refuses_rows_beyond_its_registers(oracle):
    x = torch.zeros(2, 32772, device=G.DEV)
    idx = torch.zeros(2, device=G.DEV)
    out = torch.empty(1, device=G.DEV)
    rc = G.lib().ctamd_cross_entropy_index_fused_f32(G.ptr(x), G.ptr(idx), G.ptr(out), None, G.ptr(torch.empty_like(x)), 2, 32772, G.stream())
    assert rc == -5
    rc = G.lib().ctamd_cross_entropy_index_fused_f32(G.ptr(x), G.ptr(idx), G.ptr(out), None, G.ptr(torch.empty_like(x)), 2, 8193, G.stream())
    assert rc == -5


def test_cross_entropy_edge_cases(oracle):
    print("case ce edges", flush=True)
    x = oracle.normal((19, 31), 28, 0, 2)
    idx = oracle.ints((19,), 29, 31)
    bad = idx.copy()
    bad[3] = 31
    loss, status = G.ce_index(G.dev(x), G.dev(bad))
    assert status == 1 and np.isnan(G.host(loss)[0]) and oracle.ce_index(x, bad) is None
    bad[3] = -1
    assert G.ce_index(G.dev(x), G.dev(bad))[1] == 1
    # an index is a float read by truncation: NaN, the infinities and magnitudes beyond int are out of
    # range (the reference's conversion yields the most negative int for them); 30.9 is class 30, -0.9 class 0
    for wrong in (np.nan, np.inf, -np.inf, 3e9, -3e9, 31.2):
        bad[3] = wrong
        assert G.ce_index(G.dev(x), G.dev(bad))[1] == 1 and oracle.ce_index(x, bad) is None, wrong
        assert G.ce_index_fused(G.dev(x), G.dev(bad))[1] == 1, wrong
    frac, whole = idx.copy(), idx.copy()
    frac[3], frac[4], whole[3], whole[4] = 30.9, -0.9, 30.0, 0.0
    a, b = G.ce_index(G.dev(x), G.dev(frac)), G.ce_index(G.dev(x), G.dev(whole))
    assert a[1] == 0 and b[1] == 0 and same_bits(G.host(a[0]), G.host(b[0]))
    assert abs(G.host(a[0])[0] - oracle.ce_index(x, frac)) <= 1e-5 * abs(oracle.ce_index(x, frac))
    # the 1e-10 clamp
    hx = x.copy()
    hx[:, 0] += 60.0
    oh = np.zeros_like(x)
    oh[np.arange(19), idx.astype(int)] = 1
    want = oracle.ce_onehot(hx, oh)
    assert abs(G.host(G.ce_onehot(G.dev(hx), G.dev(oh)))[0] - want) <= 1e-5 * abs(want)
    assert abs(G.host(G.ce_index(G.dev(hx), G.dev(idx))[0])[0] - want) <= 1e-5 * abs(want)
    # 1-D logits (single sample)
    want = oracle.ce_onehot(x[0], oh[0])
    assert abs(G.host(G.ce_onehot(G.dev(x[0]), G.dev(oh[0])))[0] - want) <= 1e-5 * abs(want)
    # long rows (single-pass kernel): -inf logits contribute exp(-inf) = 0, also where a whole
    # thread's share of the row is -inf
    lx = oracle.normal((3, 4096), 32, 0, 2)
    lx[:, :2600] = -np.inf
    lx[1, 5::2] = -np.inf
    lidx = np.array([3000, 3001, 4095], F)
    want = oracle.ce_index(lx, lidx)
    got, status = G.ce_index(G.dev(lx), G.dev(lidx))
    assert status == 0 and abs(G.host(got)[0] - want) <= 1e-5 * abs(want)
    # rows == 0 gives a zero loss
    assert G.host(G.ce_onehot(G.dev(np.zeros((0, 5), F)), G.dev(np.zeros((0, 5), F))))[0] == 0


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (37, 53), (127, 19), (128, 8), (301, 19), (1000, 300), (4099, 10),
                                   (700, 1028), (20000, 64)])
def test_softmax_columns(oracle, shape):
    """Column (dim 0) softmax and its gradient.  Below 128 rows one thread walks a column in the
    reference's order: 2 ulp / the same fma chain bit for bit.  Tall matrices use chunked column
    reductions: the reduction bar (1e-5 relative, fp64 as the arbiter, the oracle to the same bound)."""
    print("case softmax cols", shape, flush=True)
    x = oracle.normal(shape, 30, 0, 2)
    y = G.host(G.softmax(G.dev(x), 0))
    want = oracle.softmax(x, 0)
    w = oracle.normal(shape, 31)
    got = G.host(G.softmax_bwd(G.dev(want), G.dev(w), 0))
    want_b = oracle.softmax_bwd(want, w, 0)
    if shape[0] < 128:
        assert ulp_diff(y, want).max() <= 2
        bits_equal(got, want_b, "softmax bwd cols")   # same sequential fma chain
        return
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(0, keepdims=True))
    y64 = e64 / e64.sum(0, keepdims=True)
    assert np.all(np.abs(y - y64) <= 1e-5 * y64 + 1e-37)
    assert np.all(np.abs(y - want) <= 1e-5 * want + 1e-37)
    assert np.all(np.abs(y.astype(np.float64).sum(0) - 1.0) <= 1e-5)
    w64, s64 = w.astype(np.float64), want.astype(np.float64)
    d64 = (w64 * s64).sum(0, keepdims=True)
    scale = np.abs(s64) * (np.abs(w64) + np.abs(w64 * s64).sum(0, keepdims=True))
    assert np.all(np.abs(got - s64 * (w64 - d64)) <= 1e-5 * scale + 1e-12)
    assert np.all(np.abs(got - want_b) <= 2e-5 * scale + 1e-12)


def test_softmax_columns_tall_edge_cases(oracle):
    """The running (max, sum) pairs of the tall-matrix column softmax where they are stressed: a
    maximum that moves at every row, one that never moves, elements of -inf, a spread beyond exp's
    range, and a column that is -inf everywhere but one row."""
    print("case softmax cols tall edge cases", flush=True)
    rows, cols = 777, 12
    x = oracle.normal((rows, cols), 33, 0, 1)
    ramp = np.arange(rows, dtype=F)
    x[:, 0] = ramp * 0.25                       # ascending: every row is a new maximum
    x[:, 1] = -ramp * 0.25                      # descending: the first row stays the maximum
    x[::3, 2] = -np.inf                         # holes
    x[:, 3] = -np.inf
    x[401, 3] = 2.5                             # one finite element
    x[:, 4] = np.where(np.arange(rows) % 2 == 0, 300.0, -300.0).astype(F)
    x[:5, 5] = -np.inf                          # a chunk that begins with -inf
    x[:, 6] = 88.0 + ramp * 0.01                # exp(x) itself would overflow
    y = G.host(G.softmax(G.dev(x), 0))
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(0, keepdims=True))
    y64 = e64 / e64.sum(0, keepdims=True)
    assert np.all(np.isfinite(y))
    assert np.all(np.abs(y - y64) <= 1e-5 * y64 + 1e-37)
    assert np.all(y[x == -np.inf] == 0)
    assert y[401, 3] == 1.0
    want = oracle.softmax(x, 0)
    assert np.all(np.abs(y - want) <= 1e-5 * want + 1e-37)


MM_SHAPES = [(1, 1, 1), (5, 3, 9), (33, 29, 47), (128, 128, 16), (130, 257, 70), (256, 10, 784), (64, 256, 10),
             (784, 256, 300), (256, 10, 8192), (17, 1, 33), (1, 40, 33), (200, 200, 1), (384, 512, 1024),
             # ragged edges and a K that is no multiple of the k tile, for the 128 x 128, the 256 x 256 and
             # the 256 x 128 tile shapes (the launcher picks by rounds of tiles per CU)
             (2049, 2050, 33), (4100, 4101, 70), (4090, 4093, 40), (4090, 2047, 40),
             # an output of at most 16 columns: the streaming kernels, in rows (A row-major) and in
             # columns (A a transposed view) with and without a cut K, ragged m and k
             (8192, 10, 256), (8190, 16, 252), (1000, 1, 512), (70, 3, 8), (5000, 7, 52), (300, 16, 1000),
             (777, 13, 3001), (66000, 2, 12), (20000, 10, 256), (9000, 5, 700),
             # at most one 32 x 32 tile per CU and K <= 512: the small-product kernel (those above with
             # small extents take it too); the same extents with a longer K stay on the 64 x 64 tiles
             (256, 256, 256), (784, 256, 256), (100, 70, 300), (512, 512, 512), (31, 33, 512),
             (130, 257, 600), (70, 33, 1000), (100, 70, 513),
             # at most one block per CU with a long K: the 64 x 64 tile's kernels with four and two wave
             # groups per block and the 128 x 128 tile's with two, ragged edges, and with K cut over blocks
             (1000, 1010, 1024), (1024, 1000, 544), (2040, 2048, 1056), (512, 500, 4096), (1024, 1024, 1024),
             # aligned rows and a K that ends inside a k tile: the pipelined loop hands its last tiles to
             # the bounds-checked one (one and four wave groups, K cut over blocks, the 256 x 256 tile)
             (1024, 1024, 1000), (256, 128, 40), (300, 200, 4100), (2048, 2048, 1052), (4096, 2048, 100), (512, 512, 36)]


@pytest.mark.parametrize("m,n,k", MM_SHAPES)
def test_matmul_all_layouts_normwise(oracle, m, n, k):
    print("case matmul", m, n, k, flush=True)
    A = oracle.normal((m, k), 41)
    B = oracle.normal((k, n), 42)
    dA, dB = G.dev(A), G.dev(B)
    dAt, dBt = G.dev(np.ascontiguousarray(A.T)), G.dev(np.ascontiguousarray(B.T))
    C64 = A.astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1e-30
    small = m * n * k <= 1 << 22
    want = oracle.matmul(A, B) if small else None
    for name, a, b in [("nn", dA, dB), ("nt", dA, dBt.t()), ("tn", dAt.t(), dB), ("tt", dAt.t(), dBt.t())]:
        got = G.host(G.matmul(a, b))
        assert np.all(np.abs(got - C64) <= bound), name
        if small:
            assert np.all(np.abs(got - want) <= 2 * bound), name


@pytest.mark.parametrize("m,n,k", [(256, 128, 784), (128, 10, 64), (70, 33, 129), (8192, 256, 784), (96, 12, 4096),
                                   (2100, 2050, 40), (4090, 4093, 24), (4090, 2047, 24), (5, 7, 0),
                                   (8192, 10, 256), (256, 10, 8192), (777, 13, 3001), (256, 256, 256), (100, 70, 300),
                                   (1000, 1010, 1024), (1024, 1000, 544), (2040, 2048, 1056), (512, 500, 4096),
                                   (1024, 1024, 1000), (300, 200, 4100), (4096, 2048, 100)])
def test_fused_layer_equals_the_three_launches(oracle, m, n, k):
    """matmul + bias row + ReLU in one launch against the same three operators launched in sequence,
    bit for bit, over all tile shapes (the last four: wave groups inside a block), the K-split fold
    ((96, 12, 4096)) and ragged edges; and against
    the CPU oracle's sequence within the MatMul bound."""
    print("case fused layer", m, n, k, flush=True)
    A = oracle.normal((m, k), 61)
    B = oracle.normal((k, n), 62)
    bias = oracle.normal((n,), 63)
    dA, dB, db = G.dev(A), G.dev(B), G.dev(bias)
    dBt = G.dev(np.ascontiguousarray(B.T))
    dAt = G.dev(np.ascontiguousarray(A.T))
    for a, b in ((dA, dB), (dA, dBt.t()), (dAt.t(), dB)):
        plain = G.matmul(a, b)
        biased = G.rowbcast("add", plain, db)
        assert same_bits(G.host(G.matmul_bias(a, b, None, False)), G.host(plain))
        assert same_bits(G.host(G.matmul_bias(a, b, db, False)), G.host(biased))
        assert same_bits(G.host(G.matmul_bias(a, b, db, True)), G.host(G.unary("relu", biased)))
        assert same_bits(G.host(G.matmul_bias(a, b, None, True)), G.host(G.unary("relu", plain)))
    if m * n * max(k, 1) <= 1 << 22:
        want = oracle.relu(oracle.binary_rowbcast(ADD, oracle.matmul(A, B), bias)) if k else np.maximum(np.broadcast_to(bias, (m, n)), 0)
        bound = 2e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1e-6
        assert np.all(np.abs(G.host(G.matmul_bias(dA, dB, db, True)) - want) <= bound)


def test_matmul_exact_on_small_integers_and_unaligned_views(oracle):
    print("case matmul integers", flush=True)
    rng = np.random.default_rng(7)
    A = rng.integers(-8, 9, (150, 203)).astype(F)
    B = rng.integers(-8, 9, (203, 77)).astype(F)
    want = (A.astype(np.int64) @ B.astype(np.int64)).astype(F)
    assert np.array_equal(G.host(G.matmul(G.dev(A), G.dev(B))), want)        # ld 203 / 77: scalar loads
    # row-sliced views: unit inner stride, leading dimension larger than the extent
    Abig, Bbig = G.dev(np.pad(A, ((0, 0), (0, 5)))), G.dev(np.pad(B, ((0, 0), (0, 3))))
    assert np.array_equal(G.host(G.matmul(Abig[:, :203], Bbig[:, :77])), want)
    # a narrow output from row-sliced views (leading dimensions 208 and 80), A in rows and in columns
    assert np.array_equal(G.host(G.matmul(Abig[:, :203], Bbig[:, :9])), want[:, :9])
    Atbig = G.dev(np.pad(np.ascontiguousarray(A.T), ((0, 0), (0, 6))))
    assert np.array_equal(G.host(G.matmul(Atbig[:, :150].t(), Bbig[:, :9])), want[:, :9])
    # no unit stride at all: generic kernel
    A2, B2 = G.dev(np.repeat(A, 2, axis=1)), G.dev(np.repeat(B, 2, axis=1))
    At2 = G.dev(np.repeat(np.ascontiguousarray(A.T), 2, axis=1))
    assert np.array_equal(G.host(G.matmul(A2[:, ::2], B2[:, ::2])), want)
    assert np.array_equal(G.host(G.matmul(At2[:, ::2].t(), B2[:, ::2])), want)


def test_golden_reference_vectors_reductions_matmul_backward(golden, oracle):
    print("case golden reductions/matmul/backward", flush=True)
    g = golden("reduce_softmax_ce")
    v1, v2 = G.dev(g["v1"]), G.dev(g["v2"])
    a64, b64 = g["v1"].astype(np.float64), g["v2"].astype(np.float64)
    assert abs(G.host(G.reduce2("dot", v1, v2))[0] - g["dot"]) <= 1e-5 * np.abs(a64 * b64).sum()
    assert abs(G.host(G.reduce2("mse", v1, v2))[0] - g["mse"]) <= 1e-5 * g["mse"]
    assert abs(G.host(G.reduce2("mae", v1, v2))[0] - g["mae"]) <= 1e-5 * g["mae"]
    assert abs(G.host(G.reduce1("sum", v1))[0] - g["sum"]) <= 1e-5 * np.abs(a64).sum()
    sx = G.dev(g["sx"])
    assert np.all(np.abs(G.host(G.softmax(sx, 1)) - g["softmax_d1"]) <= 1e-5 * g["softmax_d1"])
    assert ulp_diff(G.host(G.softmax(sx, 0)), g["softmax_d0"]).max() <= 2
    assert abs(G.host(G.ce_index(sx, G.dev(g["idx"]))[0])[0] - g["ce_index"]) <= 1e-5 * g["ce_index"]
    m = golden("matmul")
    A, B = m["A"], m["B"]
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert np.all(np.abs(G.host(G.matmul(G.dev(A), G.dev(B))) - m["nn"]) <= 2 * bound)
    b = golden("backward")
    x, w = b["x"], b["w"]
    dx, dw = G.dev(x), G.dev(w)
    bits_equal(G.host(G.unary_bwd("relu", dx, dw)) + F(0), b["d_relu"], "golden relu bwd")
    for name in ("sigmoid", "tanh", "sin", "cos"):
        ulp_close(G.host(G.unary_bwd(name, dx, dw)) + F(0), b["d_" + name], 2, "golden bwd " + name)
    g1 = G.dev(np.array([0.37]))
    bits_equal(G.host(G.loss_bwd("mse", dx, G.dev(b["y"]), g1)) + F(0), b["d_mse"], "golden mse bwd")
    bits_equal(G.host(G.loss_bwd("mae", dx, G.dev(b["y"]), g1)) + F(0), b["d_mae"], "golden mae bwd")
    bits_equal(G.host(G.binary("div", dw, G.dev(b["yb"]))) + F(0), b["d_div_a"], "golden div bwd a")
    bits_equal(G.host(G.div_bwd_b(dx, G.dev(b["yb"]), dw)) + F(0), b["d_div_b"], "golden div bwd b")


@pytest.mark.parametrize("n", [1, 3, 1024, 4099, 1 << 20])
def test_comparisons_bit_exact(oracle, n):
    """The six comparison operators against a tensor and against a float: one byte per element,
    identical to the oracle, including equal values, signed zeros, infinities and NaN; aligned and
    unaligned operands."""
    print("case compare", n, flush=True)
    a = oracle.normal((n,), 70, 0, 1)
    b = oracle.normal((n,), 71, 0, 1)
    b[::3] = a[::3]                                       # equal elements
    special = f32([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, np.nan])
    k = min(n, special.size)
    a[:k] = special[:k]
    b[:k] = special[::-1][:k] if n > 1 else special[:1]
    da, db = G.dev(a), G.dev(b)
    pad_a, pad_b = G.dev(np.concatenate([[0.0], a])), G.dev(np.concatenate([[0.0], b]))
    for cmp in range(6):
        out = torch.empty(n, dtype=torch.uint8, device=G.DEV)
        G.call("ctamd_compare_f32", cmp, G.ptr(da), G.ptr(db), G.ptr(out), n, G.stream())
        assert np.array_equal(out.cpu().numpy(), oracle.compare(cmp, a, b)), cmp
        G.call("ctamd_compare_f32", cmp, G.ptr(pad_a[1:]), G.ptr(pad_b[1:]), G.ptr(out), n, G.stream())   # 4-byte aligned only
        assert np.array_equal(out.cpu().numpy(), oracle.compare(cmp, a, b)), cmp
        for s in (0.0, 0.25, float("nan")):
            G.call("ctamd_compare_scalar_f32", cmp, G.ptr(da), C.c_float(s), G.ptr(out), n, G.stream())
            assert np.array_equal(out.cpu().numpy(), oracle.compare(cmp, a, None, s)), (cmp, s)
    assert G.lib().ctamd_compare_f32(9, G.ptr(da), G.ptr(db), G.ptr(out), n, G.stream()) == -1


@pytest.mark.parametrize("m,n,k", [(256, 10, 256), (784, 256, 256), (256, 10, 8192), (784, 16, 1024), (70, 1, 129), (33, 3, 1), (1, 1, 1),
                                   (31, 33, 512), (100, 70, 513), (512, 512, 64), (300, 7, 3000), (784, 256, 8192),
                                   (520, 128, 5000), (200, 512, 3000), (130, 516, 3000), (64, 64, 100000)])
def test_product_with_the_column_sums_of_its_second_operand(oracle, m, n, k):
    """The weight gradient x^T . dz and the bias gradient (column sums of dz) from one call: the
    bits of ctamd_matmul_f32 and of ctamd_colsum_f32, whether the sums ride in the product's launch
    (a product of at most 256 tiles of 32 x 32 with K <= 512), in the two launches of a product cut
    along K on the 64 x 64 tiles (the last five shapes; 516 columns are one vector too many for that
    and K = 5000 ends inside a k tile) or follow it as launches of their own."""
    print("case matmul + column sums", m, n, k, flush=True)
    X = oracle.normal((k, m), 61)
    dZ = oracle.normal((k, n), 62)
    dX, dZd = G.dev(X), G.dev(dZ)
    l = G.lib()
    for name, a in (("x^T as a view", dX.t()), ("x^T materialised", G.dev(np.ascontiguousarray(X.T)))):
        l.ctamd_counters_reset()
        c, sums = G.matmul_colsum(a, dZd)
        by, fl, ideal, launches = C.c_double(), C.c_double(), C.c_double(), C.c_uint64()
        l.ctamd_counters_read(C.byref(by), C.byref(fl), C.byref(ideal), C.byref(launches))
        # one operator when the sums ride along, two when the column sum follows as its own
        small = -(-m // 32) * -(-n // 32) <= 256 and k <= 512            # the one-launch small-product kernel
        rides = small or (m, n, k) in ((784, 256, 8192), (520, 128, 5000), (200, 512, 3000), (64, 64, 100000))
        assert launches.value == (1 if rides else 2), (name, launches.value)
        assert same_bits(G.host(c), G.host(G.matmul(a, dZd))), name
        assert same_bits(G.host(sums), G.host(G.colsum(dZd))), name
    # a second operand that is not in contiguous rows: refused before anything is launched
    if n > 1 and k > 1:
        wide = G.dev(oracle.normal((k, n + 3), 63))
        c = torch.empty((m, n), device=G.DEV)
        sums = torch.empty((n,), device=G.DEV)
        a = G.dev(np.ascontiguousarray(X.T))
        assert l.ctamd_matmul_colsum_f32(G.ptr(a), k, 1, G.ptr(wide), n + 3, 1, G.ptr(c), G.ptr(sums), m, n, k, G.stream()) == -1
        assert l.ctamd_matmul_colsum_f32(G.ptr(a), k, 1, G.ptr(wide), 1, k, G.ptr(c), G.ptr(sums), m, n, k, G.stream()) == -1


@pytest.mark.parametrize("m,n,k", [(256, 256, 10), (8192, 256, 10), (100, 70, 300), (300, 200, 1000), (2100, 2050, 40),
                                   (4090, 2047, 24), (96, 12, 4096), (64, 10, 256), (5, 7, 0)])
def test_product_times_relu_mask_equals_the_two_launches(oracle, m, n, k):
    """(a.b) * [y > 0] in the product's launch against the product followed by the ReLU gradient
    kernel, bit for bit: the small-product kernel, the tiles with and without a cut K, ragged edges,
    the narrow and strided forms (which launch the mask by itself), an empty sum; rows of y that
    are zero, negative, NaN and infinite, and products that are."""
    print("case product times mask", m, n, k, flush=True)
    A = oracle.normal((m, k), 71)
    B = oracle.normal((k, n), 72)
    y = np.maximum(oracle.normal((m, n), 73), 0).astype(F)
    if m * n >= 16:
        y.flat[1], y.flat[2], y.flat[3], y.flat[5] = -0.0, np.nan, np.inf, -1.0
    if k:
        A[0, 0] = np.inf                 # products of row 0 are +-inf or NaN: times 0 they are NaN, as the separate launch gives
    dA, dB, dy = G.dev(A), G.dev(B), G.dev(y)
    dAt, dBt = G.dev(np.ascontiguousarray(A.T)), G.dev(np.ascontiguousarray(B.T))
    views = [(dA, dB), (dA, dBt.t()), (dAt.t(), dB)]
    if k:
        A2 = G.dev(np.repeat(A, 2, axis=1))
        views.append((A2[:, ::2], dB))       # no unit stride: the generic kernel
    for a, b in views:
        plain = G.matmul(a, b)
        want = G.host(G.unary_bwd("relu", dy, plain))
        got = G.host(G.matmul_relu_mask(a, b, dy))
        assert same_bits(got, want)

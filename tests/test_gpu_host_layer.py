"""The C++ front-end (Tensor / Storage / Ctorch_Scheduler / AutoDiff over the HIP launch layer),
driven in-process through ctorch_amd/host/src/capi_host.cpp, against the CPU oracle and the golden
vectors written from the real reference.  The test bodies read like tests/test_oracle_vs_ref.py:
the entry points have the same shape as the ones used for the reference library."""
import os
import subprocess

import numpy as np
import pytest

from support import (ADD, CE, COS, DIV, DOT, MAE, MATMUL, MSE, MUL, NEG, RELU, ROOT, SIGMOID, SIN, SOFTMAX_KERNEL,
                     SUB, TANH, HostLayer, same_bits, ulp_diff)

pytestmark = pytest.mark.gpu
F = np.float32
UNARY = [(NEG, "neg", 0), (RELU, "relu", 0), (SIN, "sin", 2), (COS, "cos", 2), (TANH, "tanh", 2), (SIGMOID, "sigmoid", 2)]


@pytest.fixture(scope="module")
def host():
    return HostLayer()


def close(got, want, max_ulp, what=""):
    got, want = np.asarray(got, F), np.asarray(want, F)
    assert got.shape == want.shape, what
    if max_ulp == 0:
        nan_both = np.isnan(got) & np.isnan(want)
        assert not ((got.view(np.uint32) != want.view(np.uint32)) & ~nan_both).any(), what
    else:
        assert np.array_equal(np.isnan(got), np.isnan(want)), what
        ok = ~np.isnan(want)
        assert ulp_diff(got[ok], want[ok]).max() <= max_ulp, what


def test_forward_operators(oracle, host):
    print("case host forward", flush=True)
    x = oracle.normal((37, 53), 10, 0, 3)
    y = oracle.normal((37, 53), 20, 0, 3)
    for code in (ADD, SUB, MUL, DIV):
        rc, out = host.binary(code, x, y, x.shape)
        assert rc == x.size
        close(out, oracle.binary(code, x, y), 0, code)
    for code, name, ulp in UNARY:
        close(host.unary(code, x), oracle.unary(code, x), ulp, name)
    for which, s in [(0, 5.0), (1, -2.5), (2, 3.0)]:
        close(host.scalar(which, x, s)[1], oracle.scalar(which, x, s), 0, which)
    b = oracle.uniform((53,), 30, 0.5, 2)
    for code in (ADD, SUB, MUL, DIV):      # row broadcast: Add as the reference, the rest by the same convention
        rc, out = host.binary(code, x, b, x.shape)
        assert rc == x.size
        close(out, oracle.binary_rowbcast(code, x, b), 0, ("rowbcast", code))
    rc, out = host.binary(ADD, x, b[:1], x.shape)
    close(out, oracle.add_scalar_tensor(x, b[:1]), 0, "b with one element")
    # error behaviour kept from the reference
    assert host.binary(ADD, b, x, x.shape)[0] == -1            # 1-D on the left: Add throws
    assert host.binary(MATMUL, x, y, (37, 53))[0] == -1        # inner dimensions differ: throws
    assert abs(host.sum(x) - x.astype(np.float64).sum()) <= 1e-5 * np.abs(x).sum()
    for code, fn in [(DOT, oracle.dot), (MSE, oracle.mse), (MAE, oracle.mae)]:
        rc, out = host.binary(code, x, y, ())
        assert rc == 1 and abs(out - fn(x, y)) <= 1e-5 * max(abs(fn(x, y)), np.abs(x * y).sum() if code == DOT else 0)
    for dim in (0, 1):
        assert np.all(np.abs(host.softmax(x, dim) - oracle.softmax(x, dim)) <= 1e-5 * oracle.softmax(x, dim))
    assert np.all(np.abs(host.unary(SOFTMAX_KERNEL, x) - oracle.softmax(x, 1)) <= 1e-5 * oracle.softmax(x, 1))


def test_cross_entropy_target_forms_and_errors(oracle, host):
    print("case host cross entropy", flush=True)
    x = oracle.normal((19, 31), 40, 0, 2)
    idx = oracle.ints((19,), 41, 31)
    oh = np.zeros_like(x)
    oh[np.arange(19), idx.astype(int)] = 1
    want = oracle.ce_onehot(x, oh)
    for t in (oh, idx):
        rc, out = host.binary(CE, x, t, ())
        assert rc == 1 and abs(out - want) <= 1e-5 * want
    rc, out = host.binary(CE, x[0], oh[0], ())
    assert rc == 1 and abs(out - oracle.ce_onehot(x[0], oh[0])) <= 1e-5 * oracle.ce_onehot(x[0], oh[0])
    bad = idx.copy()
    bad[3] = 31
    assert host.binary(CE, x, bad, ())[0] == -2          # empty Tensor, as the reference
    assert host.binary(CE, x, idx[:5], ())[0] == -2      # incompatible shapes: empty Tensor
    # class indices the host never saw (a device computation's result): the range check runs on the device
    host.set_inputs_unseen(True)
    try:
        rc, out = host.binary(CE, x, idx, ())
        assert rc == 1 and abs(out - want) <= 1e-5 * want
        assert host.binary(CE, x, bad, ())[0] == -2
        for wrong in (-1.0, 31.5, np.nan, np.inf, -np.inf, 3e9):
            bad[3] = wrong
            assert host.binary(CE, x, bad, ())[0] == -2
    finally:
        host.set_inputs_unseen(False)
    for wrong in (-1.0, 31.5, np.nan, np.inf, -np.inf, 3e9):            # and those the upload looked at
        bad[3] = wrong
        assert host.binary(CE, x, bad, ())[0] == -2
    # an index is read by truncation, as the reference reads it: 2.9 is class 2, -0.9 class 0
    frac = idx.copy()
    frac[3], frac[4] = 2.9, -0.9
    whole = idx.copy()
    whole[3], whole[4] = 2.0, 0.0
    for unseen in (False, True):
        host.set_inputs_unseen(unseen)
        try:
            assert host.binary(CE, x, frac, ()) == host.binary(CE, x, whole, ())
        finally:
            host.set_inputs_unseen(False)
    # backward: one-hot as the reference; class indices are accepted too (the reference throws)
    wantd = oracle.accumulate0(oracle.ce_bwd_onehot(x, oh, F(0.37)))
    for t in (oh, idx):
        rc, loss, dp = host.grad_loss(CE, x, t, 0.37)
        assert rc == x.size and np.abs(dp - wantd).max() <= 1e-6
    # the loss as the root of backward(): with class indices loss and gradient come from one pass over
    # the logits (the gradient waits in the front-end for backward()), or - switched off - from a
    # forward pass and a backward pass; a second backward() over the same tape recomputes
    want1 = oracle.accumulate0(oracle.ce_bwd_onehot(x, oh, F(1.0)))
    for shape, seed in (((19, 31), 40), ((6, 4096), 44), ((3, 33000), 45)):
        xs = oracle.normal(shape, seed, 0, 2)
        ids = oracle.ints((shape[0],), seed + 1, shape[1])
        ohs = np.zeros_like(xs)
        ohs[np.arange(shape[0]), ids.astype(int)] = 1
        wants = oracle.accumulate0(oracle.ce_bwd_onehot(xs, ohs, F(1.0)))
        got = []
        for one_pass in (True, False):
            host.set_ce_one_pass(one_pass)
            try:
                rc, loss, dp = host.grad_loss(CE, xs, ids, 1.0)
            finally:
                host.set_ce_one_pass(True)
            assert rc == xs.size and np.abs(dp - wants).max() <= 1e-6, (shape, one_pass)
            assert abs(loss - oracle.ce_index(xs, ids)) <= 1e-5 * abs(oracle.ce_index(xs, ids))
            got.append(dp)
        assert np.abs(got[0] - got[1]).max() <= 5e-7, shape
    assert want1.shape == x.shape


def test_matmul_layouts_and_gradients(oracle, host):
    print("case host matmul", flush=True)
    A = oracle.normal((33, 47), 41)
    B = oracle.normal((47, 29), 42)
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    want = oracle.matmul(A, B)
    for got in (host.matmul_t(A, 0, B, 0), host.matmul_t(A, 0, Bt, 1), host.matmul_t(At, 1, B, 0),
                host.matmul_t(At, 1, Bt, 1)):
        assert np.all(np.abs(got - want) <= 2 * bound)
    W = oracle.normal((33, 29), 43)
    rc, da, db = host.grad_binary(MATMUL, A, B, W)
    assert rc == A.size + B.size
    ba = 1e-5 * (np.abs(W).astype(np.float64) @ np.abs(B.T).astype(np.float64))
    bb = 1e-5 * (np.abs(A.T).astype(np.float64) @ np.abs(W).astype(np.float64))
    assert np.all(np.abs(da - oracle.matmul(W, B.T)) <= 2 * ba)
    assert np.all(np.abs(db - oracle.matmul(A.T, W)) <= 2 * bb)


def test_elementwise_gradients_through_the_tape(oracle, host, golden):
    print("case host gradients", flush=True)
    g = golden("backward")
    x, y, w = g["x"], g["y"], g["w"]
    for code, name, ulp in UNARY:
        close(host.grad_unary(code, x, w), g["d_" + name], ulp, name)          # vs the real reference
    for code, name in [(MSE, "mse"), (MAE, "mae")]:
        rc, loss, dp = host.grad_loss(code, x, y, 0.37)
        close(dp, g["d_" + name], 0, name)
    rc, da, db = host.grad_binary(DIV, x, g["yb"], w)
    close(da, g["d_div_a"], 0, "div a")
    close(db, g["d_div_b"], 0, "div b")
    rc, da, db = host.grad_binary(MUL, x, y, w)
    close(da, g["d_mul_a"], 0, "mul a")
    close(db, g["d_mul_b"], 0, "mul b")
    rc, da, db = host.grad_binary(SUB, x, y, w)
    close(da, g["d_sub_a"], 0, "sub a")
    close(db, g["d_sub_b"], 0, "sub b")
    yz = y.copy()
    yz[3, 4] = 0.0
    assert host.grad_binary(DIV, x, yz, w)[0] == -1           # zero divisor: backward throws
    for dim in (0, 1):
        got = host.grad_softmax(x, dim, w)
        want = g["d_softmax_d%d" % dim]
        assert np.abs(got - want).max() <= 1e-5 * np.abs(w).max()
    # row-broadcast operand: column sum by default, the reference's row 0 on request
    b = g["b"]
    rc, da, db = host.grad_binary(ADD, x, b, w)
    close(da, g["d_addrow_a"], 0, "add a")
    assert np.all(np.abs(db - w.astype(np.float64).sum(0)) <= 1e-5 * np.abs(w).sum(0))
    host.set_reference_row0(True)
    try:
        rc, da, db = host.grad_binary(ADD, x, b, w)
        close(db, g["d_addrow_b"], 0, "add b, reference row-0 mode")
    finally:
        host.set_reference_row0(False)
    # the other row-broadcast operators (extensions): gradients against fp64
    for code, dfa, dfb in [(SUB, lambda: w, lambda: -w), (MUL, lambda: w * b, lambda: w * x),
                           (DIV, lambda: w / b, lambda: -w * x / (b.astype(np.float64) ** 2))]:
        rc, da, db = host.grad_binary(code, x, np.abs(b) + F(0.5) if code == DIV else b, w)
        bb = (np.abs(b) + F(0.5)) if code == DIV else b
        x64, w64, b64 = x.astype(np.float64), w.astype(np.float64), bb.astype(np.float64)
        want_a = {SUB: w64, MUL: w64 * b64, DIV: w64 / b64}[code]
        want_b = {SUB: -w64, MUL: w64 * x64, DIV: -w64 * x64 / b64 ** 2}[code]
        assert np.abs(da - want_a).max() <= 1e-5 * np.abs(want_a).max(), code
        assert np.abs(db - want_b.sum(0)).max() <= 1e-5 * np.abs(want_b).sum(0).max(), code


def test_configurations_small(oracle, host, golden):
    print("case host configs", flush=True)
    g = golden("configs")
    s, ga, gb = host.chain(g["chain_a"], g["chain_b"])
    assert abs(s - g["chain_s"]) <= 1e-5 * abs(g["chain_s"])
    close(ga, g["chain_ga"], 0, "chain ga")          # bit-exact against the real reference
    close(gb, g["chain_gb"], 0, "chain gb")
    lab = g["mlp_lab"]
    oh = np.zeros((lab.size, 10), F)
    oh[np.arange(lab.size), lab.astype(int)] = 1
    args = (g["mlp_x"], g["mlp_W1"], g["mlp_b1"], g["mlp_W2"], g["mlp_b2"])
    names = ["loss", "logits", "gW1", "gb1", "gW2", "gb2"]
    host.set_reference_row0(True)
    try:
        got = host.mlp_step(*args, oh)
    finally:
        host.set_reference_row0(False)
    for n, a, b in zip(names, got, [g["mlp_" + n] for n in names]):   # the reference's own numbers
        assert np.abs(a - b).max() <= 1e-4 * max(1.0, np.abs(b).max()), n
    want = oracle.mlp_step(*args, oh, False)                            # column-sum bias gradients
    # each layer as one fused operator: the bits of the three-operator form, in both gradient modes
    for row0 in (False, True):
        host.set_reference_row0(row0)
        try:
            plain = host.mlp_step(*args, oh)
            host.set_fused_layers(True)
            fused = host.mlp_step(*args, oh)
        finally:
            host.set_fused_layers(False)
            host.set_reference_row0(False)
        for n, a, b in zip(names, fused, plain):
            assert same_bits(a, b), (n, row0)
    for target, is_index in ((oh, False), (lab, True)):
        got = host.mlp_step(*args, target, is_index)
        for n, a, b in zip(names, got, want):
            assert np.abs(a - b).max() <= 1e-4 * max(1.0, np.abs(b).max()), (n, is_index)
    X, rv, T = g["expr_X"], g["expr_r"], g["expr_T"]
    R = np.broadcast_to(rv, X.shape).copy()
    Y, mse, mae, gX, gR = host.expr(X, R, T)                           # materialised operand, as the reference
    assert ulp_diff(Y, g["expr_Y"]).max() <= 2
    assert abs(mse - g["expr_mse"]) <= 1e-5 * g["expr_mse"] and abs(mae - g["expr_mae"]) <= 1e-5 * g["expr_mae"]
    assert np.abs(gX - g["expr_gX"]).max() <= 1e-6 * np.abs(g["expr_gX"]).max() + 1e-9
    assert np.abs(gR - g["expr_gR"]).max() <= 1e-6 * np.abs(g["expr_gR"]).max() + 1e-9
    Y2, mse2, mae2, gX2, gr = host.expr(X, rv, T)                      # row vector: broadcast Div + column-sum
    assert same_bits(Y2, Y) and same_bits(gX2, gX)
    assert np.abs(gr - g["expr_gR"].astype(np.float64).sum(0)).max() <= 1e-5 * np.abs(g["expr_gR"]).sum(0).max()


@pytest.mark.parametrize("prog", ["test_scalar_grad", "test_tensor_grad", "test_activation_loss", "test_fused"])
def test_reference_style_programs(prog):
    """C++ programs written like the reference's own test executables (src/tests/test.cpp,
    test_tensor_grad.cpp, test_activation_loss.cpp), on DeviceType::kAMD; exit code 0 = all
    checks passed."""
    print("case host program", prog, flush=True)
    exe = os.path.join(ROOT, "ctorch_amd", "host", "tests", prog + ".bin")
    assert os.path.exists(exe), "build it with make -C ctorch_amd/host"
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(p.stdout[-3000:])
    assert p.returncode == 0


def test_tape_programs_against_the_reference_vectors(oracle, host, golden):
    """Sixty random straight-line programs (values re-used, several gradient contributions per node,
    x (op) x, row-vector operands) through the device tape: the forward value and every input
    gradient must have the bits the real reference produced - the operators are bit-exact and the
    tape adds the contributions in the reference's order; L = sum(...) to the reduction bar."""
    import importlib.util
    import os
    from support import program_inputs, random_program
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden",
                                                                            "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    g = golden("programs")
    host.set_reference_row0(True)
    try:
        for seed in mg.PROGRAM_SEEDS:
            print("case program", seed, flush=True)
            rows, cols = mg.program_shape(seed)
            kinds, ops = random_program(seed)
            xs, w = program_inputs(oracle, seed, kinds, rows, cols)
            rc, y, L, grads = host.program(xs, kinds, ops, w)
            assert rc >= 0, seed
            assert same_bits(y, g["p%d_y" % seed]), seed
            want_L = float(g["p%d_L" % seed])
            assert abs(float(L) - want_L) <= 1e-5 * float(np.abs(y * w).astype(np.float64).sum()) + 1e-30
            for i, got in enumerate(grads):
                assert same_bits(got, g["p%d_g%d" % (seed, i)]), (seed, i)
    finally:
        host.set_reference_row0(False)
    # default mode (column-sum gradients for broadcast row vectors): the mathematics, by the fp64 interpreter
    from support import program_fp64
    for seed in list(mg.PROGRAM_SEEDS)[::3]:
        rows, cols = mg.program_shape(seed)
        kinds, ops = random_program(seed)
        xs, w = program_inputs(oracle, seed, kinds, rows, cols)
        rc, y, L, grads = host.program(xs, kinds, ops, w)
        y64, L64, g64 = program_fp64(xs, kinds, ops, w, row0=False)
        assert rc >= 0 and np.abs(y - y64).max() <= 1e-5 * (1 + np.abs(y64).max())
        for got, want in zip(grads, g64):
            assert np.abs(got - want).max() <= 2e-5 * (1 + np.abs(want).max()), seed


def test_fused_expressions_against_the_reference_vectors(oracle, host, golden, exact_math):
    """The same random programs with every chain of elementwise operators built as ONE fused
    expression (one launch forward, one launch for all gradients): in the reference's gradient mode
    the result and every gradient must still have the reference's bits; in the default mode the
    gradients must agree with the mathematics (a row vector used twice is summed over the rows
    once instead of twice, which rounds differently).  Then the two benchmark chains."""
    import importlib.util
    import os
    from support import program_fp64, program_inputs, random_program
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden",
                                                                            "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    g = golden("programs")
    host.set_fused_expr(True)
    try:
        host.set_reference_row0(True)
        for seed in mg.PROGRAM_SEEDS:
            print("case fused program", seed, flush=True)
            rows, cols = mg.program_shape(seed)
            kinds, ops = random_program(seed)
            xs, w = program_inputs(oracle, seed, kinds, rows, cols)
            rc, y, L, grads = host.program(xs, kinds, ops, w)
            assert rc >= 0, seed
            assert same_bits(y, g["p%d_y" % seed]), seed
            for i, got in enumerate(grads):
                assert same_bits(got, g["p%d_g%d" % (seed, i)]), (seed, i)
        host.set_reference_row0(False)
        for seed in list(mg.PROGRAM_SEEDS)[::3]:
            rows, cols = mg.program_shape(seed)
            kinds, ops = random_program(seed)
            xs, w = program_inputs(oracle, seed, kinds, rows, cols)
            rc, y, L, grads = host.program(xs, kinds, ops, w)
            y64, L64, g64 = program_fp64(xs, kinds, ops, w, row0=False)
            assert rc >= 0 and np.abs(y - y64).max() <= 1e-5 * (1 + np.abs(y64).max())
            for got, want in zip(grads, g64):
                assert np.abs(got - want).max() <= 2e-5 * (1 + np.abs(want).max()), seed
        # config 1 and config 5, fused, against the operator-by-operator front-end
        c = golden("configs")
        s1, ga1, gb1 = host.chain(c["chain_a"], c["chain_b"])
        X, rv, T = c["expr_X"], c["expr_r"], c["expr_T"]
        fused5 = host.expr(X, rv, T)
        host.set_fused_expr(False)
        s0, ga0, gb0 = host.chain(c["chain_a"], c["chain_b"])
        assert s1 == s0 and same_bits(ga1, ga0) and same_bits(gb1, gb0)
        assert same_bits(ga1, c["chain_ga"]) and same_bits(gb1, c["chain_gb"])     # the reference's bits
        plain5 = host.expr(X, rv, T)
        assert same_bits(fused5[0], plain5[0]) and fused5[1] == plain5[1] and fused5[2] == plain5[2]
        assert same_bits(fused5[3], plain5[3])                                       # gX: same order of the four terms
        assert np.abs(fused5[4] - plain5[4]).max() <= 1e-5 * np.abs(plain5[4]).max()  # gr: one column sum instead of ... one
        # a zero divisor is refused in backward, as by the tape's own Div gradient
        host.set_fused_expr(True)
        rz = rv.copy()
        rz[3] = 0.0
        bad = host.expr(X, rz, T, expect_failure=True)
        assert bad is None
    finally:
        host.set_fused_expr(False)
        host.set_reference_row0(False)


def test_fused_programs_in_the_default_math_mode_against_the_mathematics(oracle, host):
    """The random tape programs as fused expressions in the default math mode (single-precision sine /
    cosine / sigmoid, negations under a sine or cosine folded away by the expression compiler): value
    and every gradient against the fp64 interpreter, as the exact mode is held to."""
    import importlib.util
    import os
    from ctorch_amd import capi
    from support import program_fp64, program_inputs, random_program
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden",
                                                                            "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    assert capi.load().ctamd_math_mode() == 0
    host.set_fused_expr(True)
    try:
        for seed in mg.PROGRAM_SEEDS:
            print("case fused program, default mode", seed, flush=True)
            rows, cols = mg.program_shape(seed)
            kinds, ops = random_program(seed)
            xs, w = program_inputs(oracle, seed, kinds, rows, cols)
            rc, y, L, grads = host.program(xs, kinds, ops, w)
            y64, L64, g64 = program_fp64(xs, kinds, ops, w, row0=False)
            assert rc >= 0 and np.abs(y - y64).max() <= 1e-5 * (1 + np.abs(y64).max()), seed
            for got, want in zip(grads, g64):
                assert np.abs(got - want).max() <= 2e-5 * (1 + np.abs(want).max()), seed
    finally:
        host.set_fused_expr(False)


def test_fused_expression_in_the_default_mode_drops_the_negations_under_sine_and_cosine(oracle, host, golden):
    """Configuration 5 as one fused expression in the default math mode: the expression compiler forms
    cos(-X) from X (and sin(-X) in the gradient program as -sin(X)), so both programs are shorter than
    the exact mode's, which keeps the negations where glibc's quadrant rounding could tell -x from x;
    value and gradients stay within the default mode's bound of the exact mode's."""
    from ctorch_amd import capi
    print("case host fused expression, default mode", flush=True)
    lib = capi.load()
    assert lib.ctamd_math_mode() == 0
    c = golden("configs")
    X, rv, T = c["expr_X"], c["expr_r"], c["expr_T"]
    host.set_fused_expr(True)
    try:
        y, mse, mae, gX, gr = host.expr(X, rv, T)
        fast = host.last_expr_stats()
        assert lib.ctamd_set_math_mode(1) == 0
        try:
            ye, msee, maee, gXe, gre = host.expr(X, rv, T)
            exact = host.last_expr_stats()
        finally:
            assert lib.ctamd_set_math_mode(0) == 0
    finally:
        host.set_fused_expr(False)
    print("  program sizes (forward, slots, backward, slots): default", fast, "exact", exact)
    assert fast[0] == exact[0] - 1 and 0 < fast[2] < exact[2]
    assert np.abs(y - ye).max() <= 8e-7
    assert abs(float(mse) - float(msee)) <= 1e-5 * float(msee) and abs(float(mae) - float(maee)) <= 1e-5 * float(maee)
    assert np.abs(gX - gXe).max() <= 1e-5 * np.abs(gXe).max()
    assert np.abs(gr - gre).max() <= 1e-5 * np.abs(gre).max()


def test_comparison_operators(oracle, host):
    """Tensor (cmp) Tensor and Tensor (cmp) float through the front-end: DType::kBool results equal
    to the oracle's; tensors of different shapes throw (src/Tensor.cpp:1124-1126)."""
    print("case host compare", flush=True)
    a = oracle.normal((7, 33), 72, 0, 1)
    b = oracle.normal((7, 33), 73, 0, 1)
    b[2] = a[2]
    for cmp in range(6):
        assert np.array_equal(host.compare(cmp, a, b), oracle.compare(cmp, a, b)), cmp
        assert np.array_equal(host.compare(cmp, a, None, 0.1), oracle.compare(cmp, a, None, 0.1)), cmp
    assert host.compare(0, a, b[:, :32].copy()) == -1


def test_tensors_that_are_not_fp32(oracle, host, golden):
    """Tensor::to(dtype), zero / ones, tensor (+ * /) float and the double softmax through the front-end,
    against the reference's vectors (bytes equal; the softmax to the bound of test_gpu_typed.py);
    backward() over a typed tensor throws, as it does in the reference."""
    from support import typed_cases
    from test_gpu_typed import check_softmax
    print("case host typed", flush=True)
    g = golden("typed")
    for name, a, dt, steps in typed_cases(oracle):
        rc, got = host.typed(a, dt, steps)
        assert rc == a.size, (name, rc)
        if name.startswith("softmax"):
            x = oracle.typed(a, dt, steps[:-1])
            check_softmax(got, g[name], x, 0 if x.ndim == 1 else int(steps[-1][1]))
        else:
            assert np.array_equal(got.view(np.uint8), g[name].view(np.uint8)), name
    x = oracle.normal((2, 3), 5, 0, 10)
    for dt in (1, 2, 3):
        for steps in ([(0, 5.0)], [(1, 3.0)], [(1, 3.0), (0, 5.0)], [(2, 4.0)]):
            assert host.typed_grad(x, dt, steps)[0] == -1, (dt, steps)
    rc, code, raw = host.typed_grad(x, 0, [(1, 3.0), (0, 5.0)])
    assert rc == 6 and code == 0 and np.array_equal(raw.view(np.float32)[:6], np.full(6, 3.0, np.float32))
    # an integer division the reference's process would not survive is an exception here
    assert host.typed(x, 2, [(2, 0.5)])[0] == -1


def test_fused_expression_in_a_recorded_step(oracle, host, exact_math):
    """A fused expression, its losses and its backward recorded into a HIP graph: the first replay
    reproduces the eager step bit for bit, a replay after the staged input was overwritten equals
    the eager step on the new input."""
    print("case fused expr recorded", flush=True)
    rows, cols = 64, 256
    X1 = oracle.uniform((rows, cols), 901, -2, 2)
    X2 = oracle.uniform((rows, cols), 902, -2, 2)
    r = oracle.uniform((cols,), 903, 0.5, 2)
    T = oracle.normal((rows, cols), 904)
    rc, y1, gx1, y2, gx2 = host.expr_graph(X1, X2, r, T)
    assert rc == rows * cols, rc
    host.set_fused_expr(True)
    try:
        e1 = host.expr(X1, r, T)
        e2 = host.expr(X2, r, T)
    finally:
        host.set_fused_expr(False)
    assert same_bits(y1, e1[0]) and same_bits(gx1, e1[3])
    assert same_bits(y2, e2[0]) and same_bits(gx2, e2[3])
    assert not same_bits(y1, y2)


def test_fused_against_unfused_on_more_programs(oracle, host, exact_math):
    """A hundred further random programs (longer, more inputs, shapes with rows that are not a
    multiple of four elements, so the 32-bit access path runs too, and a tensor large enough for
    several passes per block): the fused expression against the operator-by-operator tape on the
    device in the reference's gradient mode - bit for bit for the result and for every full-shape
    input; a row vector that is also combined with other row vectors outside the expression gets its
    contributions in another order (the expression hands the tape one sum), so it is held to 1e-5."""
    from support import program_inputs, random_program
    shapes = [(5, 7), (6, 8), (33, 20), (40, 36), (9, 130), (520, 1028)]
    host.set_reference_row0(True)
    try:
        for seed in range(1000, 1100):
            rows, cols = shapes[seed % len(shapes)] if seed % 25 else shapes[-1]
            kinds, ops = random_program(seed, n_in=3 + seed % 3, n_ops=10 + seed % 15)
            xs, w = program_inputs(oracle, seed, kinds, rows, cols)
            host.set_fused_expr(False)
            rc0, y0, L0, g0 = host.program(xs, kinds, ops, w)
            host.set_fused_expr(True)
            rc1, y1, L1, g1 = host.program(xs, kinds, ops, w)
            assert rc0 >= 0 and rc1 == rc0, seed
            assert same_bits(y1, y0), seed
            for i, (a, b) in enumerate(zip(g1, g0)):
                if kinds[i] == 0:
                    assert same_bits(a, b), (seed, i)
                else:
                    assert np.all(np.abs(a - b) <= 1e-5 * (np.abs(b) + np.abs(b).max())), (seed, i)
    finally:
        host.set_fused_expr(False)
        host.set_reference_row0(False)


def test_recorded_steps_stay_ordered_and_keep_no_stale_state(oracle, host):
    """Graphs replay on one stream: two graphs that share the device scratch and a tensor, replayed
    alternately with new inputs and no host wait, give the eager sums of the last input.  item() of a
    one-element parameter after an in-place SGD step reads the device.  A thread whose first
    backward() happens inside a recording still seeds an eager backward() with 1.  A DeviceGraph
    whose recording failed can record again."""
    print("case graph hardening", flush=True)
    X = oracle.uniform((1 << 20,), 611, -1, 1)
    X2 = oracle.uniform((1 << 20,), 612, -1, 1)
    rc, out = host.graph_hardening(X, X2)
    assert rc == 0
    assert out[0] == out[2] and out[1] == out[3]
    assert out[4] == np.float32(1.5)
    assert out[5] == np.float32(0.0) + (X[0] + X[0])      # d(sum x*x)/dx = x + x by the product rule, added to the tape's zero
    assert out[6] == 1.0


def test_kept_cross_entropy_gradients_are_capped(oracle, host, exact_math):
    """The gradient that the one-pass CrossEntropy keeps for backward() is bounded in bytes: when the
    cap holds only one of two, the older is dropped and recomputed from its logits; below the size
    of one, none is kept and backward() works from the forward pass's row statistics.  The first two
    agree bit for bit, the third to 2e-7, and all are the oracle's gradient to a few ulp."""
    print("case ce kept cap", flush=True)
    rows, cols = 96, 1000
    x1 = oracle.normal((rows, cols), 621, 0, 2)
    x2 = oracle.normal((rows, cols), 622, 0, 2)
    lab = oracle.ints((rows,), 623, cols)
    rc, g1, g2 = host.ce_kept_cap(x1, x2, lab)
    assert rc == 0, rc
    for x, g in ((x1, g1), (x2, g2)):
        want = oracle.ce_bwd_index(x, lab, 1.0)
        # the row's sum of exponentials is added in another order than the oracle's: a few ulp of each element
        rel = np.abs(g - want) / np.maximum(np.abs(want), 1e-30)
        print(f"  largest element-relative difference from the oracle {rel.max():.2e}")
        assert rel.max() <= 5e-6      # the oracle adds 1000 exponentials in order, in single precision


def test_a_gradient_read_from_the_tape_is_read_only_while_shared(oracle, host):
    """grad() hands out the tape's bytes instead of a copy (the reference copies): writing them in place
    through the front-end (fill, copy_into, sgd_step) throws while the tape still holds them."""
    print("case shared gradient read-only", flush=True)
    x = oracle.uniform((4096,), 631, -1, 1)
    import ctypes as C
    host.cdll.cth_shared_grad_is_readonly.restype = C.c_long
    assert host.cdll.cth_shared_grad_is_readonly(x.ctypes.data_as(C.POINTER(C.c_float)), C.c_long(x.size)) == 0


@pytest.mark.parametrize("batch", [8, 256, 512, 513, 4096])
def test_bias_gradient_comes_with_the_weight_gradient(oracle, host, batch):
    """A fused layer whose bias wants its gradient gets it from the call that forms the weight
    gradient (column sums of the layer's output gradient beside x^T . dz).  The gradients are the
    bits of the separate launches at every batch size; up to 512 rows (the longest K the one-launch
    small-product kernel takes) the column sums ride in the product's own launch, and a step then
    counts two operator launches fewer."""
    print("case bias gradient with the weight gradient", batch, flush=True)
    I, H, Cn = 784, 256, 10
    x = oracle.uniform((batch, I), 651, 0, 1)
    W1, b1 = oracle.uniform((I, H), 652, -0.05, 0.05), oracle.uniform((H,), 653, -0.05, 0.05)
    W2, b2 = oracle.uniform((H, Cn), 654, -0.1, 0.1), oracle.uniform((Cn,), 655, -0.1, 0.1)
    labels = oracle.ints((batch,), 656, Cn)
    host.set_fused_layers(True)
    try:
        host.set_bias_grad_with_weight_grad(False)
        apart = host.mlp_step(x, W1, b1, W2, b2, labels, True)
        _, launches_apart = host.time_mlp(x, W1, b1, W2, b2, labels)
        host.set_bias_grad_with_weight_grad(True)
        together = host.mlp_step(x, W1, b1, W2, b2, labels, True)
        _, launches_together = host.time_mlp(x, W1, b1, W2, b2, labels)
    finally:
        host.set_bias_grad_with_weight_grad(True)
        host.set_fused_layers(False)
    for name, a, b in zip(["loss", "logits", "gW1", "gb1", "gW2", "gb2"], together, apart):
        assert same_bits(a, b), name
    print(f"  operator launches per step: {launches_together} together, {launches_apart} apart")
    assert launches_together == launches_apart - (2 if batch <= 512 else 0)


@pytest.mark.parametrize("batch", [8, 300, 4096])
def test_relu_mask_rides_in_the_products_of_backward(oracle, host, batch):
    """The gradient of a ReLU layer's output, when one product alone reads that output, is formed
    already multiplied by the layer's mask (one launch fewer per hidden layer).  A three-layer
    network: the six parameter gradients and the gradients of both hidden activations (which the
    tape then has to form on request) equal the ones of the separate mask launch bit for bit, after
    one backward pass and after two passes over the same tape; and backward launches fewer kernels."""
    print("case relu mask in the product", batch, flush=True)
    import ctypes as C
    I, H1, H2, Cn = 200, 96, 72, 10
    x = oracle.uniform((batch, I), 641, 0, 1)
    W1, b1 = oracle.uniform((I, H1), 642, -0.1, 0.1), oracle.uniform((H1,), 643, -0.1, 0.1)
    W2, b2 = oracle.uniform((H1, H2), 644, -0.15, 0.15), oracle.uniform((H2,), 645, -0.1, 0.1)
    W3, b3 = oracle.uniform((H2, Cn), 646, -0.2, 0.2), oracle.uniform((Cn,), 647, -0.1, 0.1)
    labels = oracle.ints((batch,), 648, Cn)
    FP = C.POINTER(C.c_float)
    fp = lambda a: a.ctypes.data_as(FP)
    L = C.c_long
    out = (C.c_double * 2)()
    host.cdll.cth_relu_mask_fusion.restype = C.c_long
    rc = host.cdll.cth_relu_mask_fusion(fp(x), L(batch), L(I), fp(W1), fp(b1), L(H1), fp(W2), fp(b2), L(H2), fp(W3), fp(b3),
                                        L(Cn), fp(labels), out)
    assert rc == 0, rc
    print(f"  kernels launched by backward: {int(out[0])} with the mask in the products, {int(out[1])} without")
    assert out[0] == out[1] - 2


@pytest.mark.parametrize("batch", [8, 300, 4096])
def test_the_one_pass_head_against_the_two_operator_form(oracle, host, batch):
    """Tensor::linear_cross_entropy (logits, loss and the gradients of the last layer formed in one
    pass over the hidden activations) against x.linear(W, b).cross_entropy(labels) in a three-layer
    network: loss, logits, the six parameter gradients and the gradients of both hidden activations
    (the second of which the one pass leaves at the ReLU layer's pre-activation, so the tape forms it on
    request) within the MatMul bound - the head adds its products in another order - for the loss as
    root and for a scaled root (the kept gradient of the logits rescaled); two passes over one tape give
    the head's inputs exactly twice one pass's gradients; and a step is three operator launches shorter."""
    print("case one-pass head", batch, flush=True)
    I, H1, H2, Cn = 200, 96, 72, 10
    x = oracle.uniform((batch, I), 741, 0, 1)
    W1, b1 = oracle.uniform((I, H1), 742, -0.1, 0.1), oracle.uniform((H1,), 743, -0.1, 0.1)
    W2, b2 = oracle.uniform((H1, H2), 744, -0.15, 0.15), oracle.uniform((H2,), 745, -0.1, 0.1)
    W3, b3 = oracle.uniform((H2, Cn), 746, -0.2, 0.2), oracle.uniform((Cn,), 747, -0.1, 0.1)
    labels = oracle.ints((batch,), 748, Cn)
    rc, worst, with_head, without = host.head_fusion(x, W1, b1, W2, b2, W3, b3, labels, 2e-5)
    print(f"  worst difference / largest magnitude {worst:.2e}; operator launches of a step: {int(with_head)} with the head, {int(without)} without")
    assert rc == 0, (rc, worst)
    assert with_head <= without - 3


def test_mlp_step_with_the_one_pass_head_against_the_oracle(oracle, host, golden):
    """configs[2]'s step with fused layers and the one-pass head: loss, logits and the four gradients
    against the CPU oracle at the bar of the other forms of the step."""
    print("case mlp step one-pass head", flush=True)
    g = golden("configs")
    lab = g["mlp_lab"]
    oh = np.zeros((lab.size, 10), F)
    oh[np.arange(lab.size), lab.astype(int)] = 1
    args = (g["mlp_x"], g["mlp_W1"], g["mlp_b1"], g["mlp_W2"], g["mlp_b2"])
    names = ["loss", "logits", "gW1", "gb1", "gW2", "gb2"]
    want = oracle.mlp_step(*args, oh, False)
    host.set_fused_layers(True)
    host.set_fused_head(True)
    try:
        got = host.mlp_step(*args, lab, True)
    finally:
        host.set_fused_head(False)
        host.set_fused_layers(False)
    for n, a, b in zip(names, got, want):
        assert np.abs(a - b).max() <= 1e-4 * max(1.0, np.abs(b).max()), n


def test_class_indices_seen_at_upload_or_checked_on_the_device(oracle, host, golden):
    """A step's class indices come from the host (the upload looked at them: nothing to wait for, a bad
    one refused before anything is computed) or from the device (the loss kernel's flag is read): the
    same results bit for bit, the same refusal, with the one-pass head and without."""
    print("case class indices seen / unseen", flush=True)
    import ctypes as C
    g = golden("configs")
    args = (g["mlp_x"], g["mlp_W1"], g["mlp_b1"], g["mlp_W2"], g["mlp_b2"])
    lab = g["mlp_lab"]
    bad = lab.copy()
    bad[5] = 10.0

    def refused(labels):
        x, W1, b1, W2, b2, t = (np.ascontiguousarray(a, dtype=np.float32) for a in args + (labels,))
        FP = C.POINTER(C.c_float)
        fp = lambda a: a.ctypes.data_as(FP)
        L = C.c_long
        outs = [np.empty(n, np.float32) for n in (1, x.shape[0] * 10, W1.size, b1.size, W2.size, b2.size)]
        host.cdll.cth_mlp_step.restype = C.c_long
        rc = host.cdll.cth_mlp_step(fp(x), L(x.shape[0]), L(x.shape[1]), fp(W1), fp(b1), L(W1.shape[1]), fp(W2), fp(b2), L(10), fp(t),
                                    *(fp(o) for o in outs), C.c_int(1))
        return rc < 0

    host.set_fused_layers(True)
    try:
        for head in (False, True):
            host.set_fused_head(head)
            seen = host.mlp_step(*args, lab, True)
            assert refused(bad)
            host.set_inputs_unseen(True)
            try:
                unseen = host.mlp_step(*args, lab, True)
                assert refused(bad)
            finally:
                host.set_inputs_unseen(False)
            for a, b in zip(seen, unseen):
                assert same_bits(np.asarray(a), np.asarray(b)), head
    finally:
        host.set_fused_head(False)
        host.set_fused_layers(False)


def test_reading_a_gradient_the_tape_holds_at_a_pre_activation(oracle, host):
    """The gradient of a hidden ReLU layer's output, which the tape keeps multiplied by the layer's mask:
    formed once on the first read, gone with the consumer's gradient when that is cleared, and back
    with the next pass over the tape."""
    print("case premasked gradient reads", flush=True)
    import ctypes as C
    B, I, H, Cn = 64, 40, 32, 10
    x = oracle.uniform((B, I), 841, 0, 1)
    W1, b1 = oracle.uniform((I, H), 842, -0.3, 0.3), oracle.uniform((H,), 843, -0.1, 0.1)
    W2, b2 = oracle.uniform((H, Cn), 844, -0.3, 0.3), oracle.uniform((Cn,), 845, -0.1, 0.1)
    labels = oracle.ints((B,), 846, Cn)
    FP = C.POINTER(C.c_float)
    fp = lambda a: np.ascontiguousarray(a, dtype=np.float32).ctypes.data_as(FP)
    L = C.c_long
    host.cdll.cth_premasked_grad_reads.restype = C.c_long
    rc = host.cdll.cth_premasked_grad_reads(fp(x), L(B), L(I), fp(W1), fp(b1), L(H), fp(W2), fp(b2), L(Cn), fp(labels))
    assert rc == 0, rc

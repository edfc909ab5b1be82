"""Fused elementwise expressions (ctamd_expr_run_f32) through the C ABI: random programs against the
CPU oracle's interpreter bit for bit, the config-5 expression against the operator-by-operator
launches, shapes that take the 32-bit access path, and the launcher's refusal of bad programs."""
import numpy as np
import pytest

import gpu_support as G
from support import EX, f32, random_slot_program, same_bits

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(autouse=True)
def _exact_unless_asked(request):
    """The bit-for-bit comparisons below hold in the library's exact mode; tests named *fast_mode* run in
    the default single-precision one."""
    if "fast_mode" in request.node.name:
        yield
        return
    prev = G.set_math_mode(G.MATH_EXACT)
    yield
    G.set_math_mode(prev)


def same_bits_or_both_nan(a, b):
    """Bit equality, except that where both are NaN any NaN will do (x86 and the GPU give the
    invalid-operation NaN opposite signs)."""
    a, b = f32(a), f32(b)
    nan = np.isnan(a) & np.isnan(b)
    return a.shape == b.shape and np.array_equal(np.where(nan, 0, a.view(np.uint32)), np.where(nan, 0, b.view(np.uint32)))


def inputs_for(oracle, seed, n_full, n_row, rows, cols):
    xs = [oracle.uniform((rows, cols), seed * 10 + k, -2, 2) for k in range(n_full)]
    xs += [oracle.uniform((cols,), seed * 10 + 5 + k, 0.5, 2) for k in range(n_row)]
    return xs


@pytest.mark.parametrize("seed", range(24))
def test_random_programs_against_the_oracle_interpreter(oracle, seed):
    print("case expr program", seed, flush=True)
    n_full, n_row = 1 + seed % 3, seed % 3
    prog = random_slot_program(seed, n_full, n_row, n_ops=10 + seed, n_out=1 + seed % 3, slots=4 + seed)
    # aligned rows (128-bit accesses), ragged rows (32-bit accesses), more than one pass per block
    for rows, cols in ((16, 64), (7, 33), (300, 1028)):
        xs = inputs_for(oracle, seed, n_full, n_row, rows, cols)
        want, want_status = oracle.expr_run(prog, xs, 1 + seed % 3, rows, cols)
        got, status = G.expr_run(prog, [G.dev(x) for x in xs], 1 + seed % 3, rows, cols)
        assert status == want_status
        for k, (g, w) in enumerate(zip(got, want)):
            assert same_bits_or_both_nan(G.host(g), w), (seed, rows, cols, k)


def config5_program():
    """Y = sigmoid(X / r) - tanh(X) * sin(X) + cos(-X); X full (input 0), r a row vector (input 1)."""
    E = EX
    return [(E["LOAD_FULL"], 0, 0, 0, 0.0), (E["LOAD_ROW"], 1, 1, 0, 0.0),
            (E["DIV"], 2, 0, 1, 0.0), (E["SIGMOID"], 2, 2, 0, 0.0),
            (E["TANH"], 3, 0, 0, 0.0), (E["SIN"], 4, 0, 0, 0.0), (E["MUL"], 3, 3, 4, 0.0),
            (E["SUB"], 2, 2, 3, 0.0), (E["NEG"], 3, 0, 0, 0.0), (E["COS"], 3, 3, 0, 0.0),
            (E["ADD"], 2, 2, 3, 0.0), (E["STORE"], 0, 2, 0, 0.0)]


@pytest.mark.parametrize("rows,cols", [(64, 256), (1024, 4096), (33, 100)])
def test_config5_expression_equals_the_nine_launches(oracle, rows, cols):
    print("case expr config5", rows, cols, flush=True)
    X = oracle.uniform((rows, cols), 501, -2, 2)
    r = oracle.uniform((cols,), 502, 0.5, 2)
    dX, dr = G.dev(X), G.dev(r)
    (Y,), _ = G.expr_run(config5_program(), [dX, dr], 1, rows, cols)
    q = G.rowbcast("div", dX, dr)
    s = G.unary("sigmoid", q)
    m = G.binary("mul", G.unary("tanh", dX), G.unary("sin", dX))
    want = G.binary("add", G.binary("sub", s, m), G.unary("cos", G.unary("neg", dX)))
    assert same_bits(G.host(Y), G.host(want))
    if rows * cols <= 1 << 16:
        (cpu,), _ = oracle.expr_run(config5_program(), [X, r], 1, rows, cols)
        assert same_bits(G.host(Y), cpu)


def test_special_values_and_the_divisor_check(oracle):
    print("case expr specials", flush=True)
    E = EX
    x = f32([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 1e-8, -1e-8, 3e38, 1e-40, 200.0, -200.0, 1e5, 1e9, 0.5, 88.8]).reshape(2, 8)
    prog = [(E["LOAD_FULL"], 0, 0, 0, 0.0)]
    for k, op in enumerate(("NEG", "RELU", "SIGMOID", "TANH", "SIN", "COS")):
        prog += [(E[op], 1, 0, 0, 0.0), (E["STORE"], k, 1, 0, 0.0)]
    prog += [(E["RELUMUL"], 1, 0, 0, 0.0), (E["STORE_ZP"], 6, 1, 0, 0.0), (E["DIVCHK"], 0, 0, 0, 0.0)]
    want, want_status = oracle.expr_run(prog, [x], 7, 2, 8)
    got, status = G.expr_run(prog, [G.dev(x)], 7, 2, 8)
    assert status == want_status == 1                     # zeros and 1e-8 are below FLT_EPSILON
    for k, (g, w) in enumerate(zip(got, want)):
        assert same_bits_or_both_nan(G.host(g), w), k
    # no small divisor: the status word stays clear
    _, status = G.expr_run(prog, [G.dev(np.abs(x) + F(1))], 7, 2, 8)
    assert status == 0


def test_malformed_programs_are_refused(oracle):
    print("case expr refusals", flush=True)
    E = EX
    x = G.dev(oracle.uniform((4, 8), 1, -1, 1))
    bad = [
        [(E["ADD"], 0, 1, 2, 0.0)],                                        # reads slots nobody wrote
        [(E["LOAD_FULL"], 0, 3, 0, 0.0)],                                  # input 3 of 1
        [(E["LOAD_FULL"], 0, 0, 0, 0.0), (E["STORE"], 5, 0, 0, 0.0)],      # output 5 of 1
        [(E["LOAD_FULL"], 40, 0, 0, 0.0)],                                 # slot out of range
        [(99, 0, 0, 0, 0.0)],                                              # unknown operator
    ]
    for prog in bad:
        rc = -5 if prog[0][1] == 40 else -1
        G.expr_run(prog, [x], 1, 4, 8, expect=rc)
    G.expr_run([(E["LOAD_FULL"], 0, 0, 0, 0.0)] * 161, [x], 1, 4, 8, expect=-5)   # too long
    outs, _ = G.expr_run([], [x], 1, 4, 8)                                        # empty: nothing happens
    assert not G.host(outs[0]).any()


def test_fast_mode_transcendentals_within_2_ulp_of_the_oracle(oracle):
    """The default mode evaluates the transcendental operators in single precision: sin / cos within
    2 ulp of the oracle's glibc calls over a sweep of the argument range (histograms printed); sigmoid,
    the reference's formula on an exponential within 1 ulp and a reciprocal within 1 ulp, within 4 ulp
    of the oracle's; tanh - the reference's (e^x - e^-x) / (e^x + e^-x) loses its digits near zero, as
    does the 1 - 2 / (e^2|x| + 1) used here - within 2 ulp for |x| >= 1 and 2.5e-7 absolute below."""
    print("case expr fast mode ulp", flush=True)
    assert G.lib().ctamd_math_mode() == G.MATH_FAST
    E = EX
    from support import ulp_diff
    u = np.arange(0, 1 << 32, 4099, dtype=np.uint64).astype(np.uint32).view(F)
    x = u[np.isfinite(u)]
    x = np.concatenate([x[np.abs(x) < 200.0], oracle.uniform((200000,), 7, -120, 120), oracle.normal((200000,), 8, 0, 2)])
    x = x[: (x.size // 1024) * 1024].reshape(-1, 1024)
    prog = [(E["LOAD_FULL"], 0, 0, 0, 0.0)]
    for k, op in enumerate(("SIN", "COS", "SIGMOID", "TANH")):
        prog += [(E[op], 1, 0, 0, 0.0), (E["STORE"], k, 1, 0, 0.0)]
    got, _ = G.expr_run(prog, [G.dev(x)], 4, x.shape[0], x.shape[1])
    want, _ = oracle.expr_run(prog, [x], 4, x.shape[0], x.shape[1])
    for k, name in enumerate(("sin", "cos", "sigmoid", "tanh")):
        g, w = G.host(got[k]).reshape(-1), want[k].reshape(-1)
        ok = np.isfinite(w) & (np.abs(w) >= F(2.0 ** -126))
        if name == "tanh":
            big = ok & (np.abs(x.reshape(-1)) >= 1.0)
            d = ulp_diff(g[big], w[big])
            small = np.isfinite(w) & ~big
            print(f"  tanh: |x| >= 1 ulp histogram { {int(v): int((d == v).sum()) for v in np.unique(d)} }; below: max abs error {np.abs(g[small] - w[small]).max():.2e}")
            assert d.max() <= 2 and np.abs(g[small] - w[small]).max() <= 2.5e-7
        else:
            d = ulp_diff(g[ok], w[ok])
            print(f"  {name}: ulp histogram { {int(v): int((d == v).sum()) for v in np.unique(d)} }")
            # 1 / (1 + e): the sum is rounded where floats are up to four times as far apart as at
            # the quotient, so one ulp of the exponential can move the result by four
            assert d.max() <= (4 if name == "sigmoid" else 2), name
        assert np.array_equal(np.isnan(g), np.isnan(w)), name


@pytest.mark.parametrize("rows,cols", [(64, 256), (33, 100)])
def test_fast_mode_config5_expression_against_the_oracle(oracle, rows, cols):
    print("case expr config5 fast mode", rows, cols, flush=True)
    X = oracle.uniform((rows, cols), 501, -2, 2)
    r = oracle.uniform((cols,), 502, 0.5, 2)
    (Y,), _ = G.expr_run(config5_program(), [G.dev(X), G.dev(r)], 1, rows, cols)
    (cpu,), _ = oracle.expr_run(config5_program(), [X, r], 1, rows, cols)
    # three terms of size <= 1 each, every one within 2 ulp (2.5e-7 absolute for the tanh factor)
    assert np.abs(G.host(Y) - cpu).max() <= 8e-7

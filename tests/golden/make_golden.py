"""Writes the golden vectors under tests/golden/ by running the REAL reference library
(oracle/_ref/libctorch_ref.so, built by oracle/Makefile from the mounted reference sources) on
inputs from this repository's seeded generator.  Run only where the reference is mounted:

    make -C oracle && python tests/golden/make_golden.py

Each .npz holds inputs and the reference's outputs, nothing else.  The tests read them with
numpy.load(allow_pickle=False).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from support import (ADD, CE, COS, DIV, DOT, MAE, MATMUL, MSE, MUL, NEG, RELU, SIGMOID, SIN,  # noqa: E402
                     SOFTMAX_KERNEL, SUB, TANH, Oracle, Reference)

SPECIAL = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 1e-38, -1e-38,
                    88.8, -88.8, 100.0, -100.0, 1.0, -1.0, 0.5, -0.5, 1e-3, -1e-3, 1e-6, 20.0, -20.0,
                    3.14159274, 1.57079637, 6.28318548, 1e4, -1e4, 1e7, 1e22, 87.3, -87.3, 103.9],
                   np.float32)


PROGRAM_SEEDS = range(60)


def program_shape(seed):
    return (6, 8) if seed < 45 else (21, 36)


def programs():
    """Random straight-line programs through the reference's tape (support.random_program): the last
    value, L and the gradients of every input, as the reference computes them."""
    from support import program_inputs, random_program
    o = Oracle()
    r = Reference()
    g = {}
    for seed in PROGRAM_SEEDS:
        rows, cols = program_shape(seed)
        kinds, ops = random_program(seed)
        xs, w = program_inputs(o, seed, kinds, rows, cols)
        rc, y, L, grads = r.program(xs, kinds, ops, w)
        assert rc >= 0, seed
        g["p%d_kinds" % seed] = np.array(kinds, np.int32)
        g["p%d_ops" % seed] = np.array(ops, np.int32)
        g["p%d_y" % seed], g["p%d_L" % seed] = y, L
        for i, t in enumerate(grads):
            g["p%d_g%d" % (seed, i)] = t
    np.savez_compressed(os.path.join(HERE, "programs.npz"), **g)


def mnist():
    """The MNIST demo's path: loader, accuracy, the training loop over the reference library, and
    the printed results of the demo program's own main() on the synthetic data set."""
    import contextlib
    import io
    import re
    import tempfile
    from support import write_mnist_dir
    o = Oracle()
    r = Reference()
    g = {}
    with tempfile.TemporaryDirectory() as d:
        tr_i, tr_l, te_i, te_l = write_mnist_dir(d)
        images, labels = r.mnist_load(d, True)
        g["loader_first_rows"] = images[:4]
        g["loader_labels"] = labels[:64]
        # the demo program's own main(), its stdout captured
        sys.stdout.flush()
        saved = os.dup(1)
        with tempfile.TemporaryFile() as cap:
            os.dup2(cap.fileno(), 1)
            try:
                rc = r.mnist_main_in(d)
            finally:
                sys.stdout.flush()
                os.dup2(saved, 1)
                os.close(saved)
            cap.seek(0)
            text = cap.read().decode("utf-8", "replace")
        assert rc == 0
        g["demo_epoch_losses"] = np.array([v for _, v in re.findall(r"Epoch (\d)/5 Loss: ([0-9.]+)", text)])
        g["demo_accuracies"] = np.array(re.findall(r"准确率: ([0-9.]+)%", text))
    g["demo_W1_head"] = r.mnist_xavier((784, 128), 784, reseed=42)[0, :32]
    rng = np.random.default_rng(3)
    pred = rng.random((300, 10)).astype(np.float32)
    pred[5] = 0.1
    pred[6, 3] = pred[6, 7] = 2.0
    pred[7] = -2.0
    lab = rng.integers(0, 10, 300).astype(np.float32)
    lab[5], lab[6], lab[7] = 0, 3, 0
    g["acc_pred"], g["acc_labels"], g["acc"] = pred, lab, r.mnist_accuracy(pred, lab)
    for tag, (I, H1, H2, n, batch, steps) in (("s", (20, 12, 8, 48, 16, 9)), ("m", (64, 32, 16, 96, 32, 12))):
        seed = 600 + I
        x = o.uniform((n, I), seed, 0, 1)
        y = o.ints((n,), seed + 1, 10)
        params = [o.uniform((I, H1), seed + 2, -I ** -0.5, I ** -0.5), np.zeros(H1, np.float32),
                  o.uniform((H1, H2), seed + 3, -H1 ** -0.5, H1 ** -0.5), np.zeros(H2, np.float32),
                  o.uniform((H2, 10), seed + 4, -H2 ** -0.5, H2 ** -0.5), np.zeros(10, np.float32)]
        losses, trained = r.mnist_train(x, y, params, batch, steps, 0.01)
        g[tag + "_x"], g[tag + "_y"], g[tag + "_losses"] = x, y, losses
        g[tag + "_cfg"] = np.array([batch, steps], np.int64)
        for k, (p0, p1) in enumerate(zip(params, trained)):
            g["%s_p%d" % (tag, k)], g["%s_q%d" % (tag, k)] = p0, p1
    np.savez_compressed(os.path.join(HERE, "mnist.npz"), **g)


def typed():
    """Tensors that are not fp32 (support.typed_cases): the reference's Tensor::to, zero / ones, scalar
    operators and double softmax; only the outputs are stored, the inputs come from the seeded generator."""
    from support import typed_cases
    o = Oracle()
    r = Reference()
    g = {}
    for name, a, dt, steps in typed_cases(o):
        rc, out = r.typed(a, dt, steps)
        assert rc == a.size, (name, rc)
        g[name] = out
    np.savez_compressed(os.path.join(HERE, "typed.npz"), **g)


def main():
    o = Oracle()   # only for its input generator
    r = Reference()
    out = {}

    # ---- elementwise forward
    x = np.concatenate([o.normal((1500,), 1, 0, 3), SPECIAL])
    y = np.concatenate([o.normal((1500,), 2, 0, 3), SPECIAL[::-1]])
    g = {"x": x, "y": y}
    for code, name in [(ADD, "add"), (SUB, "sub"), (MUL, "mul"), (DIV, "div")]:
        rc, g[name] = r.binary(code, x, y, x.shape)
        assert rc == x.size
    for code, name in [(NEG, "neg"), (RELU, "relu"), (SIN, "sin"), (COS, "cos"), (TANH, "tanh"),
                       (SIGMOID, "sigmoid")]:
        g[name] = r.unary(code, x)
    for w, s, name in [(0, 5.0, "scalar_add"), (1, 2.0, "scalar_mul"), (2, 7.0, "scalar_div")]:
        rc, g[name] = r.scalar(w, x, s)
    # dense sweep of the transcendental inputs that matter for tanh/sigmoid cancellation
    t = np.concatenate([o.uniform((4000,), 3, -2, 2), o.uniform((2000,), 4, -0.02, 0.02),
                        o.uniform((2000,), 5, -90, 90), o.uniform((2000,), 6, -1000, 1000)])
    g["t"] = t
    for code, name in [(SIN, "t_sin"), (COS, "t_cos"), (TANH, "t_tanh"), (SIGMOID, "t_sigmoid")]:
        g[name] = r.unary(code, t)
    np.savez_compressed(os.path.join(HERE, "elementwise.npz"), **g)

    # ---- broadcast Add forms
    a = o.normal((37, 53), 11, 0, 2)
    b = o.uniform((53,), 12, -1, 1)
    g = {"a": a, "b": b}
    rc, g["add_rowbcast"] = r.binary(ADD, a, b, a.shape)
    rc, g["add_scalar_tensor"] = r.binary(ADD, a, b[:1], a.shape)
    # the reference's own answers for the forms it does not support (return codes only)
    g["rc_sub_rowbcast"] = np.int64(r.binary(SUB, a, b, a.shape)[0])
    g["rc_mul_rowbcast"] = np.int64(r.binary(MUL, a, b, a.shape)[0])
    g["rc_add_left_1d"] = np.int64(r.binary(ADD, b, a, a.shape)[0])
    # same-shape kernels on a hand-materialised row operand: what the row-broadcast forms must equal
    bm = np.broadcast_to(b, a.shape).copy()
    for code, name in [(SUB, "sub_mat"), (MUL, "mul_mat"), (DIV, "div_mat")]:
        rc, g[name] = r.binary(code, a, bm, a.shape)
    np.savez_compressed(os.path.join(HERE, "broadcast.npz"), **g)

    # ---- reductions, softmax, cross entropy
    v1 = o.uniform((100003,), 21, -1, 1)
    v2 = o.uniform((100003,), 22, -1, 1)
    g = {"v1": v1, "v2": v2}
    for code, name in [(DOT, "dot"), (MSE, "mse"), (MAE, "mae")]:
        rc, val = r.binary(code, v1, v2, ())
        g[name] = val
    g["sum"] = r.sum(v1)
    sx = o.normal((19, 301), 23, 0, 2)
    g["sx"] = sx
    g["softmax_d1"] = r.softmax(sx, 1)
    g["softmax_d0"] = r.softmax(sx, 0)
    g["softmax_1d"] = r.softmax(sx[0], 0)
    g["softmax_kernel"] = r.unary(SOFTMAX_KERNEL, sx)
    idx = o.ints((19,), 24, 301)
    oh = np.zeros_like(sx)
    oh[np.arange(19), idx.astype(int)] = 1
    g["idx"] = idx
    rc, g["ce_onehot"] = r.binary(CE, sx, oh, ())
    rc, g["ce_index"] = r.binary(CE, sx, idx, ())
    rc, g["ce_1d"] = r.binary(CE, sx[0], oh[0], ())
    bad = idx.copy()
    bad[3] = 301
    g["rc_ce_bad_index"] = np.int64(r.binary(CE, sx, bad, ())[0])
    # saturated rows: pred underflows below the 1e-10 clamp
    hx = sx.copy()
    hx[:, 0] += 60.0
    g["hx"] = hx
    rc, g["ce_onehot_clamped"] = r.binary(CE, hx, oh, ())
    np.savez_compressed(os.path.join(HERE, "reduce_softmax_ce.npz"), **g)

    # ---- matmul, all four operand layouts
    A = o.normal((33, 47), 31)
    B = o.normal((47, 29), 32)
    At, Bt = np.ascontiguousarray(A.T), np.ascontiguousarray(B.T)
    g = {"A": A, "B": B}
    g["nn"] = r.matmul_t(A, 0, B, 0)
    g["nt"] = r.matmul_t(A, 0, Bt, 1)
    g["tn"] = r.matmul_t(At, 1, B, 0)
    g["tt"] = r.matmul_t(At, 1, Bt, 1)
    A2 = o.normal((130, 257), 33)
    B2 = o.normal((257, 70), 34)
    g["A2"], g["B2"], g["nn2"] = A2, B2, r.matmul_t(A2, 0, B2, 0)
    np.savez_compressed(os.path.join(HERE, "matmul.npz"), **g)

    # ---- backward pieces through the reference's tape
    x = o.normal((37, 53), 41, 0, 2)
    y = o.normal((37, 53), 42, 0, 2)
    w = o.normal((37, 53), 43)
    g = {"x": x, "y": y, "w": w}
    for code, name in [(NEG, "neg"), (RELU, "relu"), (SIN, "sin"), (COS, "cos"), (TANH, "tanh"),
                       (SIGMOID, "sigmoid")]:
        g["d_" + name] = r.grad_unary(code, x, w)
    g["d_softmax_d1"] = r.grad_softmax(x, 1, w)
    g["d_softmax_d0"] = r.grad_softmax(x, 0, w)
    for code, name in [(MSE, "mse"), (MAE, "mae")]:
        rc, loss, dp = r.grad_loss(code, x, y, 0.37)
        g["d_" + name] = dp
    lg = o.normal((19, 31), 44, 0, 2)
    idx = o.ints((19,), 45, 31)
    oh = np.zeros_like(lg)
    oh[np.arange(19), idx.astype(int)] = 1
    g["lg"], g["lg_idx"] = lg, idx
    rc, loss, g["d_ce_onehot"] = r.grad_loss(CE, lg, oh, 0.37)
    g["rc_d_ce_index"] = np.int64(r.grad_loss(CE, lg, idx, 0.37)[0])
    yb = (y + np.float32(4.0) * np.sign(y)).astype(np.float32)
    g["yb"] = yb
    rc, g["d_div_a"], g["d_div_b"] = r.grad_binary(DIV, x, yb, w)
    rc, g["d_mul_a"], g["d_mul_b"] = r.grad_binary(MUL, x, y, w)
    rc, g["d_sub_a"], g["d_sub_b"] = r.grad_binary(SUB, x, y, w)
    b = o.uniform((53,), 46, -1, 1)
    g["b"] = b
    rc, g["d_addrow_a"], g["d_addrow_b"] = r.grad_binary(ADD, x, b, w)
    yz = y.copy()
    yz[3, 4] = 0.0
    g["rc_d_div_zero"] = np.int64(r.grad_binary(DIV, x, yz, w)[0])
    A = o.normal((33, 47), 47)
    B = o.normal((47, 29), 48)
    W = o.normal((33, 29), 49)
    g["A"], g["B"], g["W"] = A, B, W
    rc, g["d_matmul_a"], g["d_matmul_b"] = r.grad_binary(MATMUL, A, B, W)
    np.savez_compressed(os.path.join(HERE, "backward.npz"), **g)

    # ---- whole configurations at miniature sizes (seeds as in the full-size runs)
    a = o.uniform((4099,), 101, -1, 1)
    bb = o.uniform((4099,), 102, -1, 1)
    s, ga, gb = r.chain(a, bb)
    g = {"chain_a": a, "chain_b": bb, "chain_s": s, "chain_ga": ga, "chain_gb": gb}
    Bn, I, H, Cn = 16, 40, 24, 10
    xx = (o.ints((Bn, I), 301, 256) / np.float32(255.0)).astype(np.float32)
    lab = o.ints((Bn,), 302, Cn)
    oh = np.zeros((Bn, Cn), np.float32)
    oh[np.arange(Bn), lab.astype(int)] = 1
    k1, k2 = 1 / np.sqrt(I), 1 / np.sqrt(H)
    W1, b1 = o.uniform((I, H), 311, -k1, k1), o.uniform((H,), 312, -k1, k1)
    W2, b2 = o.uniform((H, Cn), 313, -k2, k2), o.uniform((Cn,), 314, -k2, k2)
    loss, logits, gW1, gb1, gW2, gb2 = r.mlp_step(xx, W1, b1, W2, b2, oh)
    g.update(mlp_x=xx, mlp_lab=lab, mlp_W1=W1, mlp_b1=b1, mlp_W2=W2, mlp_b2=b2, mlp_loss=loss,
             mlp_logits=logits, mlp_gW1=gW1, mlp_gb1=gb1, mlp_gW2=gW2, mlp_gb2=gb2)
    X = o.uniform((12, 8), 501, -2, 2)
    rv = o.uniform((8,), 502, 0.5, 2)
    T = o.normal((12, 8), 503)
    R = np.broadcast_to(rv, X.shape).copy()
    Y, mse, mae, gX, gR = r.expr(X, R, T)
    g.update(expr_X=X, expr_r=rv, expr_T=T, expr_Y=Y, expr_mse=mse, expr_mae=mae, expr_gX=gX, expr_gR=gR)
    np.savez_compressed(os.path.join(HERE, "configs.npz"), **g)

    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    if "mnist" in sys.argv[1:]:
        mnist()
    elif "programs" in sys.argv[1:]:
        programs()
    elif "typed" in sys.argv[1:]:
        typed()
    else:
        main()
        mnist()
        programs()
        typed()

"""The MNIST demo's path on the MI355X: the four launch-layer entry points through the C ABI
(bit-exact against the oracle), and the loader / model / training loop of the C++ front-end against
the oracle and the vectors written from the real reference."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import gpu_support as G
from support import HostLayer, libc_xavier, same_bits, synthetic_digits, write_idx_images, write_mnist_dir

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def host():
    return HostLayer()


@pytest.mark.parametrize("n", [1, 15, 16, 4096, 28 * 28 * 37, 1 << 20])
def test_pixel_bytes_to_unit_floats(oracle, n):
    print("case u8_to_unit", n, flush=True)
    rng = np.random.default_rng(n)
    src = rng.integers(0, 256, n + 3).astype(np.uint8)
    src[:min(n, 256)] = np.arange(min(n, 256))            # every byte value when it fits
    for off in (0, 3):                                     # aligned, and a pointer that is not 16-byte aligned
        d_src = torch.from_numpy(src).to(G.DEV)
        out = torch.full((n + 1,), -7.0, device=G.DEV)
        G.call("ctamd_u8_to_unit_f32", C.c_void_p(d_src.data_ptr() + off), G.ptr(out), n, G.stream())
        got = G.host(out)
        assert same_bits(got[:n], oracle.u8_to_unit(src[off:off + n])) and got[n] == -7.0


@pytest.mark.parametrize("shape", [(1, 1), (128, 10), (5, 3), (1000, 37)])
def test_onehot(oracle, shape):
    print("case onehot", shape, flush=True)
    rows, classes = shape
    labels = oracle.ints((rows,), 40 + rows, classes)
    out = torch.empty(rows, classes, device=G.DEV)
    d_labels = G.dev(labels)
    G.call("ctamd_onehot_f32", G.ptr(d_labels), G.ptr(out), rows, classes, G.stream())
    assert same_bits(G.host(out), oracle.onehot(labels, classes))


@pytest.mark.parametrize("n", [1, 7, 4096, 100003, 1 << 22])
def test_sgd_step_is_two_roundings(oracle, n):
    print("case sgd", n, flush=True)
    p = oracle.uniform((n,), 50, -1, 1)
    g = oracle.normal((n,), 51, 0, 3)
    for lr in (0.01, 0.1, 1e-3):
        d_p, d_g = G.dev(p), G.dev(g)
        G.call("ctamd_sgd_step_f32", G.ptr(d_p), G.ptr(d_g), C.c_float(lr), n, G.stream())
        assert same_bits(G.host(d_p), oracle.sgd_step(p, g, lr))


def test_count_correct(oracle, golden):
    print("case count_correct", flush=True)
    g = golden("mnist")
    cnt = torch.full((1,), 99, dtype=torch.int32, device=G.DEV)
    d_pred, d_labels = G.dev(g["acc_pred"]), G.dev(g["acc_labels"])     # named: the buffers must outlive the launch
    G.call("ctamd_count_correct_f32", G.ptr(d_pred), G.ptr(d_labels), G.ptr(cnt), 300, 10, G.stream())
    assert F(int(cnt.item())) / F(300) == g["acc"]
    for rows, classes in ((1, 1), (257, 10), (5000, 10), (1000, 3)):
        pred = oracle.uniform((rows, classes), 60 + rows, 0, 1)
        pred[::7] = pred[::7, :1]                          # ties: the first index wins
        labels = oracle.ints((rows,), 61 + rows, classes)
        d_pred, d_labels = G.dev(pred), G.dev(labels)
        G.call("ctamd_count_correct_f32", G.ptr(d_pred), G.ptr(d_labels), G.ptr(cnt), rows, classes, G.stream())
        assert int(cnt.item()) == oracle.count_correct(pred, labels)
    G.call("ctamd_count_correct_f32", None, None, G.ptr(cnt), 0, 10, G.stream())
    assert int(cnt.item()) == 0


def test_loader_reads_idx_files_into_hbm(oracle, host, golden, tmp_path):
    print("case loader", flush=True)
    tr_i, tr_l, te_i, te_l = write_mnist_dir(str(tmp_path))
    for train, img, lab in ((True, tr_i, tr_l), (False, te_i, te_l)):
        images, labels = host.mnist_load(str(tmp_path), train)
        assert same_bits(images, oracle.u8_to_unit(img.reshape(img.shape[0], 784)))
        assert np.array_equal(labels, lab.astype(F))
    images, _ = host.mnist_load(str(tmp_path), True)
    assert same_bits(images[:4], golden("mnist")["loader_first_rows"])      # the reference loader's output
    # a truncated image file is an error, not garbage
    with open(os.path.join(str(tmp_path), "train-images-idx3-ubyte"), "r+b") as f:
        f.truncate(16 + 784 * 100)
    dims = (C.c_long * 2)()
    assert host.cdll.cth_mnist_load(str(tmp_path).encode(), 1, None, None, dims) == -1


def test_accuracy(host, golden):
    g = golden("mnist")
    assert host.mnist_accuracy(g["acc_pred"], g["acc_labels"]) == g["acc"]


@pytest.mark.parametrize("tag", ["s", "m"])
def test_training_loop_against_the_reference_vectors(host, oracle, golden, tag):
    """The demo's loop with the reference's tape properties: losses and trained parameters of the
    real reference.  MatMul and the row sums are tree-ordered on the device, so the bar is the
    reduction bar (1e-5 relative per operator), compounded over the steps."""
    print("case training", tag, flush=True)
    g = golden("mnist")
    batch, steps = (int(v) for v in g[tag + "_cfg"])
    params = [g["%s_p%d" % (tag, k)] for k in range(6)]
    losses, trained = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=True)
    assert np.all(np.abs(losses - g[tag + "_losses"]) <= 1e-4 * np.abs(g[tag + "_losses"]))
    for k in range(6):
        want = g["%s_q%d" % (tag, k)]
        assert np.all(np.abs(trained[k] - want) <= 1e-4 * np.abs(want) + 2e-5)
    # live leaves + column-sum bias gradients: the oracle with both properties switched off
    losses2, trained2 = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=False)
    want_l, want_p = oracle.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, False, False)
    assert np.all(np.abs(losses2 - want_l) <= 1e-4 * np.abs(want_l))
    for k in range(6):
        assert np.all(np.abs(trained2[k] - want_p[k]) <= 1e-4 * np.abs(want_p[k]) + 2e-5)
    assert not np.allclose(losses2, losses, rtol=1e-6, atol=0)        # and the two modes do differ


def test_demo_on_a_synthetic_data_set(host, oracle, tmp_path):
    """The whole demo (load, 784-128-64-10, 3 epochs of 4 batches of 128, evaluate) against the
    oracle run from the same rand() weights, at a learning rate where training is stable (at the
    demo's 0.01 the sum-reduced loss diverges on this data, in the reference too)."""
    print("case demo", flush=True)
    tr_i, tr_l, te_i, te_l = write_mnist_dir(str(tmp_path))
    lr = 1e-3
    x, y = oracle.u8_to_unit(tr_i.reshape(-1, 784)), tr_l.astype(F)
    xt, yt = oracle.u8_to_unit(te_i.reshape(-1, 784)), te_l.astype(F)
    for reference_tape in (True, False):
        rc, losses, acc, seconds = host.mnist_demo(str(tmp_path), epochs=3, lr=lr, reference_tape=reference_tape)
        assert rc == 12
        params = [libc_xavier((784, 128), 784, reseed=42), np.zeros(128, F), libc_xavier((128, 64), 128),
                  np.zeros(64, F), libc_xavier((64, 10), 64), np.zeros(10, F)]
        step_losses, trained = oracle.mnist_train(x, y, params, 128, 12, lr, reference_tape, reference_tape)
        want = step_losses.reshape(3, 4).astype(np.float64).mean(1)
        assert np.all(np.abs(losses - want) <= 2e-4 * want), (losses, want)
        assert losses[2] < losses[0]                                   # it learns
        want_train = oracle.count_correct(oracle.mnist_predict(x, trained), y) / 512
        want_test = oracle.count_correct(oracle.mnist_predict(xt, trained), yt) / 256
        assert abs(acc[0] - want_train) <= 0.02 and abs(acc[1] - want_test) <= 0.02


@pytest.mark.parametrize("tag", ["s", "m"])
def test_recorded_step_replays_to_the_same_bits(host, golden, tag):
    """The training step recorded into a HIP graph at the first batch and replayed for every batch,
    with unrelated eager launches and host reads between the replays: every loss and every trained
    parameter must have the bits of the step-by-step run (same kernels, same order)."""
    print("case recorded step", tag, flush=True)
    g = golden("mnist")
    batch, steps = (int(v) for v in g[tag + "_cfg"])
    params = [g["%s_p%d" % (tag, k)] for k in range(6)]
    eager_l, eager_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=0)
    graph_l, graph_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=2)
    assert same_bits(graph_l, eager_l)
    for a, b in zip(graph_p, eager_p):
        assert same_bits(a, b)


def test_sgd_step_of_several_tensors_in_one_launch(oracle):
    """ctamd_sgd_step_multi_f32 against the single-tensor update on the gradient with its -0 turned
    into +0 (what reading it from the tape does), for 40 tensors (two launches of at most 32), sizes
    from 1 to beyond one block's chunk, one of them empty, with -0 gradients on -0 parameters."""
    print("case sgd multi", flush=True)
    sizes = [1, 7, 2047, 2048, 2049, 100003, 0, 10, 784 * 128, 64] + [33 + 17 * k for k in range(30)]
    ps = [oracle.uniform((n,), 500 + k, -1, 1) for k, n in enumerate(sizes)]
    gs = [oracle.normal((n,), 600 + k, 0, 3) for k, n in enumerate(sizes)]
    ps[2][:50] = -0.0
    gs[2][:100:2] = -0.0
    gs[2][1:100:2] = 0.0
    d_p = [G.dev(p) for p in ps]
    d_g = [G.dev(g) for g in gs]
    ptrs_p = (C.c_void_p * len(sizes))(*[t.data_ptr() if t.numel() else None for t in d_p])
    ptrs_g = (C.c_void_p * len(sizes))(*[t.data_ptr() if t.numel() else None for t in d_g])
    counts = (C.c_size_t * len(sizes))(*sizes)
    G.call("ctamd_sgd_step_multi_f32", ptrs_p, ptrs_g, counts, len(sizes), C.c_float(0.01), G.stream())
    for k, n in enumerate(sizes):
        want = oracle.sgd_step(ps[k], gs[k] + F(0), 0.01) if n else ps[k]
        assert same_bits(G.host(d_p[k]), want), k
    assert np.signbit(G.host(d_p[2])[:50]).all()               # -0 - (+0 * lr) stays -0; without the "0 +" it would be +0


@pytest.mark.parametrize("tag", ["s", "m"])
def test_fused_layers_and_update_give_the_same_bits(host, golden, tag):
    """Each layer as one fused operator (matmul + bias + ReLU in one launch, one tape entry) and the
    optimiser update of the six tensors as one launch: every loss and trained parameter has the
    bits of the operator-by-operator run, in each tape mode (live leaves, the reference's tape,
    recorded step)."""
    print("case fused layers", tag, flush=True)
    g = golden("mnist")
    batch, steps = (int(v) for v in g[tag + "_cfg"])
    params = [g["%s_p%d" % (tag, k)] for k in range(6)]
    for mode in (0, 1, 2):
        plain_l, plain_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=mode)
        fused_l, fused_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=mode + 4)
        assert same_bits(fused_l, plain_l), mode
        for a, b in zip(fused_p, plain_p):
            assert same_bits(a, b), mode


def test_demo_with_a_recorded_step(host, tmp_path):

    print("case demo recorded", flush=True)
    write_mnist_dir(str(tmp_path))
    rc1, l1, a1, _ = host.mnist_demo(str(tmp_path), epochs=3, lr=1e-3, reference_tape=0)
    rc2, l2, a2, _ = host.mnist_demo(str(tmp_path), epochs=3, lr=1e-3, reference_tape=2)
    assert rc1 == rc2 == 12
    assert same_bits(l1, l2) and same_bits(a1, a2)


def test_demo_adds_its_epoch_loss_on_the_device(host, tmp_path):
    """The demo adds the batch losses of an epoch on the device (the reference's fp32 additions in the
    reference's order) and reads the sum once per epoch; with every step reading its loss instead (mode
    bit 16) the epoch losses and accuracies are the same bits - operator by operator, with fused layers
    and with the one-pass head."""
    print("case demo epoch loss on the device", flush=True)
    write_mnist_dir(str(tmp_path))
    for mode in (0, 4, 12):
        rc1, l1, a1, _ = host.mnist_demo(str(tmp_path), epochs=3, lr=1e-3, reference_tape=mode)
        rc2, l2, a2, _ = host.mnist_demo(str(tmp_path), epochs=3, lr=1e-3, reference_tape=mode + 16)
        assert rc1 == rc2 == 12, mode
        assert same_bits(l1, l2) and same_bits(a1, a2), mode


def test_demo_as_the_first_device_work_of_a_process(host, tmp_path):
    """The demo seeds the C library's generator and draws its weights from it, as the reference does; bringing
    the GPU runtime up draws from the same generator, so the device is initialised before the seed is set.
    A fresh process whose first device work is the demo trains to the same losses as this one."""
    print("case demo in a fresh process", flush=True)
    import subprocess
    import sys
    write_mnist_dir(str(tmp_path))
    rc, want, acc, _ = host.mnist_demo(str(tmp_path), epochs=2, lr=1e-3, reference_tape=0)
    assert rc == 8
    code = ("import sys; sys.path.insert(0, %r); from support import HostLayer; h = HostLayer(); h.cdll.cth_quiet(); "
            "rc, l, a, _ = h.mnist_demo(%r, epochs=2, lr=1e-3, reference_tape=0); print('LOSSES', rc, ' '.join(float(v).hex() for v in l))"
            % (os.path.dirname(os.path.abspath(__file__)), str(tmp_path)))
    p = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    line = [ln for ln in p.stdout.splitlines() if ln.startswith("LOSSES")]
    assert p.returncode == 0 and line, p.stdout[-2000:]
    assert line[0].split()[1] == "8" and line[0].split()[2:] == [float(v).hex() for v in want], (line[0], want)


@pytest.mark.parametrize("tag", ["s", "m"])
def test_training_with_the_one_pass_head(host, golden, tag):
    """The training loop with the last layer and its loss as the one-pass head (class indices instead of
    the one-hot matrix, products added in another order): losses and trained parameters agree with the
    operator-by-operator run to the reduction bar compounded over the steps, eagerly and as a recorded
    step."""
    print("case training with the one-pass head", tag, flush=True)
    g = golden("mnist")
    batch, steps = (int(v) for v in g[tag + "_cfg"])
    params = [g["%s_p%d" % (tag, k)] for k in range(6)]
    plain_l, plain_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=0)
    for mode in (0, 2):
        head_l, head_p = host.mnist_train(g[tag + "_x"], g[tag + "_y"], params, batch, steps, 0.01, reference_tape=mode + 12)
        assert np.abs(head_l - plain_l).max() <= 1e-4 * np.abs(plain_l).max(), mode
        for a, b in zip(head_p, plain_p):
            assert np.abs(a - b).max() <= 1e-4 * max(1.0, np.abs(b).max()), mode

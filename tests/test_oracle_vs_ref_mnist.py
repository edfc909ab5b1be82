"""The MNIST demo's path: the CPU oracle against the reference itself (its loader, its accuracy and
batch functions, its training loop over the reference library, and the demo program's own main()
run on a small synthetic data set).  Runs only where oracle/_ref has been built."""
import os
import re

import numpy as np
import pytest

from support import Reference, f32, libc_xavier, ref_available, same_bits, write_mnist_dir

pytestmark = pytest.mark.skipif(not ref_available(), reason="reference build (oracle/_ref) not present")
F = np.float32


@pytest.fixture(scope="module")
def ref():
    return Reference()


@pytest.fixture(scope="module")
def data_dir(tmp_path_factory):
    d = tmp_path_factory.mktemp("idx")
    return str(d), write_mnist_dir(str(d))


def test_loader_arithmetic(ref, oracle, data_dir):
    d, (tr_i, tr_l, te_i, te_l) = data_dir
    for train, img, lab in ((True, tr_i, tr_l), (False, te_i, te_l)):
        images, labels = ref.mnist_load(d, train)
        assert images.shape == (img.shape[0], 784)
        assert same_bits(images, oracle.u8_to_unit(img.reshape(img.shape[0], 784)))
        assert np.array_equal(labels, lab.astype(F))
    # every byte value
    allb = np.arange(256, dtype=np.uint8)
    assert same_bits(oracle.u8_to_unit(allb), (allb.astype(F) / F(255.0)).astype(F))


def test_accuracy_and_batches(ref, oracle):
    rng = np.random.default_rng(3)
    pred = f32(rng.random((300, 10)))
    pred[5] = 0.1                  # a full tie: the first index wins
    pred[6, 3] = pred[6, 7] = 2.0  # a two-way tie
    pred[7] = -2.0                 # nothing exceeds the starting value -1: label 0
    labels = f32(rng.integers(0, 10, 300))
    labels[5], labels[6], labels[7] = 0, 3, 0
    want = ref.mnist_accuracy(pred, labels)
    got = oracle.count_correct(pred, labels)
    assert np.float32(got) / np.float32(300) == want
    images = f32(rng.random((70, 12)))
    lab = f32(rng.integers(0, 10, 70))
    for idx in (0, 1, 2):          # the last batch is ragged (70 = 2*32 + 6)
        bi, bl = ref.mnist_get_batch(images, lab, 32, idx)
        assert same_bits(bi, images[idx * 32:(idx + 1) * 32]) and same_bits(bl, lab[idx * 32:(idx + 1) * 32])


def small_problem(oracle, I, H1, H2, n, seed):
    x = oracle.uniform((n, I), seed, 0, 1)
    y = oracle.ints((n,), seed + 1, 10)
    params = [oracle.uniform((I, H1), seed + 2, -I ** -0.5, I ** -0.5), np.zeros(H1, F),
              oracle.uniform((H1, H2), seed + 3, -H1 ** -0.5, H1 ** -0.5), np.zeros(H2, F),
              oracle.uniform((H2, 10), seed + 4, -H2 ** -0.5, H2 ** -0.5), np.zeros(10, F)]
    return x, y, params


@pytest.mark.parametrize("shape", [(20, 12, 8, 48, 16, 9), (64, 32, 16, 96, 32, 12)])
def test_training_loop_bit_for_bit(ref, oracle, shape):
    I, H1, H2, n, batch, steps = shape
    x, y, params = small_problem(oracle, I, H1, H2, n, 600 + I)
    want_losses, want_params = ref.mnist_train(x, y, params, batch, steps, 0.01)
    got_losses, got_params = oracle.mnist_train(x, y, params, batch, steps, 0.01, True, True)
    assert same_bits(got_losses, want_losses)
    for g, w in zip(got_params, want_params):
        assert same_bits(g, w)
    # the two tape properties are what make it so: without either, the bits differ
    for row0, stale in ((False, True), (True, False)):
        other, _ = oracle.mnist_train(x, y, params, batch, steps, 0.01, row0, stale)
        assert not same_bits(other, want_losses)


def test_optimiser_update_is_not_fused(oracle):
    p = oracle.uniform((4096,), 70, -1, 1)
    g = oracle.uniform((4096,), 71, -1, 1)
    lr = F(0.01)
    got = oracle.sgd_step(p, g, lr)
    assert same_bits(got, (p - (g * lr).astype(F)).astype(F))
    fused = (p.astype(np.float64) - g.astype(np.float64) * np.float64(lr)).astype(F)
    assert not same_bits(got, fused)       # a single rounding would differ somewhere in 4096 values


def test_demo_program_end_to_end(ref, oracle, data_dir, capfd):
    """The reference demo's own main() on the synthetic set: 784-128-64-10, batch 128, lr 0.01,
    5 epochs (mnist/mnist.cpp:236-246); its printed epoch losses and accuracies against the oracle
    run with the same initial weights (srand(42), rand() in the demo's order)."""
    d, (tr_i, tr_l, te_i, te_l) = data_dir
    rc = ref.mnist_main_in(d)
    out = capfd.readouterr().out
    assert rc == 0
    epoch_losses = re.findall(r"Epoch (\d)/5 Loss: ([0-9.]+)", out)
    accs = re.findall(r"准确率: ([0-9.]+)%", out)
    assert [e for e, _ in epoch_losses] == list("12345") and len(accs) == 2

    W1 = ref.mnist_xavier((784, 128), 784, reseed=42)
    W2 = ref.mnist_xavier((128, 64), 128)
    W3 = ref.mnist_xavier((64, 10), 64)
    # the same numbers from the C library directly (what tests without the reference build use)
    assert same_bits(W1, libc_xavier((784, 128), 784, reseed=42)) and same_bits(W2, libc_xavier((128, 64), 128))
    assert same_bits(W3, libc_xavier((64, 10), 64))
    params = [W1, np.zeros(128, F), W2, np.zeros(64, F), W3, np.zeros(10, F)]
    x = oracle.u8_to_unit(tr_i.reshape(-1, 784))
    y = tr_l.astype(F)
    nb = 512 // 128
    losses, trained = oracle.mnist_train(x, y, params, 128, 5 * nb, 0.01, True, True)
    for e in range(5):
        acc = F(0)
        for b in range(nb):
            acc = F(acc + losses[e * nb + b])
        acc = F(acc / F(nb))
        assert "%.4f" % acc == epoch_losses[e][1]
    xt = oracle.u8_to_unit(te_i.reshape(-1, 784))
    train_acc = F(oracle.count_correct(oracle.mnist_predict(x, trained), y)) / F(512)
    test_acc = F(oracle.count_correct(oracle.mnist_predict(xt, trained), te_l.astype(F))) / F(256)
    assert "%.2f" % (train_acc * 100) == accs[0] and "%.2f" % (test_acc * 100) == accs[1]

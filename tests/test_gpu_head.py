"""The classifier head in one pass (ctamd_linear_ce_head_f32): logits, summed cross entropy, and the
gradients of the logits, the hidden activations, the weights and the bias, against an fp64 evaluation
of the same formulas (every result within 1e-5 of the sum of the magnitudes of its terms) and against
the five launches it replaces."""
import numpy as np
import pytest

import gpu_support as G

pytestmark = pytest.mark.gpu
F = np.float32


def inputs(oracle, B, H, N, seed):
    h = oracle.uniform((B, H), seed, -1, 1)
    h = np.where(h > 0, h, F(0)).astype(F)                       # what a ReLU layer hands on: half zeros
    k = F(1.0 / np.sqrt(H))
    w = oracle.uniform((H, N), seed + 1, -k, k) * F(4)
    b = oracle.uniform((N,), seed + 2, -k, k)
    lab = oracle.ints((B,), seed + 3, N).astype(F)
    return h, w, b, lab


def fp64_head(h, w, b, lab, mask):
    h64, w64 = h.astype(np.float64), w.astype(np.float64)
    z = h64 @ w64 + b.astype(np.float64)
    e = np.exp(z - z.max(axis=1, keepdims=True))
    sm = e / e.sum(axis=1, keepdims=True)
    idx = lab.astype(int)
    loss = -np.log(np.maximum(sm[np.arange(len(idx)), idx], 1e-10)).sum()
    dz = sm.copy()
    dz[np.arange(len(idx)), idx] -= 1.0
    dh = dz @ w64.T
    if mask:
        dh = dh * (h64 > 0)
    return z, loss, dz, dh, h64.T @ dz, dz.sum(axis=0)


@pytest.mark.parametrize("mode", [G.MATH_FAST, G.MATH_EXACT])
@pytest.mark.parametrize("B,H,N", [(256, 256, 10), (8192, 256, 10), (37, 64, 10), (5, 4, 2), (1000, 128, 16), (64, 252, 3), (4099, 256, 7)])
def test_head_against_fp64(oracle, B, H, N, mode):
    print("case head", B, H, N, mode, flush=True)
    h, w, b, lab = inputs(oracle, B, H, N, 4000 + B)
    prev = G.set_math_mode(mode)
    try:
        for mask in (0, 1):
            loss, status, z, dz, dh, gw, gb = G.linear_ce_head(G.dev(h), G.dev(w), G.dev(b), G.dev(lab), mask)
            assert status == 0
            Z, L, DZ, DH, GW, GB = fp64_head(h, w, b, lab, mask)
            az = np.abs(h).astype(np.float64) @ np.abs(w) + np.abs(b)
            assert (np.abs(G.host(z) - Z) <= 1e-5 * az).all()
            # a softmax element moves by at most its own size times the error of the logits (twice: max and sum)
            dz_tol = 2e-5 * az.max(axis=1, keepdims=True) + 4e-7
            assert (np.abs(G.host(dz) - DZ) <= dz_tol).all()
            assert abs(float(loss.item()) - L) <= 1e-5 * np.abs(np.log(np.maximum(DZ + (DZ < 0), 1e-10))).sum() + 1e-5 * az.max() * B
            assert (np.abs(G.host(dh) - DH) <= 1e-5 * (np.abs(DZ) @ np.abs(w).T) + (dz_tol * np.abs(w).sum(axis=1).max())).all()
            assert (np.abs(G.host(gw) - GW) <= 1e-5 * (np.abs(h).T.astype(np.float64) @ np.abs(DZ)) + dz_tol.max() * np.abs(h).sum(axis=0)[:, None]).all()
            assert (np.abs(G.host(gb) - GB) <= 1e-5 * np.abs(DZ).sum(axis=0) + dz_tol.max() * B).all()
    finally:
        G.set_math_mode(prev)


def test_head_against_the_five_launches(oracle):
    """The same step as the library's separate launches compute it (product with bias, cross entropy with
    its gradient, the masked product, the weight gradient with the column sums): equal within the
    MatMul bound - the head adds in another order."""
    print("case head vs launches", flush=True)
    B, H, N = 512, 256, 10
    h, w, b, lab = inputs(oracle, B, H, N, 77)
    dh_, dw_, db_, dl_ = G.dev(h), G.dev(w), G.dev(b), G.dev(lab)
    loss, status, z, dz, dh, gw, gb = G.linear_ce_head(dh_, dw_, db_, dl_, 1)
    z2 = G.matmul_bias(dh_, dw_, db_, False)
    loss2, status2, dz2 = G.ce_index_fused(z2, dl_)
    dh2 = G.matmul_relu_mask(dz2, dw_.t(), dh_)
    gw2 = G.matmul(dh_.t(), dz2)
    gb2 = G.colsum(dz2)
    assert status == status2 == 0
    close = lambda a, c, tol: float((a - c).abs().max()) <= tol
    assert close(z, z2, 1e-5 * 8) and close(dz, dz2, 4e-6)
    assert abs(float(loss.item()) - float(loss2.item())) <= 1e-5 * float(loss2.item())
    assert close(dh, dh2, 2e-5) and close(gw, gw2, 1e-5 * B) and close(gb, gb2, 1e-5 * B)
    # deterministic: the same bits on a second call
    again = G.linear_ce_head(dh_, dw_, db_, dl_, 1)
    for x, y in zip((loss, z, dz, dh, gw, gb), (again[0],) + again[2:]):
        assert bool((x == y).all())


def test_head_edges(oracle):
    print("case head edges", flush=True)
    h, w, b, lab = inputs(oracle, 40, 64, 10, 91)
    lab[7] = 10.0                                                # out of range: status 1, NaN loss, the other rows as usual
    loss, status, z, dz, dh, gw, gb = G.linear_ce_head(G.dev(h), G.dev(w), G.dev(b), G.dev(lab), 0)
    assert status == 1 and np.isnan(float(loss.item()))
    for wrong in (np.nan, np.inf, -1.0, 3e9):                    # read as the reference reads an index: none of these is a class
        lab[7] = wrong
        assert G.linear_ce_head(G.dev(h), G.dev(w), G.dev(b), G.dev(lab), 0)[1] == 1, wrong
    lab[7] = 3.0
    loss, status, z2, dz2, _, _, _ = G.linear_ce_head(G.dev(h), G.dev(w), G.dev(b), G.dev(lab), 0, want_dh=False)
    assert status == 0 and np.isfinite(float(loss.item()))
    keep = np.arange(40) != 7
    assert (G.host(dz)[keep] == G.host(dz2)[keep]).all() and (G.host(z) == G.host(z2)).all()
    # shapes the head does not take
    assert G.lib().ctamd_linear_ce_head_fits(256, 10) == 1
    for H, N in ((260, 10), (256, 17), (254, 10), (256, 1)):
        assert G.lib().ctamd_linear_ce_head_fits(H, N) == 0
    hh = G.dev(np.zeros((8, 260), F))
    G.linear_ce_head(hh, G.dev(np.zeros((260, 10), F)), G.dev(np.zeros(10, F)), G.dev(np.zeros(8, F)), 0, expect=-5)

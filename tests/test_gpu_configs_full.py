"""The five BASELINE configurations at their full sizes.  Where the CPU oracle finishes in seconds it
is the checker (configs 1, 3 at batch 256); at the large sizes the checks are the size-independent
ones: closed forms (dC = ones turns the MatMul gradients into row / column sums), fp64 recomputation
on the device by torch as an independent arbiter, conservation laws (softmax rows sum to 1, dlogits
rows sum to 0) and agreement of sampled rows with the oracle."""
import numpy as np
import pytest
import torch

import gpu_support as G
from support import HostLayer, same_bits

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def host():
    return HostLayer()


def test_config1_elementwise_chain_2e20(oracle, host):
    print("case config 1", flush=True)
    n = 1 << 20
    a = oracle.uniform((n,), 101, -1, 1)
    b = oracle.uniform((n,), 102, -1, 1)
    s, ga, gb = host.chain(a, b)
    ws, wga, wgb = oracle.chain(a, b)
    c = (a * b + F(5.0)).astype(F)
    assert abs(float(s) - float(ws)) <= 1e-5 * float(np.maximum(c, 0).astype(np.float64).sum())
    assert abs(float(s) - np.maximum(c, 0).astype(np.float64).sum()) <= 1e-5 * np.maximum(c, 0).astype(np.float64).sum()
    assert same_bits(ga, wga) and same_bits(gb, wgb)           # grad(a) = b*[c>0], grad(b) = a*[c>0]
    assert same_bits(ga, (b * (c > 0)).astype(F) + F(0)) and same_bits(gb, (a * (c > 0)).astype(F) + F(0))


@pytest.mark.parametrize("M", [1024, 2048, 4096])
def test_config2_matmul_forward_backward(oracle, M):
    print("case config 2 M", M, flush=True)
    A = G.dev(oracle.normal((M, M), 201))       # the configuration's seeds: 201 / 202 (203 for the linearity check)
    B = G.dev(oracle.normal((M, M), 202))
    C = G.matmul(A, B)
    rows = torch.tensor([0, 1, M // 3, M - 1], device=G.DEV)
    ref = A[rows].double() @ B.double()
    bound = 1e-5 * (A[rows].abs().double() @ B.abs().double())
    assert bool(((C[rows].double() - ref).abs() <= bound).all())
    cols = torch.tensor([0, 7, M // 2, M - 1], device=G.DEV)
    refc = A.double() @ B[:, cols].double()
    boundc = 1e-5 * (A.abs().double() @ B[:, cols].abs().double())
    assert bool(((C[:, cols].double() - refc).abs() <= boundc).all())
    if M == 1024:       # the oracle's own rows (sequential fused accumulation) agree to the same bound
        a_np, b_np = G.host(A[:4]), G.host(B)
        want = oracle.matmul(a_np, b_np)
        bnd = 2e-5 * (np.abs(a_np).astype(np.float64) @ np.abs(b_np).astype(np.float64))
        assert np.all(np.abs(G.host(C[:4]) - want) <= bnd)
    # backward with dC = ones: dA = dC . B^T has rows equal to the row sums of B, dB = A^T . dC the
    # column sums of A (closed form; B and A enter as transposed views)
    dC = torch.ones(M, M, device=G.DEV)
    dA = G.matmul(dC, B.t())
    dB = G.matmul(A.t(), dC)
    rs, cs = B.double().sum(1), A.double().sum(0)
    assert bool(((dA.double() - rs[None, :]).abs() <= 1e-5 * B.abs().double().sum(1)[None, :]).all())
    assert bool(((dB.double() - cs[:, None]).abs() <= 1e-5 * A.abs().double().sum(0)[:, None]).all())
    # linearity: A.(B + B2) = A.B + A.B2 up to rounding
    B2 = G.dev(oracle.normal((M, M), 203))
    lhs = G.matmul(A, B + B2)
    rhs = C + G.matmul(A, B2)
    scale = A.abs().double() @ (B.abs() + B2.abs()).double()[:, :8]
    assert bool(((lhs[:, :8] - rhs[:, :8]).abs().double() <= 3e-5 * scale).all())


def test_config2_dot_2e26(oracle):
    print("case config 2 dot", flush=True)
    n = 1 << 26
    a = G.dev(oracle.uniform((n,), 211, -1, 1))
    b = G.dev(oracle.uniform((n,), 212, -1, 1))
    got = float(G.reduce2("dot", a, b).item())
    want = float(torch.dot(a.double(), b.double()).item())
    assert abs(got - want) <= 1e-5 * float((a.double() * b.double()).abs().sum().item())
    # Cauchy-Schwarz equality case and sign symmetry
    assert abs(float(G.reduce2("dot", a, a).item()) - float((a.double() ** 2).sum().item())) <= 1e-5 * float((a.double() ** 2).sum().item())
    assert float(G.reduce2("dot", a, -b).item()) == -got


@pytest.mark.parametrize("B", [256, 8192])
def test_config3_mlp_train_step(oracle, host, B):
    print("case config 3 B", B, flush=True)
    I, H, C = 784, 256, 10
    x = (oracle.ints((B, I), 301, 256) / F(255.0)).astype(F)
    lab = oracle.ints((B,), 302, C)
    k1, k2 = 1 / np.sqrt(I), 1 / np.sqrt(H)
    W1, b1 = oracle.uniform((I, H), 311, -k1, k1), oracle.uniform((H,), 312, -k1, k1)
    W2, b2 = oracle.uniform((H, C), 313, -k2, k2), oracle.uniform((C,), 314, -k2, k2)
    got = host.mlp_step(x, W1, b1, W2, b2, lab, True)       # class-index targets, column-sum bias gradients
    names = ["loss", "logits", "gW1", "gb1", "gW2", "gb2"]
    if B == 256:
        oh = np.zeros((B, C), F)
        oh[np.arange(B), lab.astype(int)] = 1
        want = oracle.mlp_step(x, W1, b1, W2, b2, oh, False)
        for n, a, w in zip(names, got, want):
            assert np.abs(a - w).max() <= 1e-4 * max(1.0, np.abs(w).max()), n
        host.set_reference_row0(True)       # and the reference's own bias gradients (row 0) on request
        try:
            got0 = host.mlp_step(x, W1, b1, W2, b2, oh, False)
        finally:
            host.set_reference_row0(False)
        want0 = oracle.mlp_step(x, W1, b1, W2, b2, oh, True)
        for n, a, w in zip(names, got0, want0):
            assert np.abs(a - w).max() <= 1e-4 * max(1.0, np.abs(w).max()), ("row0", n)
    # fp64 autograd of torch as the arbiter at both sizes
    d = torch.float64
    tx = torch.from_numpy(x).to(G.DEV, d)
    p = [torch.from_numpy(t).to(G.DEV, d).requires_grad_(True) for t in (W1, b1, W2, b2)]
    logits = torch.relu(tx @ p[0] + p[1]) @ p[2] + p[3]
    loss = torch.nn.functional.cross_entropy(logits, torch.from_numpy(lab).to(G.DEV).long(), reduction="sum")
    loss.backward()
    assert abs(float(got[0]) - float(loss)) <= 1e-5 * float(loss)
    assert np.abs(got[1] - logits.detach().cpu().numpy()).max() <= 1e-4
    for a, t, n in zip(got[2:], p, names[2:]):
        w = t.grad.cpu().numpy()
        assert np.abs(a - w).max() <= 1e-5 * max(1.0, np.abs(w).max()) * (B / 256) ** 0.5, n


def test_config4_softmax_cross_entropy_8192x32000(oracle):
    print("case config 4", flush=True)
    rows, cols = 8192, 32000
    x = G.dev(oracle.normal((rows, cols), 401, 0.0, 2.0))     # the configuration's seeds: 401 / 402
    idxf = G.dev(oracle.ints((rows,), 402, cols))
    idx = idxf.long()
    loss, status = G.ce_index(x, idxf)
    assert status == 0
    lse = torch.logsumexp(x.double(), dim=1)
    want = float((lse - x.double()[torch.arange(rows, device=G.DEV), idx]).sum())
    assert abs(float(loss) - want) <= 1e-5 * want            # the SUM over rows; mean = sum / rows
    one = G.fill(1, 1.0)
    d = G.ce_bwd(x, idxf, one, True)
    rs = d.double().sum(1)
    assert float(rs.abs().max()) <= 1e-4                      # each row of softmax - onehot sums to 0
    sample = torch.tensor([0, 17, 4095, rows - 1], device=G.DEV)
    sm = torch.softmax(x[sample].double(), dim=1)
    sm[torch.arange(4, device=G.DEV), idx[sample]] -= 1
    assert float((d[sample].double() - sm).abs().max()) <= 1e-6
    y = G.softmax(x, 1)
    assert float((y.double().sum(1) - 1).abs().max()) <= 1e-5
    assert float((y[sample].double() - torch.softmax(x[sample].double(), dim=1)).abs().max()) <= 1e-7
    # loss and gradient from one pass over the logits: the same loss to the reduction bar, the same
    # gradient to 5e-7 (rows this long use the hardware exponential, as the backward pass from forward
    # statistics does)
    loss1, status1, d1pass = G.ce_index_fused(x, idxf)
    assert status1 == 0 and abs(float(loss1) - want) <= 1e-5 * want
    assert float((d1pass - d).abs().max()) <= 5e-7
    assert float(d1pass.double().sum(1).abs().max()) <= 1e-4
    assert float((d1pass[sample].double() - sm).abs().max()) <= 1e-6
    del d, y, d1pass
    # linearity of the gradient in the upstream scalar
    half = G.fill(1, 0.5)
    dh = G.ce_bwd(x[:64].contiguous(), idxf[:64].contiguous(), half, True)
    d1 = G.ce_bwd(x[:64].contiguous(), idxf[:64].contiguous(), one, True)
    assert torch.equal(dh, d1 * 0.5)


def test_config5_broadcast_expression_4096(oracle, host):
    print("case config 5", flush=True)
    n = 4096
    X = oracle.uniform((n, n), 501, -2, 2)
    r = oracle.uniform((n,), 502, 0.5, 2)
    T = oracle.normal((n, n), 503)
    Y, mse, mae, gX, gr = host.expr(X, r, T)
    # sampled rows against the oracle's arithmetic (bit-identical transcendentals, row-broadcast Div)
    R8 = np.broadcast_to(r, (8, n)).copy()
    Yo = oracle.expr(X[:8], R8, T[:8])[0]
    assert same_bits(Y[:8], Yo)
    d = torch.float64
    tX = torch.from_numpy(X).to(G.DEV, d).requires_grad_(True)
    tr = torch.from_numpy(r).to(G.DEV, d).requires_grad_(True)
    tT = torch.from_numpy(T).to(G.DEV, d)
    tY = torch.sigmoid(tX / tr) - torch.tanh(tX) * torch.sin(tX) + torch.cos(-tX)
    l1, l2 = ((tY - tT) ** 2).mean(), (tY - tT).abs().mean()
    (l1 + l2).backward()
    assert np.abs(Y - tY.detach().cpu().numpy()).max() <= 1e-6
    assert abs(float(mse) - float(l1)) <= 1e-5 * float(l1) and abs(float(mae) - float(l2)) <= 1e-5 * float(l2)
    wX, wr = tX.grad.cpu().numpy(), tr.grad.cpu().numpy()
    assert np.abs(gX - wX).max() <= 1e-5 * np.abs(wX).max()
    assert np.abs(gr - wr).max() <= 1e-5 * np.abs(wr).max() + 1e-9      # broadcast-sum reduction over 4096 rows

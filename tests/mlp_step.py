"""The 784-256-10 MLP train step expressed as the sequence of C-ABI calls the tape makes
(forward: MatMul, row-broadcast Add, ReLU, MatMul, Add, CrossEntropy; backward: the gradient
arithmetic of src/AutoDiff.cpp for those nodes, each edge accumulated into a zeroed gradient).
Shared by the smoke check, the parity tests and the benchmark's MLP leg."""
import torch

import gpu_support as G


def mlp_step_device(x, W1, b1, W2, b2, labels, bias_grad="colsum"):
    """All arguments are device tensors; labels are class indices held as floats.
    bias_grad: "colsum" (sum over the batch) or "row0" (the reference's slice).
    Returns (loss[1], logits, gW1, gb1, gW2, gb2)."""
    B, H, C = x.shape[0], W1.shape[1], W2.shape[1]
    z1 = G.matmul(x, W1)
    a1 = G.rowbcast("add", z1, b1)
    h = G.unary("relu", a1)
    z2 = G.matmul(h, W2)
    logits = G.rowbcast("add", z2, b2)
    loss, status = G.ce_index(logits, labels)
    assert status == 0
    # backward: root gradient 1.0 stays on the device
    one = G.fill(1, 1.0)

    def landed(val):        # grad = 0 + val, the tape's accumulate into a zeroed gradient
        return G.accumulate(torch.zeros_like(val), val)

    gl = landed(G.ce_bwd(logits, labels, one, True))
    gz2 = landed(gl)

    def bias(g):
        if bias_grad == "row0":
            return landed(g[0].clone())
        return landed(G.colsum(g))

    gb2 = bias(gl)
    gh = landed(G.matmul(gz2, W2.t()))
    gW2 = landed(G.matmul(h.t(), gz2))
    ga1 = landed(G.unary_bwd("relu", a1, gh))
    gz1 = landed(ga1)
    gb1 = bias(ga1)
    gW1 = landed(G.matmul(x.t(), gz1))
    return loss, logits, gW1, gb1, gW2, gb2

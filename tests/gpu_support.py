"""GPU-side test plumbing: torch provides device memory, every computation goes through the
C ABI of ctorch_amd/libctorch_amd.so (ctypes), nothing else."""
import ctypes as C

import numpy as np
import torch

from ctorch_amd import capi

DEV = "cuda:0"
_inited = False


def lib():
    global _inited
    l = capi.load()
    if not _inited:
        torch.cuda.init()
        torch.zeros(1, device=DEV)   # torch's context on device 0 first; the library shares it
        capi.check(l.ctamd_init(0))
        _inited = True
    return l


def dev(a):
    """numpy fp32 array -> device tensor (keeps shape)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(DEV)


def host(t):
    return t.detach().cpu().numpy()


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def empty_like(t):
    return torch.empty_like(t)


def call(name, *args):
    capi.check(getattr(lib(), name)(*args))


def binary(op, a, b):
    r = torch.empty_like(a)
    call("ctamd_%s_f32" % op, ptr(a), ptr(b), ptr(r), a.numel(), stream())
    return r


def rowbcast(op, a, b):
    r = torch.empty_like(a)
    call("ctamd_%s_rowbcast_f32" % op, ptr(a), ptr(b), ptr(r), a.shape[0], a.shape[1], stream())
    return r


def bscalar(op, a, b1):
    r = torch.empty_like(a)
    call("ctamd_%s_bscalar_f32" % op, ptr(a), ptr(b1), ptr(r), a.numel(), stream())
    return r


def rsub(a1, b):
    r = torch.empty_like(b)
    call("ctamd_rsub_ascalar_f32", ptr(a1), ptr(b), ptr(r), b.numel(), stream())
    return r


def scalar(op, a, s):
    r = torch.empty_like(a)
    call("ctamd_%s_scalar_f32" % op, ptr(a), C.c_float(s), ptr(r), a.numel(), stream())
    return r


def unary(op, a):
    r = torch.empty_like(a)
    call("ctamd_%s_f32" % op, ptr(a), ptr(r), a.numel(), stream())
    return r


def unary_bwd(op, x, g):
    r = torch.empty_like(x)
    call("ctamd_%s_backward_f32" % op, ptr(x), ptr(g), ptr(r), x.numel(), stream())
    return r


def reduce1(name, a):
    out = torch.empty(1, device=DEV)
    call("ctamd_%s_f32" % name, ptr(a), ptr(out), a.numel(), stream())
    return out


def reduce2(name, a, b):
    out = torch.empty(1, device=DEV)
    call("ctamd_%s_f32" % name, ptr(a), ptr(b), ptr(out), a.numel(), stream())
    return out


def colsum(g):
    out = torch.empty(g.shape[1], device=DEV)
    call("ctamd_colsum_f32", ptr(g), ptr(out), g.shape[0], g.shape[1], stream())
    return out


def any_tiny(b):
    flag = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    call("ctamd_any_abs_lt_eps_f32", ptr(b), ptr(flag), b.numel(), stream())
    return int(flag.item())


def softmax(x, dim=1):
    y = torch.empty_like(x)
    rows, cols = (1, x.numel()) if x.dim() == 1 else x.shape
    name = "ctamd_softmax_rows_f32" if (x.dim() == 1 or dim == 1) else "ctamd_softmax_cols_f32"
    call(name, ptr(x), ptr(y), rows, cols, stream())
    return y


def softmax_bwd(y, g, dim=1):
    dx = torch.empty_like(y)
    rows, cols = (1, y.numel()) if y.dim() == 1 else y.shape
    name = "ctamd_softmax_backward_rows_f32" if (y.dim() == 1 or dim == 1) else "ctamd_softmax_backward_cols_f32"
    call(name, ptr(y), ptr(g), ptr(dx), rows, cols, stream())
    return dx


def ce_onehot(x, t):
    out = torch.empty(1, device=DEV)
    rows, cols = (1, x.numel()) if x.dim() == 1 else x.shape
    call("ctamd_cross_entropy_onehot_f32", ptr(x), ptr(t), ptr(out), rows, cols, stream())
    return out


def ce_index(x, idx):
    out = torch.empty(1, device=DEV)
    status = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    call("ctamd_cross_entropy_index_f32", ptr(x), ptr(idx), ptr(out), ptr(status), x.shape[0], x.shape[1], stream())
    return out, int(status.item())


def ce_index_fused(x, idx):
    """loss, status and the gradient for an upstream gradient of 1, one launch over the logits"""
    out = torch.empty(1, device=DEV)
    status = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    dx = torch.empty_like(x)
    call("ctamd_cross_entropy_index_fused_f32", ptr(x), ptr(idx), ptr(out), ptr(status), ptr(dx), x.shape[0], x.shape[1], stream())
    return out, int(status.item()), dx


def ce_bwd(x, t, g1, index):
    dx = torch.empty_like(x)
    rows, cols = (1, x.numel()) if x.dim() == 1 else x.shape
    name = "ctamd_cross_entropy_backward_%s_f32" % ("index" if index else "onehot")
    call(name, ptr(x), ptr(t), ptr(g1), ptr(dx), rows, cols, stream())
    return dx


def loss_bwd(name, p, t, g1):
    dp = torch.empty_like(p)
    call("ctamd_%s_backward_f32" % name, ptr(p), ptr(t), ptr(g1), ptr(dp), p.numel(), stream())
    return dp


def unary_bwd_acc(name, x, g, acc):
    dx = torch.empty_like(x)
    call("ctamd_%s_backward_acc_f32" % name, ptr(x), ptr(g), ptr(acc), ptr(dx), x.numel(), stream())
    return dx


def loss_bwd_acc(name, p, t, g1, acc):
    dp = torch.empty_like(p)
    call("ctamd_%s_backward_acc_f32" % name, ptr(p), ptr(t), ptr(g1), ptr(acc), ptr(dp), p.numel(), stream())
    return dp


def div_bwd_b_rowbcast(a, b, g):
    r = torch.empty_like(a)
    call("ctamd_div_backward_b_rowbcast_f32", ptr(a), ptr(b), ptr(g), ptr(r), a.shape[0], a.shape[1], stream())
    return r


def div_bwd_b(a, b, g):
    r = torch.empty_like(a)
    call("ctamd_div_backward_b_f32", ptr(a), ptr(b), ptr(g), ptr(r), a.numel(), stream())
    return r


def fill(n, v):
    r = torch.empty(n, device=DEV)
    call("ctamd_fill_f32", ptr(r), C.c_float(v), n, stream())
    return r


def fill_from(n, v1):
    r = torch.empty(n, device=DEV)
    call("ctamd_fill_from_f32", ptr(r), ptr(v1), n, stream())
    return r


def accumulate(grad, val):
    call("ctamd_accumulate_f32", ptr(grad), ptr(val), grad.numel(), stream())
    return grad


def matmul_bias(a, b, bias, relu):
    """The fused layer: a.b (+ bias row) (then ReLU); bias may be None."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2 and (bias is None or bias.numel() == n)
    c = torch.empty((m, n), device=DEV)
    call("ctamd_matmul_bias_f32", ptr(a), a.stride(0), a.stride(1), ptr(b), b.stride(0), b.stride(1),
         ptr(bias) if bias is not None else None, int(relu), ptr(c), m, n, k, stream())
    return c


def matmul_relu_mask(a, b, y):
    """(a.b) * [y > 0]: the gradient at a ReLU layer's pre-activation, in the product's launch."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2 and tuple(y.shape) == (m, n) and y.is_contiguous()
    c = torch.empty((m, n), device=DEV)
    call("ctamd_matmul_relu_mask_f32", ptr(a), a.stride(0), a.stride(1), ptr(b), b.stride(0), b.stride(1), ptr(y), ptr(c),
         m, n, k, stream())
    return c


def matmul_colsum(a, b):
    """a.b and the column sums of b (the weight and bias gradients of a layer) from one call."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = torch.full((m, n), float("nan"), device=DEV)
    sums = torch.full((n,), float("nan"), device=DEV)
    call("ctamd_matmul_colsum_f32", ptr(a), a.stride(0), a.stride(1), ptr(b), b.stride(0), b.stride(1), ptr(c), ptr(sums), m, n, k,
         stream())
    return c, sums


def matmul(a, b):
    """a, b: 2-D device tensors, possibly transposed views (strides are passed through)."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    c = torch.empty((m, n), device=DEV)
    call("ctamd_matmul_f32", ptr(a), a.stride(0), a.stride(1), ptr(b), b.stride(0), b.stride(1), ptr(c), m, n, k,
         stream())
    return c


def linear_ce_head(h, w, bias, labels, mask_by_h, want_z=True, want_dh=True, expect=0):
    """The classifier head in one pass: returns (loss, status, z, dz, dh, gw, gb) as device tensors / ints."""
    B, H = h.shape
    N = w.shape[1]
    pair = torch.zeros(2, device=DEV)
    status = torch.full((1,), -7, dtype=torch.int32, device=DEV)
    z = torch.zeros((B, N), device=DEV) if want_z else None
    dz = torch.zeros((B, N), device=DEV)
    dh = torch.zeros((B, H), device=DEV) if want_dh else None
    gw = torch.zeros((H, N), device=DEV)
    gb = torch.zeros(N, device=DEV)
    rc = lib().ctamd_linear_ce_head_f32(ptr(h), ptr(w), ptr(bias), ptr(labels), ptr(pair), ptr(status), ptr(z), ptr(dz), ptr(dh),
                                        int(mask_by_h), ptr(gw), ptr(gb), B, H, N, stream())
    assert rc == expect, (rc, lib().ctamd_last_error().decode())
    return pair[:1], int(status.item()), z, dz, dh, gw, gb


class ExprInsn(C.Structure):
    _fields_ = [("op", C.c_uint8), ("dst", C.c_uint8), ("a", C.c_uint8), ("b", C.c_uint8), ("imm", C.c_float)]


def expr_run(prog, inputs, n_out, rows, cols, expect=0):
    """Runs a fused-expression program [(op, dst, a, b, imm)] on device tensors; returns (outputs,
    status word).  expect: the return code the call must give."""
    arr = (ExprInsn * max(1, len(prog)))(*[ExprInsn(*q) for q in prog])
    outs = [torch.zeros((rows, cols), device=DEV) for _ in range(n_out)]
    status = torch.zeros(1, dtype=torch.int32, device=DEV)
    pin = (C.c_void_p * max(1, len(inputs)))(*[t.data_ptr() for t in inputs])
    pout = (C.c_void_p * max(1, n_out))(*[t.data_ptr() for t in outs])
    rc = lib().ctamd_expr_run_f32(arr, len(prog), pin, len(inputs), pout, n_out, ptr(status), rows, cols, stream())
    assert rc == expect, (rc, lib().ctamd_last_error().decode())
    return outs, int(status.cpu()[0])


# ----------------------------------------------------------------- tensors that are not fp32
DT_F32, DT_F64, DT_I32, DT_I64, DT_BOOL = range(5)
TORCH_DTYPE = {DT_F32: torch.float32, DT_F64: torch.float64, DT_I32: torch.int32, DT_I64: torch.int64, DT_BOOL: torch.uint8}


def fill_typed(dtype, value, n):
    r = torch.empty(n, dtype=TORCH_DTYPE[dtype], device=DEV)
    call("ctamd_fill_typed", ptr(r), dtype, C.c_double(value), n, stream())
    return r


def cast_from_f32(x, dtype):
    r = torch.empty(x.shape, dtype=TORCH_DTYPE[dtype], device=DEV)
    call("ctamd_cast_from_f32", ptr(x), ptr(r), dtype, x.numel(), stream())
    return r


def scalar_op_typed(x, dtype, op, s):
    r = torch.empty_like(x)
    call("ctamd_scalar_op_typed", ptr(x), ptr(r), dtype, op, C.c_float(s), x.numel(), stream())
    return r


def accumulate_typed(acc, val, dtype):
    call("ctamd_accumulate_typed", ptr(acc), ptr(val), dtype, acc.numel(), stream())
    return acc


def softmax_f64(x, dim):
    r = torch.empty_like(x)
    rows, cols = (1, x.numel()) if x.dim() == 1 else x.shape
    call("ctamd_softmax_f64", ptr(x), ptr(r), rows, cols, 1 if x.dim() == 1 else dim, stream())
    return r


def set_expr_jit(threshold):
    """After how many launches a fused-expression program is compiled at run time (0: never, 1: at
    first sight); returns the previous setting."""
    l = lib()
    prev = l.ctamd_expr_jit()
    capi.check(l.ctamd_set_expr_jit(threshold))
    return prev


def expr_jit_stats():
    """(programs compiled, compilations failed, launches of compiled kernels, launches of the interpreter)."""
    v = [C.c_uint64(0) for _ in range(4)]
    lib().ctamd_expr_jit_stats(*[C.byref(x) for x in v])
    return tuple(int(x.value) for x in v)


MATH_FAST, MATH_EXACT = 0, 1


def set_math_mode(mode):
    """CTAMD_MATH_FAST (0, the default) or CTAMD_MATH_EXACT (1) for later launches; returns the previous mode."""
    l = lib()
    prev = l.ctamd_math_mode()
    capi.check(l.ctamd_set_math_mode(mode))
    return prev

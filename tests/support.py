"""ctypes doors for the tests: the CPU oracle (oracle/liboracle.so) and, where it has been built,
the real reference library behind oracle/ref_driver.cpp (oracle/_ref/libctorch_ref.so).

Test infrastructure only; nothing here is imported by the package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

FP = C.POINTER(C.c_float)
DP = C.POINTER(C.c_double)
LP = C.POINTER(C.c_long)

# op codes of oracle/ref_driver.cpp
ADD, SUB, MUL, DIV, MATMUL, DOT, MSE, MAE, CE = range(9)
NEG, RELU, SIN, COS, TANH, SIGMOID, SOFTMAX_KERNEL = range(20, 27)


NP_DTYPE = {0: np.float32, 1: np.float64, 2: np.int32, 3: np.int64, 4: np.uint8}


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(FP)


def bits(a):
    return f32(a).view(np.uint32)


def same_bits(a, b):
    a, b = f32(a), f32(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def ulp_diff(a, b):
    """Distance in units in the last place between two fp32 arrays (finite values)."""
    def key(x):
        i = f32(x).view(np.int32).astype(np.int64)
        return np.where(i < 0, -(i & 0x7FFFFFFF), i)
    return np.abs(key(a) - key(b))


def build_oracle():
    if not os.path.exists(os.path.join(ORACLE_DIR, "liboracle.so")):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "all"], stdout=subprocess.DEVNULL)


class Oracle:
    """Thin numpy wrapper over oracle/liboracle.so."""

    def __init__(self):
        build_oracle()
        self.lib = C.CDLL(os.path.join(ORACLE_DIR, "liboracle.so"))
        L = self.lib
        L.co_dot.restype = C.c_float
        L.co_mse.restype = C.c_float
        L.co_mae.restype = C.c_float
        L.co_sum.restype = C.c_float
        L.co_ce_onehot.restype = C.c_float
        L.co_ce_index.restype = C.c_int
        L.co_any_abs_lt_eps.restype = C.c_int

    # ---- inputs
    def uniform(self, shape, seed, lo, hi):
        r = np.empty(shape, np.float32)
        self.lib.co_fill_uniform(fp(r), C.c_long(r.size), C.c_uint64(seed), C.c_double(lo), C.c_double(hi))
        return r

    def normal(self, shape, seed, mean=0.0, sigma=1.0):
        r = np.empty(shape, np.float32)
        self.lib.co_fill_normal(fp(r), C.c_long(r.size), C.c_uint64(seed), C.c_double(mean), C.c_double(sigma))
        return r

    def ints(self, shape, seed, rng):
        r = np.empty(shape, np.float32)
        self.lib.co_fill_int(fp(r), C.c_long(r.size), C.c_uint64(seed), C.c_long(rng))
        return r

    # ---- helpers
    def _ew2(self, name, a, b):
        a, b = f32(a), f32(b)
        assert a.shape == b.shape
        r = np.empty_like(a)
        getattr(self.lib, name)(fp(a), fp(b), fp(r), C.c_long(a.size))
        return r

    def _ew1(self, name, a):
        a = f32(a)
        r = np.empty_like(a)
        getattr(self.lib, name)(fp(a), fp(r), C.c_long(a.size))
        return r

    def add(self, a, b): return self._ew2("co_add", a, b)
    def sub(self, a, b): return self._ew2("co_sub", a, b)
    def mul(self, a, b): return self._ew2("co_mul", a, b)
    def div(self, a, b): return self._ew2("co_div", a, b)
    def neg(self, a): return self._ew1("co_neg", a)
    def relu(self, a): return self._ew1("co_relu", a)
    def sin(self, a): return self._ew1("co_sin", a)
    def cos(self, a): return self._ew1("co_cos", a)
    def tanh(self, a): return self._ew1("co_tanh", a)
    def sigmoid(self, a): return self._ew1("co_sigmoid", a)

    def binary(self, op, a, b):
        return [self.add, self.sub, self.mul, self.div][op](a, b)

    def unary(self, code, a):
        return {NEG: self.neg, RELU: self.relu, SIN: self.sin, COS: self.cos, TANH: self.tanh,
                SIGMOID: self.sigmoid}[code](a)

    def add_scalar_tensor(self, a, b1):
        a, b1 = f32(a), f32(b1).reshape(1)
        r = np.empty_like(a)
        self.lib.co_add_scalar_tensor(fp(a), fp(b1), fp(r), C.c_long(a.size))
        return r

    def binary_rowbcast(self, op, a, b):
        a, b = f32(a), f32(b)
        rows, cols = a.shape
        assert b.shape == (cols,)
        r = np.empty_like(a)
        if op == ADD:
            self.lib.co_add_rowbcast(fp(a), fp(b), fp(r), C.c_long(rows), C.c_long(cols))
        else:
            self.lib.co_binary_rowbcast(C.c_int(op), fp(a), fp(b), fp(r), C.c_long(rows), C.c_long(cols))
        return r

    def softmax(self, x, dim=1, guard=False):
        x = f32(x)
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        d = 1 if x.ndim == 1 else dim
        y = np.empty_like(x2)
        self.lib.co_softmax(fp(x2), fp(y), C.c_long(x2.shape[0]), C.c_long(x2.shape[1]), C.c_int(d), C.c_int(int(guard)))
        return y.reshape(x.shape)

    def matmul(self, a, b):
        """a, b may be non-contiguous 2-D views of fp32 arrays (e.g. .T); strides are honoured."""
        assert a.dtype == np.float32 and b.dtype == np.float32
        m, k = a.shape
        k2, n = b.shape
        assert k == k2
        c = np.empty((m, n), np.float32)
        pa = C.cast(a.ctypes.data, FP)
        pb = C.cast(b.ctypes.data, FP)
        self.lib.co_matmul(pa, C.c_long(a.strides[0] // 4), C.c_long(a.strides[1] // 4),
                           pb, C.c_long(b.strides[0] // 4), C.c_long(b.strides[1] // 4),
                           fp(c), C.c_long(m), C.c_long(n), C.c_long(k))
        return c

    def dot(self, a, b):
        a, b = f32(a), f32(b)
        return np.float32(self.lib.co_dot(fp(a), fp(b), C.c_long(a.size)))

    def mse(self, a, b):
        a, b = f32(a), f32(b)
        return np.float32(self.lib.co_mse(fp(a), fp(b), C.c_long(a.size)))

    def mae(self, a, b):
        a, b = f32(a), f32(b)
        return np.float32(self.lib.co_mae(fp(a), fp(b), C.c_long(a.size)))

    def sum(self, a):
        a = f32(a)
        return np.float32(self.lib.co_sum(fp(a), C.c_long(a.size)))

    def ce_onehot(self, x, t):
        x, t = f32(x), f32(t)
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        return np.float32(self.lib.co_ce_onehot(fp(x2), fp(t), C.c_long(x2.shape[0]), C.c_long(x2.shape[1])))

    def ce_index(self, x, idx):
        x, idx = f32(x), f32(idx)
        out = C.c_float(0)
        rc = self.lib.co_ce_index(fp(x), fp(idx), C.c_long(x.shape[0]), C.c_long(x.shape[1]), C.byref(out))
        return None if rc != 0 else np.float32(out.value)

    def scalar(self, which, a, s):
        a = f32(a)
        r = np.empty_like(a)
        name = ["co_scalar_add", "co_scalar_mul", "co_scalar_div"][which]
        getattr(self.lib, name)(fp(a), C.c_float(s), fp(r), C.c_long(a.size))
        return r

    # ---- backward pieces
    def accumulate0(self, val):
        """0 + val: what a single edge leaves in a zero-initialised gradient."""
        val = f32(val)
        g = np.zeros_like(val)
        self.lib.co_accumulate(fp(g), fp(val), C.c_long(val.size))
        return g

    def _bwd2(self, name, x, g):
        x, g = f32(x), f32(g)
        r = np.empty_like(x)
        getattr(self.lib, name)(fp(x), fp(g), fp(r), C.c_long(x.size))
        return r

    def relu_bwd(self, x, g): return self._bwd2("co_relu_bwd", x, g)
    def sigmoid_bwd(self, x, g): return self._bwd2("co_sigmoid_bwd", x, g)
    def tanh_bwd(self, x, g): return self._bwd2("co_tanh_bwd", x, g)
    def sin_bwd(self, x, g): return self._bwd2("co_sin_bwd", x, g)
    def cos_bwd(self, x, g): return self._bwd2("co_cos_bwd", x, g)

    def unary_bwd(self, code, x, g):
        if code == NEG:
            return self.neg(g)
        return {RELU: self.relu_bwd, SIN: self.sin_bwd, COS: self.cos_bwd, TANH: self.tanh_bwd,
                SIGMOID: self.sigmoid_bwd}[code](x, g)

    def softmax_bwd(self, y, g, dim=1):
        y, g = f32(y), f32(g)
        y2 = y.reshape(1, -1) if y.ndim == 1 else y
        d = 1 if y.ndim == 1 else dim
        r = np.empty_like(y2)
        self.lib.co_softmax_bwd(fp(y2), fp(g), fp(r), C.c_long(y2.shape[0]), C.c_long(y2.shape[1]), C.c_int(d))
        return r.reshape(y.shape)

    def mse_bwd(self, p, t, g):
        p, t = f32(p), f32(t)
        r = np.empty_like(p)
        self.lib.co_mse_bwd(fp(p), fp(t), C.c_float(g), fp(r), C.c_long(p.size))
        return r

    def mae_bwd(self, p, t, g):
        p, t = f32(p), f32(t)
        r = np.empty_like(p)
        self.lib.co_mae_bwd(fp(p), fp(t), C.c_float(g), fp(r), C.c_long(p.size))
        return r

    def ce_bwd_onehot(self, x, t, g):
        x, t = f32(x), f32(t)
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        r = np.empty_like(x2)
        self.lib.co_ce_bwd_onehot(fp(x2), fp(t), C.c_float(g), fp(r), C.c_long(x2.shape[0]), C.c_long(x2.shape[1]))
        return r.reshape(x.shape)

    def ce_bwd_index(self, x, idx, g):
        x, idx = f32(x), f32(idx)
        r = np.empty_like(x)
        self.lib.co_ce_bwd_index(fp(x), fp(idx), C.c_float(g), fp(r), C.c_long(x.shape[0]), C.c_long(x.shape[1]))
        return r

    def div_bwd_a(self, g, b): return self._ew2("co_div_bwd_a", g, b)

    def div_bwd_b(self, a, b, g):
        a, b, g = f32(a), f32(b), f32(g)
        r = np.empty_like(a)
        self.lib.co_div_bwd_b(fp(a), fp(b), fp(g), fp(r), C.c_long(a.size))
        return r

    def any_abs_lt_eps(self, b):
        b = f32(b)
        return bool(self.lib.co_any_abs_lt_eps(fp(b), C.c_long(b.size)))

    def adjust_row0(self, g):
        g = f32(g)
        r = np.empty(g.shape[1], np.float32)
        self.lib.co_adjust_row0(fp(g), fp(r), C.c_long(g.shape[0]), C.c_long(g.shape[1]))
        return r

    def colsum_f64(self, g):
        g = f32(g)
        r = np.empty(g.shape[1], np.float64)
        self.lib.co_colsum_f64(fp(g), r.ctypes.data_as(DP), C.c_long(g.shape[0]), C.c_long(g.shape[1]))
        return r

    # ---- gradient shape adjustment (the reference's whole function) and its mathematical twin
    def adjust_grad_shape(self, g, target_shape):
        """co_adjust_grad_shape; None where the reference would read beyond its gradient buffer."""
        gshape = np.shape(g)                      # (a 0-D array would come out of f32() as [1])
        g = f32(g).reshape(-1)
        gs = (C.c_long * max(1, len(gshape)))(*gshape)
        ts = (C.c_long * max(1, len(target_shape)))(*target_shape)
        out = np.empty(target_shape, np.float32)
        rc = self.lib.co_adjust_grad_shape(fp(g), gs, C.c_int(len(gshape)), fp(out.reshape(-1)), ts, C.c_int(len(target_shape)))
        assert rc in (0, -1), rc
        return out if rc == 0 else None

    def broadcast_reduce(self, g, target_shape):
        g = f32(g)
        gs = (C.c_long * max(1, g.ndim))(*g.shape)
        ts = (C.c_long * max(1, len(target_shape)))(*target_shape)
        out = np.empty(target_shape, np.float32)
        rc = self.lib.co_broadcast_reduce(fp(g.reshape(-1)), gs, C.c_int(g.ndim), fp(out.reshape(-1)), ts, C.c_int(len(target_shape)))
        return out if rc == 0 else None

    # ---- methods the reference declares and never defines
    UNARY_EXT = {"abs": 0, "exp": 1, "log": 2, "sqrt": 3, "square": 4, "tan": 5, "leaky_relu": 6, "sub_scalar": 7}

    def unary_ext(self, name, a, p=0.0):
        a = f32(a)
        r = np.empty_like(a)
        self.lib.co_unary_ext(C.c_int(self.UNARY_EXT[name]), fp(a), C.c_float(p), fp(r), C.c_long(a.size))
        return r

    def unary_ext_bwd(self, name, v, g, p=0.0):
        v, g = f32(v), f32(g)
        r = np.empty_like(v)
        self.lib.co_unary_ext_bwd(C.c_int(self.UNARY_EXT[name]), fp(v), fp(g), C.c_float(p), fp(r), C.c_long(v.size))
        return r

    REDUCE = {"sum": 0, "mean": 1, "max": 2, "min": 3, "var": 4, "std": 5}

    def reduce_dim(self, kind, x, outer, length, inner, ddof=1):
        """-> (out [outer, inner], index int32 [outer, inner], mean [outer, inner])"""
        x = f32(x)
        assert x.size == outer * length * inner
        out = np.empty((outer, inner), np.float32)
        index = np.zeros((outer, inner), np.int32)
        mean = np.zeros((outer, inner), np.float32)
        self.lib.co_reduce_dim(C.c_int(self.REDUCE[kind]), fp(x.reshape(-1)), fp(out.reshape(-1)), index.ctypes.data_as(C.c_void_p),
                               fp(mean.reshape(-1)), C.c_long(outer), C.c_long(length), C.c_long(inner), C.c_int(ddof))
        return out, index, mean

    def reduce_dim_bwd(self, kind, x, y, index, mean, g, outer, length, inner, ddof=1):
        x, y, mean, g = f32(x), f32(y), f32(mean), f32(g)
        index = np.ascontiguousarray(index, np.int32)
        dx = np.empty(outer * length * inner, np.float32)
        self.lib.co_reduce_dim_bwd(C.c_int(self.REDUCE[kind]), fp(x.reshape(-1)), fp(y.reshape(-1)), index.ctypes.data_as(C.c_void_p),
                                   fp(mean.reshape(-1)), fp(g.reshape(-1)), fp(dx), C.c_long(outer), C.c_long(length), C.c_long(inner),
                                   C.c_int(ddof))
        return dx.reshape(x.shape)

    def log_softmax(self, x, dim=1):
        x = f32(x)
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        y = np.empty_like(x2)
        self.lib.co_log_softmax(fp(x2), fp(y), C.c_long(x2.shape[0]), C.c_long(x2.shape[1]), C.c_int(1 if x.ndim == 1 else dim))
        return y.reshape(x.shape)

    def log_softmax_bwd(self, y, g, dim=1):
        y, g = f32(y), f32(g)
        y2 = y.reshape(1, -1) if y.ndim == 1 else y
        r = np.empty_like(y2)
        self.lib.co_log_softmax_bwd(fp(y2), fp(g), fp(r), C.c_long(y2.shape[0]), C.c_long(y2.shape[1]), C.c_int(1 if y.ndim == 1 else dim))
        return r.reshape(y.shape)

    # ---- configurations
    def chain(self, a, b):
        a, b = f32(a), f32(b)
        s = C.c_float(0)
        ga, gb = np.empty_like(a), np.empty_like(b)
        self.lib.co_chain(fp(a), fp(b), C.c_long(a.size), C.byref(s), fp(ga), fp(gb))
        return np.float32(s.value), ga, gb

    def mlp_step(self, x, W1, b1, W2, b2, onehot, strict_row0):
        x, W1, b1, W2, b2, onehot = map(f32, (x, W1, b1, W2, b2, onehot))
        B, I = x.shape
        H = W1.shape[1]
        Cn = W2.shape[1]
        loss = C.c_float(0)
        logits = np.empty((B, Cn), np.float32)
        gW1, gb1, gW2, gb2 = (np.empty_like(t) for t in (W1, b1, W2, b2))
        self.lib.co_mlp_step(fp(x), C.c_long(B), C.c_long(I), fp(W1), fp(b1), C.c_long(H), fp(W2), fp(b2),
                             C.c_long(Cn), fp(onehot), C.c_int(int(strict_row0)), C.byref(loss), fp(logits),
                             fp(gW1), fp(gb1), fp(gW2), fp(gb2))
        return np.float32(loss.value), logits, gW1, gb1, gW2, gb2

    def expr(self, X, R, T):
        X, R, T = f32(X), f32(R), f32(T)
        rows, cols = X.shape
        Y, gX, gR = np.empty_like(X), np.empty_like(X), np.empty_like(X)
        mse, mae = C.c_float(0), C.c_float(0)
        self.lib.co_expr(fp(X), fp(R), fp(T), C.c_long(rows), C.c_long(cols), fp(Y), C.byref(mse), C.byref(mae),
                         fp(gX), fp(gR))
        return Y, np.float32(mse.value), np.float32(mae.value), gX, gR

    # ---- the MNIST demo's path
    def compare(self, cmp, a, b=None, s=0.0):
        """cmp: 0 '>', 1 '<', 2 '==', 3 '>=', 4 '<=', 5 '!='; b an array of a's shape or None (compare with s)."""
        a = f32(a)
        out = np.empty(a.shape, np.uint8)
        self.lib.co_compare(C.c_int(cmp), fp(a), fp(f32(b)) if b is not None else None, C.c_float(s),
                            out.ctypes.data_as(C.c_void_p), C.c_long(a.size))
        return out

    # ---- tensors that are not fp32 (dtype codes: 1 double, 2 int32, 3 int64, 4 bool)
    def cast_from_f32(self, a, dtype):
        a = f32(a)
        out = np.empty(a.shape, NP_DTYPE[dtype])
        rc = self.lib.co_cast_from_f32(fp(a), out.ctypes.data_as(C.c_void_p), C.c_int(dtype), C.c_long(a.size))
        assert rc == 0
        return out

    def scalar_op_typed(self, x, dtype, op, s):
        """op: 0 '+', 1 '*', 2 '/'; returns None where the reference's process would stop (integer division by 0)."""
        x = np.ascontiguousarray(x, NP_DTYPE[dtype])
        out = np.empty_like(x)
        rc = self.lib.co_scalar_op_typed(x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), C.c_int(dtype), C.c_int(op),
                                         C.c_float(s), C.c_long(x.size))
        return out if rc == 0 else None

    def accumulate_typed(self, acc, val, dtype):
        acc = np.array(acc, NP_DTYPE[dtype])
        val = np.ascontiguousarray(val, NP_DTYPE[dtype])
        rc = self.lib.co_accumulate_typed(acc.ctypes.data_as(C.c_void_p), val.ctypes.data_as(C.c_void_p), C.c_int(dtype), C.c_long(acc.size))
        assert rc == 0
        return acc

    def softmax_f64(self, x, dim):
        x = np.ascontiguousarray(x, np.float64)
        out = np.empty_like(x)
        rows, cols = (1, x.size) if x.ndim == 1 else x.shape
        self.lib.co_softmax_f64(x.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p), C.c_long(rows), C.c_long(cols),
                                C.c_int(1 if x.ndim == 1 else dim))
        return out

    def typed(self, a, dtype, steps):
        """The fp32 array converted to dtype, then the steps [(what, scalar)] in order: 0 '+', 1 '*', 2 '/',
        3 zero(), 4 ones(), 5 softmax(dim = scalar).  None where a step has no defined result."""
        t = self.cast_from_f32(a, dtype)
        for what, s in steps:
            if what <= 2:
                t = self.scalar_op_typed(t, dtype, what, s)
                if t is None:
                    return None
            elif what == 3:
                t = np.zeros_like(t)
            elif what == 4:
                t = np.ones_like(t)
            else:
                t = self.softmax_f64(t, int(s))
        return t

    def expr_run(self, prog, inputs, n_out, rows, cols):
        """prog: [(op, dst, a, b, imm)] of the fused-expression opcodes; inputs: full [rows, cols] or
        row-vector [cols] arrays; returns (outputs, status)."""
        prog = list(prog)
        codes = np.ascontiguousarray([[q[0], q[1], q[2], q[3]] for q in prog], np.int32).reshape(-1, 4)
        imm = f32([q[4] for q in prog]) if prog else f32([0])
        ins = [f32(x) for x in inputs]
        outs = [np.zeros((rows, cols), np.float32) for _ in range(n_out)]
        pin = (C.c_void_p * max(1, len(ins)))(*[x.ctypes.data for x in ins])
        pout = (C.c_void_p * max(1, n_out))(*[x.ctypes.data for x in outs])
        status = C.c_int(0)
        self.lib.co_expr_run.restype = C.c_int
        rc = self.lib.co_expr_run(codes.ctypes.data_as(C.c_void_p), fp(imm), C.c_int(len(prog)), pin, C.c_int(len(ins)), pout,
                                  C.c_int(n_out), C.c_long(rows), C.c_long(cols), C.byref(status))
        assert rc == 0, rc
        return outs, status.value

    def u8_to_unit(self, src):
        src = np.ascontiguousarray(src, dtype=np.uint8)
        r = np.empty(src.shape, np.float32)
        self.lib.co_u8_to_unit(src.ctypes.data_as(C.POINTER(C.c_ubyte)), fp(r), C.c_long(src.size))
        return r

    def onehot(self, labels, classes):
        labels = f32(labels)
        r = np.empty((labels.size, classes), np.float32)
        self.lib.co_onehot(fp(labels), fp(r), C.c_long(labels.size), C.c_long(classes))
        return r

    def sgd_step(self, p, g, lr):
        p, g = f32(p).copy(), f32(g)
        self.lib.co_sgd_step(fp(p), fp(g), C.c_float(lr), C.c_long(p.size))
        return p

    def count_correct(self, pred, labels):
        pred, labels = f32(pred), f32(labels)
        self.lib.co_count_correct.restype = C.c_long
        return int(self.lib.co_count_correct(fp(pred), fp(labels), C.c_long(pred.shape[0]), C.c_long(pred.shape[1])))

    def mnist_train(self, images, labels, params, batch, steps, lr, strict_row0, stale_snapshot):
        """params = [W1, b1, W2, b2, W3, b3]; returns (losses, updated params)."""
        images, labels = f32(images), f32(labels)
        P = [f32(q).copy() for q in params]
        I, H1 = P[0].shape
        H2, Cn = P[4].shape
        losses = np.empty(steps, np.float32)
        self.lib.co_mnist_train(fp(images), fp(labels), C.c_long(images.shape[0]), C.c_long(I), C.c_long(H1),
                                C.c_long(H2), C.c_long(Cn), *[fp(q) for q in P], C.c_long(batch), C.c_long(steps),
                                C.c_float(lr), C.c_int(int(strict_row0)), C.c_int(int(stale_snapshot)), fp(losses))
        return losses, P

    def mnist_predict(self, x, params):
        x = f32(x)
        P = [f32(q) for q in params]
        I, H1 = P[0].shape
        H2, Cn = P[4].shape
        probs = np.empty((x.shape[0], Cn), np.float32)
        self.lib.co_mnist_predict(fp(x), C.c_long(x.shape[0]), C.c_long(I), C.c_long(H1), C.c_long(H2), C.c_long(Cn),
                                  *[fp(q) for q in P], fp(probs))
        return probs


def synthetic_digits(n, seed):
    """[n, 28, 28] uint8 images with a class-dependent bright patch over noise, and labels 0..9
    (a stand-in for the MNIST image files, which the reference does not ship)."""
    rng = np.random.default_rng(seed)
    labels = rng.integers(0, 10, n).astype(np.uint8)
    img = rng.integers(0, 96, (n, 28, 28)).astype(np.uint8)
    for i, c in enumerate(labels):
        r, col = 2 + 5 * (int(c) // 5) * 2, 1 + 5 * (int(c) % 5)
        img[i, r:r + 8, col:col + 6] = rng.integers(160, 256, (8, 6)).astype(np.uint8)
    return img, labels


def write_mnist_dir(directory, n_train=512, n_test=256):
    """The four IDX files of the MNIST demo, filled with synthetic_digits (seeds 1 and 2)."""
    tr_i, tr_l = synthetic_digits(n_train, 1)
    te_i, te_l = synthetic_digits(n_test, 2)
    write_idx_images(os.path.join(directory, "train-images-idx3-ubyte"), tr_i)
    write_idx_labels(os.path.join(directory, "train-labels-idx1-ubyte"), tr_l)
    write_idx_images(os.path.join(directory, "t10k-images-idx3-ubyte"), te_i)
    write_idx_labels(os.path.join(directory, "t10k-labels-idx1-ubyte"), te_l)
    return tr_i, tr_l, te_i, te_l


def libc_xavier(shape, fan_in, reseed=None):
    """The demo's weight initialisation (mnist/mnist.cpp:21-27) from the C library's rand():
    r = 2.0f * rand() / float(RAND_MAX) - 1.0f, w = r * sqrt(1.0f / fan_in), all in fp32."""
    libc = C.CDLL("libc.so.6")
    if reseed is not None:
        libc.srand(C.c_uint(reseed))
    n = int(np.prod(shape))
    raw = np.array([libc.rand() for _ in range(n)], dtype=np.int64)
    r = (np.float32(2.0) * raw.astype(np.float32)) / np.float32(2147483647) - np.float32(1.0)
    return (r.astype(np.float32) * np.sqrt(np.float32(1.0) / np.float32(fan_in))).astype(np.float32).reshape(shape)


# opcodes of the fused-expression programs (include/ctorch_amd.h, CTAMD_EX_*)
EX = dict(LOAD_FULL=0, LOAD_ROW=1, ADD=2, SUB=3, MUL=4, DIV=5, NEG=6, RELU=7, SIGMOID=8, TANH=9, SIN=10, COS=11,
          ADDS=12, MULS=13, DIVS=14, RSUBS=15, RELUMUL=16, DIVCHK=17, STORE=18, STORE_ZP=19)


def random_slot_program(seed, n_full=2, n_row=1, n_ops=20, n_out=2, slots=12):
    """A random well-formed fused-expression program: loads of every input, n_ops operators over
    slots that have been written (slots are overwritten freely), then n_out stores.  Inputs are
    ordered full tensors first, then row vectors.  Returns [(op, dst, a, b, imm)]."""
    rng = np.random.default_rng(seed)
    prog, written = [], []
    for k in range(n_full + n_row):
        prog.append((EX["LOAD_FULL"] if k < n_full else EX["LOAD_ROW"], k, k, 0, 0.0))
        written.append(k)
    binary = [EX[n] for n in ("ADD", "SUB", "MUL", "DIV", "RELUMUL")]
    unary = [EX[n] for n in ("NEG", "RELU", "SIGMOID", "TANH", "SIN", "COS")]
    scalar = [EX[n] for n in ("ADDS", "MULS", "DIVS", "RSUBS")]
    for _ in range(n_ops):
        r = rng.integers(0, 10)
        dst = int(rng.integers(0, slots))
        a, b = int(rng.choice(written)), int(rng.choice(written))
        if r < 4:
            prog.append((int(rng.choice(binary)), dst, a, b, 0.0))
        elif r < 8:
            prog.append((int(rng.choice(unary)), dst, a, 0, 0.0))
        else:
            prog.append((int(rng.choice(scalar)), dst, a, 0, float(np.float32(0.5 + 0.25 * rng.integers(0, 8)))))
        if dst not in written:
            written.append(dst)
    prog.append((EX["DIVCHK"], 0, int(rng.choice(written)), 0, 0.0))
    for k in range(n_out):
        prog.append((EX["STORE_ZP"] if k % 2 else EX["STORE"], k, int(written[-1 - k % len(written)]), 0, 0.0))
    return prog


def random_program(seed, rows=6, cols=8, n_in=4, n_ops=14):
    """A random straight-line program for the tape tests: (kinds, ops).  Inputs 0..n_in-1 (kind 0 =
    [rows, cols], 1 = row vector; input 0 is always full, the last input is a positive divisor), ops
    = (code, a, b) as the program entry points of the two C doorways understand them.  Values are
    re-used freely, so nodes receive several gradient contributions; some ops use one value twice."""
    rng = np.random.default_rng(seed)
    kinds = [0] + [int(rng.integers(0, 4) == 0) for _ in range(n_in - 2)] + [0]
    vals = list(kinds)                          # kind of every value so far
    ops = []
    full = lambda: [i for i, k in enumerate(vals) if k == 0]
    vecs = lambda: [i for i, k in enumerate(vals) if k == 1]
    for step in range(n_ops):
        r = rng.integers(0, 10)
        if r < 5:                                # binary
            code = int(rng.integers(0, 4))
            if code == 3:                        # Div: only by the positive input, same shape
                a, b = int(rng.choice(full())), n_in - 1
            elif code == 0 and vecs() and rng.integers(0, 2):
                a, b = int(rng.choice(full())), int(rng.choice(vecs()))       # full + row vector
            else:
                pool = full() if (not vecs() or rng.integers(0, 3)) else vecs()
                a = int(rng.choice(pool))
                b = a if rng.integers(0, 6) == 0 else int(rng.choice(pool))  # now and then x (op) x
            ops.append((code, a, b))
            vals.append(vals[a])
        elif r < 8:                              # unary
            a = int(rng.integers(0, len(vals)))
            ops.append((int(rng.choice([20, 21, 22, 23, 24, 25])), a, 0))
            vals.append(vals[a])
        else:                                    # scalar
            a = int(rng.integers(0, len(vals)))
            ops.append((int(rng.choice([30, 31])), a, int(rng.integers(0, 6))))   # no tensor / scalar: the reference's gradient of it reads out of bounds
            vals.append(vals[a])
    # fold every value that nothing has consumed into the result, so that no input is dead code and
    # the last value is a full tensor
    used = {a for _, a, _ in ops} | {b for c, _, b in ops if c < 20}
    acc = full()[-1]
    for i in range(len(vals) - 1, -1, -1):
        if i in used or i == acc:
            continue
        ops.append((0, acc, i) if vals[i] == 1 or vals[acc] == 0 else (0, i, acc))
        vals.append(0)
        acc = len(vals) - 1
    if acc != len(vals) - 1:
        ops.append((30, acc, 0))
        vals.append(0)
    return kinds, ops


def program_fp64(inputs, kinds, ops, w, row0=True, same_operand_as_first=True):
    """The same program by a small fp64 reverse-mode interpreter (an independent statement of the
    mathematics).  row0: the gradient of a row vector added to a full tensor is row 0 of the upstream
    gradient, as the reference computes it; False gives the column sum.  same_operand_as_first: in
    x - x and x / x the reference treats both visits of the operand as the first one (it tells
    operands apart by tensor id, src/AutoDiff.cpp:1222-1233, :1259-1316), giving 2g and 2g/x where
    the mathematics gives 0.  Returns (y, L, grads)."""
    v = [np.asarray(x, np.float64) for x in inputs]
    for code, a, b in ops:
        x = v[a]
        if code < 20:
            z = v[b]
            v.append(x + z if code == 0 else x - z if code == 1 else x * z if code == 2 else x / z)
        elif code < 30:
            v.append({20: lambda t: -t, 21: lambda t: np.maximum(t, 0), 22: np.sin, 23: np.cos, 24: np.tanh,
                      25: lambda t: 1 / (1 + np.exp(-t))}[code](x))
        else:
            sc = 0.5 + 0.25 * b
            v.append(x + sc if code == 30 else x * sc)
    g = [np.zeros_like(t) for t in v]
    g[-1] = np.asarray(w, np.float64).copy()

    def push(i, val):
        if g[i].shape != val.shape:
            val = val[0] if row0 else val.sum(0)
        g[i] = g[i] + val

    for k in range(len(ops) - 1, -1, -1):
        code, a, b = ops[k]
        out = len(inputs) + k
        go, x = g[out], v[a]
        if code == 0:
            push(a, go); push(b, go)
        elif code == 1:
            push(a, go); push(b, go if (a == b and same_operand_as_first) else -go)
        elif code == 2:
            push(a, go * v[b]); push(b, go * x)
        elif code == 3:
            push(a, go / v[b]); push(b, go / v[b] if (a == b and same_operand_as_first) else -x * go / (v[b] * v[b]))
        elif code == 20:
            push(a, -go)
        elif code == 21:
            push(a, go * (x > 0))
        elif code == 22:
            push(a, go * np.cos(x))
        elif code == 23:
            push(a, -go * np.sin(x))
        elif code == 24:
            push(a, go * (1 - np.tanh(x) ** 2))
        elif code == 25:
            sg = 1 / (1 + np.exp(-x))
            push(a, go * sg * (1 - sg))
        elif code == 30:
            push(a, go)
        else:
            push(a, go * (0.5 + 0.25 * b))
    return v[-1], float((v[-1] * np.asarray(w, np.float64)).sum()), g[:len(inputs)]


def program_inputs(oracle, seed, kinds, rows, cols):
    xs = []
    for i, k in enumerate(kinds):
        shape = (cols,) if k else (rows, cols)
        lo, hi = (0.5, 2.0) if i == len(kinds) - 1 else (-1.5, 1.5)
        xs.append(oracle.uniform(shape, 7000 + 10 * seed + i, lo, hi))
    return xs, oracle.uniform((rows, cols), 7000 + 10 * seed + 9, -1, 1)


def write_idx_images(path, pixels_u8):
    """IDX3 file as the MNIST loader reads it (mnist/mnist_loader.cpp:7-44): big-endian magic 2051,
    count, rows, cols, then one unsigned byte per pixel.  pixels_u8: [n, rows, cols] uint8."""
    a = np.ascontiguousarray(pixels_u8, dtype=np.uint8)
    with open(path, "wb") as f:
        f.write(np.array([2051, a.shape[0], a.shape[1], a.shape[2]], dtype=">i4").tobytes())
        f.write(a.tobytes())


def write_idx_labels(path, labels_u8):
    """IDX1 file (mnist/mnist_loader.cpp:46-73): big-endian magic 2049, count, one byte per label."""
    a = np.ascontiguousarray(labels_u8, dtype=np.uint8)
    with open(path, "wb") as f:
        f.write(np.array([2049, a.shape[0]], dtype=">i4").tobytes())
        f.write(a.tobytes())


def ref_available():
    return os.path.exists(os.path.join(ORACLE_DIR, "_ref", "libctorch_ref.so"))


def _dims(shape):
    arr = (C.c_long * max(len(shape), 1))(*shape)
    return arr, len(shape)


class _Lib:
    """Maps lib.ref_<name> to <prefix><name> of a loaded library."""

    def __init__(self, cdll, prefix):
        self._cdll, self._prefix = cdll, prefix

    def __getattr__(self, name):
        assert name.startswith("ref_")
        return getattr(self._cdll, self._prefix + name[4:])


class Reference:
    """The real reference library through oracle/ref_driver.cpp.  Exists only where it was built.

    HostLayer (below) drives this repository's C++ front-end on the GPU through entry points of the
    same shape, so the methods here serve both."""

    ENTRY_POINTS = ("binary", "unary", "scalar", "sum", "softmax", "matmul_t", "grad_unary", "grad_softmax",
                    "grad_binary", "grad_loss", "chain", "mlp_step", "expr", "typed", "typed_grad")

    def __init__(self, path=None, prefix="ref_"):
        cdll = C.CDLL(path or os.path.join(ORACLE_DIR, "_ref", "libctorch_ref.so"))
        self.cdll = cdll
        self.lib = _Lib(cdll, prefix)
        for n in self.ENTRY_POINTS:
            getattr(cdll, prefix + n).restype = C.c_long
        self.lib.ref_quiet()

    def binary(self, code, a, b, out_shape):
        a, b = f32(a), f32(b)
        ad, an = _dims(a.shape)
        bd, bn = _dims(b.shape)
        out = np.empty(out_shape, np.float32)
        rc = self.lib.ref_binary(code, fp(a), ad, an, fp(b), bd, bn, fp(out))
        return rc, out

    def unary(self, code, a):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty_like(a)
        rc = self.lib.ref_unary(code, fp(a), ad, an, fp(out))
        assert rc == a.size, rc
        return out

    def scalar(self, which, a, s):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty_like(a)
        rc = self.lib.ref_scalar(which, fp(a), ad, an, C.c_float(s), fp(out))
        return rc, out

    def typed(self, a, dtype, steps):
        """The fp32 array converted by Tensor::to(dtype), then the steps [(what, scalar)] in order (see
        Oracle.typed); returns (rc, result)."""
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty(a.shape, NP_DTYPE[dtype])
        whats = (C.c_int * max(1, len(steps)))(*[w for w, _ in steps])
        scalars = (C.c_float * max(1, len(steps)))(*[s for _, s in steps])
        rc = self.lib.ref_typed(fp(a), ad, C.c_int(an), C.c_int(dtype), whats, scalars, C.c_int(len(steps)),
                                out.ctypes.data_as(C.c_void_p))
        return rc, out

    def typed_grad(self, a, dtype, steps):
        """backward() through scalar operators ([(what, scalar)], 0 '+', 1 '*', 2 '/') on to(dtype) of a:
        returns (rc, dtype code of the gradient, its bytes)."""
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.zeros(a.size * 8, np.uint8)
        code = C.c_int(-1)
        whats = (C.c_int * len(steps))(*[w for w, _ in steps])
        scalars = (C.c_float * len(steps))(*[s for _, s in steps])
        rc = self.lib.ref_typed_grad(fp(a), ad, C.c_int(an), C.c_int(dtype), whats, scalars, C.c_int(len(steps)),
                                     out.ctypes.data_as(C.c_void_p), C.byref(code))
        return rc, code.value, out

    def sum(self, a):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty((), np.float32)
        rc = self.lib.ref_sum(fp(a), ad, an, out.ctypes.data_as(FP))
        assert rc == 1
        return np.float32(out)

    def softmax(self, a, dim):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty_like(a)
        rc = self.lib.ref_softmax(fp(a), ad, an, dim, fp(out))
        assert rc == a.size
        return out

    def matmul_t(self, a, ta, b, tb):
        a, b = f32(a), f32(b)
        m = a.shape[1] if ta else a.shape[0]
        n = b.shape[0] if tb else b.shape[1]
        out = np.empty((m, n), np.float32)
        rc = self.lib.ref_matmul_t(fp(a), C.c_long(a.shape[0]), C.c_long(a.shape[1]), int(ta), fp(b),
                                   C.c_long(b.shape[0]), C.c_long(b.shape[1]), int(tb), fp(out))
        assert rc == m * n, rc
        return out

    def grad_unary(self, code, x, w):
        x, w = f32(x), f32(w)
        xd, xn = _dims(x.shape)
        dx = np.empty_like(x)
        rc = self.lib.ref_grad_unary(code, fp(x), xd, xn, fp(w), fp(dx))
        assert rc == x.size, rc
        return dx

    def grad_softmax(self, x, dim, w):
        x, w = f32(x), f32(w)
        xd, xn = _dims(x.shape)
        dx = np.empty_like(x)
        rc = self.lib.ref_grad_softmax(fp(x), xd, xn, dim, fp(w), fp(dx))
        assert rc == x.size, rc
        return dx

    def grad_binary(self, code, a, b, w):
        a, b, w = f32(a), f32(b), f32(w)
        ad, an = _dims(a.shape)
        bd, bn = _dims(b.shape)
        wd, wn = _dims(w.shape)
        da, db = np.empty_like(a), np.empty_like(b)
        rc = self.lib.ref_grad_binary(code, fp(a), ad, an, fp(b), bd, bn, fp(w), wd, wn, fp(da), fp(db))
        return rc, da, db

    def grad_loss(self, code, p, t, scale):
        p, t = f32(p), f32(t)
        pd, pn = _dims(p.shape)
        td, tn = _dims(t.shape)
        loss = C.c_float(0)
        dp = np.empty_like(p)
        rc = self.lib.ref_grad_loss(code, fp(p), pd, pn, fp(t), td, tn, C.c_float(scale), C.byref(loss), fp(dp))
        return rc, np.float32(loss.value), dp

    def adjust_grad_shape(self, g, target_shape):
        """The gradient a root of `target_shape` holds after backward(root, grad_output = g): the
        reference's check_and_adjust_grad_shape (src/AutoDiff.cpp:562-1049) through its public door
        (:1124-1126).  None when the call failed."""
        gshape = np.shape(g)                      # (a 0-D array would come out of f32() as [1])
        g = f32(g).reshape(-1)
        out = np.empty(target_shape, np.float32)
        gd, gn = _dims(gshape)
        td, tn = _dims(tuple(target_shape))
        n = self.lib.ref_adjust_grad_shape(fp(g), gd, gn, td, tn, fp(out.reshape(-1)))
        return out if n == out.size else None

    def chain(self, a, b):
        a, b = f32(a), f32(b)
        s = C.c_float(0)
        ga, gb = np.empty_like(a), np.empty_like(b)
        rc = self.lib.ref_chain(fp(a), fp(b), C.c_long(a.size), C.byref(s), fp(ga), fp(gb))
        assert rc == a.size
        return np.float32(s.value), ga, gb

    def mlp_step(self, x, W1, b1, W2, b2, target, *extra):
        x, W1, b1, W2, b2, target = map(f32, (x, W1, b1, W2, b2, target))
        B, I = x.shape
        H = W1.shape[1]
        Cn = W2.shape[1]
        loss = C.c_float(0)
        logits = np.empty((B, Cn), np.float32)
        gW1, gb1, gW2, gb2 = (np.empty_like(t) for t in (W1, b1, W2, b2))
        rc = self.lib.ref_mlp_step(fp(x), C.c_long(B), C.c_long(I), fp(W1), fp(b1), C.c_long(H), fp(W2), fp(b2),
                                   C.c_long(Cn), fp(target), C.byref(loss), fp(logits), fp(gW1), fp(gb1),
                                   fp(gW2), fp(gb2), *extra)
        assert rc == B, rc
        return np.float32(loss.value), logits, gW1, gb1, gW2, gb2

    def expr(self, X, R, T, *extra):
        X, R, T = f32(X), f32(R), f32(T)
        rows, cols = X.shape
        Y, gX, gR = np.empty_like(X), np.empty_like(X), np.empty_like(R)
        mse, mae = C.c_float(0), C.c_float(0)
        rc = self.lib.ref_expr(fp(X), fp(R), fp(T), C.c_long(rows), C.c_long(cols), fp(Y), C.byref(mse),
                               C.byref(mae), fp(gX), fp(gR), *extra)
        assert rc == rows * cols, rc
        return Y, np.float32(mse.value), np.float32(mae.value), gX, gR

    def program(self, inputs, kinds, ops, w):
        """Runs a straight-line program (see random_program) through the tape; returns
        (rc, last value, L, [gradients of the inputs])."""
        rows, cols = w.shape
        flat = np.concatenate([f32(x).ravel() for x in inputs])
        kinds_a = (C.c_int * len(kinds))(*kinds)
        ops_a = (C.c_int * (3 * len(ops)))(*[v for op in ops for v in op])
        y = np.empty((rows, cols), np.float32)
        L = C.c_float(0)
        grads = np.empty(flat.size, np.float32)
        fn = self.lib.ref_program
        fn.restype = C.c_long
        rc = fn(fp(flat), kinds_a, C.c_int(len(kinds)), ops_a, C.c_int(len(ops)), fp(f32(w)), C.c_long(rows),
                C.c_long(cols), fp(y), C.byref(L), fp(grads))
        out, pos = [], 0
        for x in inputs:
            out.append(grads[pos:pos + x.size].reshape(x.shape).copy())
            pos += x.size
        return rc, y, np.float32(L.value), out

    # ---- the MNIST demo (oracle/ref_mnist_driver.cpp); reference build only
    def mnist_load(self, directory, train):
        dims = (C.c_long * 2)()
        self.lib.ref_mnist_load.restype = C.c_long
        n = self.lib.ref_mnist_load(directory.encode(), C.c_int(int(train)), None, None, dims)
        assert n >= 0, n
        images = np.empty((dims[0], dims[1]), np.float32)
        labels = np.empty(n, np.float32)
        self.lib.ref_mnist_load(directory.encode(), C.c_int(int(train)), fp(images), fp(labels), dims)
        return images, labels

    def mnist_accuracy(self, pred, labels):
        pred, labels = f32(pred), f32(labels)
        self.lib.ref_mnist_accuracy.restype = C.c_float
        return np.float32(self.lib.ref_mnist_accuracy(fp(pred), fp(labels), C.c_long(pred.shape[0])))

    def mnist_get_batch(self, images, labels, batch, idx):
        images, labels = f32(images), f32(labels)
        n, px = images.shape
        bi, bl = np.empty((batch, px), np.float32), np.empty(batch, np.float32)
        self.lib.ref_mnist_get_batch.restype = C.c_long
        got = self.lib.ref_mnist_get_batch(fp(images), fp(labels), C.c_long(n), C.c_long(px), C.c_long(batch),
                                            C.c_long(idx), fp(bi), fp(bl))
        return bi[:got], bl[:got]

    def mnist_xavier(self, shape, fan_in, reseed=None):
        w = np.empty(shape, np.float32)
        self.lib.ref_mnist_xavier(fp(w), C.c_long(w.size), C.c_long(fan_in), C.c_int(reseed is not None),
                                   C.c_uint(reseed or 0))
        return w

    def mnist_train(self, images, labels, params, batch, steps, lr):
        images, labels = f32(images), f32(labels)
        P = [f32(q).copy() for q in params]
        I, H1 = P[0].shape
        H2, Cn = P[4].shape
        losses = np.empty(steps, np.float32)
        self.lib.ref_mnist_train.restype = C.c_long
        rc = self.lib.ref_mnist_train(fp(images), fp(labels), C.c_long(images.shape[0]), C.c_long(I), C.c_long(H1),
                                      C.c_long(H2), C.c_long(Cn), *[fp(q) for q in P], C.c_long(batch),
                                      C.c_long(steps), C.c_float(lr), *self._train_extra(), fp(losses),
                                      *self._train_tail())
        assert rc == steps, rc
        return losses, P

    def _train_extra(self):
        return ()

    def _train_tail(self):
        return ()

    def mnist_main_in(self, directory):
        return int(self.lib.ref_mnist_main_in(directory.encode()))


HOST_LIB = os.path.join(ROOT, "ctorch_amd", "host", "tests", "harness", "libctorch_amd_harness.so")


class HostLayer(Reference):
    """This repository's C++ front-end (Tensor / Ctorch_Scheduler / AutoDiff over the HIP launch layer)
    through the test doorway ctorch_amd/host/tests/harness/capi_host.cpp.  Needs a GPU for every call."""

    DECLARED = {"abs": 40, "exp": 41, "log": 42, "sqrt": 43, "square": 44, "tan": 45, "leaky_relu": 46, "sub_scalar": 47,
                "lrelu_dispatch": 48}
    REDUCE = {"sum": 0, "mean": 1, "max": 2, "min": 3, "var": 4, "std": 5}

    def __init__(self):
        Reference.__init__(self, HOST_LIB, "cth_")
        for n in ("declared_unary", "grad_declared_unary", "reduce", "grad_reduce", "log_softmax", "grad_log_softmax",
                  "adjust_grad_shape", "grad_dot"):
            getattr(self.cdll, "cth_" + n).restype = C.c_long

    # ---- the methods the reference declares without defining them
    def declared_unary(self, name, a, p=0.0):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty_like(a)
        rc = self.cdll.cth_declared_unary(self.DECLARED[name], fp(a), ad, an, C.c_float(p), fp(out))
        return out if rc == a.size else None

    def grad_declared_unary(self, name, x, w, p=0.0):
        x, w = f32(x), f32(w)
        xd, xn = _dims(x.shape)
        dx = np.empty_like(x)
        rc = self.cdll.cth_grad_declared_unary(self.DECLARED[name], fp(x), xd, xn, C.c_float(p), fp(w), fp(dx))
        return dx if rc == x.size else None

    def reduce(self, kind, a, dims=(), keepdim=False, ddof=-1):
        """-> the result with its shape, or None when the call threw"""
        ashape = np.shape(a)                      # (a 0-D array would come out of f32() as [1])
        a = f32(a).reshape(-1)
        ad, an = _dims(ashape)
        ds = (C.c_int * max(1, len(dims)))(*dims)
        out = np.empty(max(1, a.size), np.float32)
        od = (C.c_long * 8)()
        orank = C.c_int(0)
        rc = self.cdll.cth_reduce(self.REDUCE[kind], fp(a), ad, an, ds, len(dims), int(keepdim), ddof, fp(out), od, C.byref(orank))
        if rc < 0:
            return None
        shape = tuple(od[i] for i in range(orank.value))
        return out[:rc].reshape(shape)

    def grad_reduce(self, kind, x, w, dims=(), keepdim=False, ddof=-1):
        xshape = np.shape(x)
        x, w = f32(x).reshape(-1), f32(w).reshape(-1)
        xd, xn = _dims(xshape)
        ds = (C.c_int * max(1, len(dims)))(*dims)
        dx = np.empty_like(x)
        rc = self.cdll.cth_grad_reduce(self.REDUCE[kind], fp(x), xd, xn, ds, len(dims), int(keepdim), ddof, fp(w), fp(dx))
        return dx.reshape(xshape) if rc == x.size else None

    def log_softmax(self, a, dim):
        a = f32(a)
        ad, an = _dims(a.shape)
        out = np.empty_like(a)
        rc = self.cdll.cth_log_softmax(fp(a), ad, an, dim, fp(out))
        return out if rc == a.size else None

    def grad_log_softmax(self, x, dim, w):
        x, w = f32(x), f32(w)
        xd, xn = _dims(x.shape)
        dx = np.empty_like(x)
        rc = self.cdll.cth_grad_log_softmax(fp(x), xd, xn, dim, fp(w), fp(dx))
        return dx if rc == x.size else None

    def grad_dot(self, a, b, scale):
        a, b = f32(a), f32(b)
        da, db = np.empty_like(a), np.empty_like(b)
        value = C.c_float(0)
        rc = self.cdll.cth_grad_dot(fp(a), fp(b), C.c_long(a.size), C.c_float(scale), C.byref(value), fp(da), fp(db))
        assert rc == 2 * a.size, rc
        return np.float32(value.value), da, db

    def set_reference_row0(self, on):
        self.cdll.cth_set_reference_row0(int(on))

    def set_ce_one_pass(self, on):
        self.cdll.cth_set_ce_one_pass(int(on))

    def set_inputs_unseen(self, on):
        """Inputs then reach the front-end as if the device had computed them: what the upload saw of
        them (class indices in range or not) is forgotten, and range checks run on the device."""
        self.cdll.cth_set_inputs_unseen(int(on))

    def compare(self, cmp, a, b=None, s=0.0):
        """The Tensor comparison operators on the device; returns the bool tensor as uint8, or the
        negative return code."""
        a = f32(a)
        out = np.empty(a.shape, np.uint8)
        ad = (C.c_long * a.ndim)(*a.shape)
        if b is not None:
            b = f32(b)
            bd = (C.c_long * b.ndim)(*b.shape)
            rc = self.cdll.cth_compare(C.c_int(cmp), fp(a), ad, C.c_int(a.ndim), fp(b), bd, C.c_int(b.ndim), C.c_float(0),
                                       out.ctypes.data_as(C.c_void_p))
        else:
            rc = self.cdll.cth_compare(C.c_int(cmp), fp(a), ad, C.c_int(a.ndim), None, None, C.c_int(0), C.c_float(s),
                                       out.ctypes.data_as(C.c_void_p))
        return out if rc == a.size else rc

    def expr_graph(self, X1, X2, r, T):
        """The fused config-5 expression in a recorded step: eager on X1, recorded, replayed on X1 and
        (after overwriting the staged input) on X2.  Returns (rc, y1, gx1, y2, gx2)."""
        X1, X2, r, T = f32(X1), f32(X2), f32(r), f32(T)
        rows, cols = X1.shape
        outs = [np.empty_like(X1) for _ in range(4)]
        self.cdll.cth_expr_graph.restype = C.c_long
        rc = self.cdll.cth_expr_graph(fp(X1), fp(X2), fp(r), fp(T), C.c_long(rows), C.c_long(cols), *[fp(o) for o in outs])
        return (rc, *outs)

    def graph_hardening(self, X, X2):
        """Two graphs replayed alternately without host waits, a parameter read after an in-place SGD
        step, a thread's first backward() inside a recording, a DeviceGraph re-recorded after a failed
        recording.  Returns (rc, out[7])."""
        X, X2 = f32(X), f32(X2)
        out = np.zeros(7, dtype=np.float32)
        self.cdll.cth_graph_hardening.restype = C.c_long
        rc = self.cdll.cth_graph_hardening(fp(X), fp(X2), C.c_long(X.size), fp(out))
        return rc, out

    def ce_kept_cap(self, x1, x2, labels):
        """CrossEntropy gradients of two logits matrices under three caps on kept one-pass gradients.
        Returns (rc, g1, g2); rc == 0: the runs agree (see cth_ce_kept_cap)."""
        x1, x2, labels = f32(x1), f32(x2), f32(labels)
        rows, cols = x1.shape
        g1, g2 = np.empty_like(x1), np.empty_like(x2)
        self.cdll.cth_ce_kept_cap.restype = C.c_long
        rc = self.cdll.cth_ce_kept_cap(fp(x1), fp(x2), fp(labels), C.c_long(rows), C.c_long(cols), fp(g1), fp(g2))
        return rc, g1, g2

    def set_fused_expr(self, on):
        """chain, expr, program and their timed versions evaluate their elementwise part as one fused
        expression (Expr::eval): one launch forward, one backward."""
        self.cdll.cth_set_fused_expr(int(on))

    def last_expr_stats(self):
        """(forward instructions, forward slots, backward instructions, backward slots) of the programs the
        last fused expression compiled; zeros when it was evaluated operator by operator."""
        out = (C.c_int * 4)()
        self.cdll.cth_last_expr_stats(out)
        return tuple(out)

    def set_fused_layers(self, on):
        """mlp_step builds each layer with Tensor::linear (matmul + bias + ReLU as one operator)."""
        self.cdll.cth_set_fused_layers(int(on))

    def set_fused_head(self, on):
        """With fused layers: the last layer and its class-index cross entropy as one operator
        (Tensor::linear_cross_entropy) in mlp_step and time_mlp."""
        self.cdll.cth_set_fused_head(int(on))

    def head_fusion(self, x, W1, b1, W2, b2, W3, b3, labels, tol, scale=3.0):
        """cth_head_fusion: (rc, worst ratio, launches with the one-pass head, without)."""
        x, W1, b1, W2, b2, W3, b3, labels = map(f32, (x, W1, b1, W2, b2, W3, b3, labels))
        out = (C.c_double * 3)(0, 0, 0)
        self.cdll.cth_head_fusion.restype = C.c_long
        rc = self.cdll.cth_head_fusion(fp(x), C.c_long(x.shape[0]), C.c_long(x.shape[1]), fp(W1), fp(b1), C.c_long(W1.shape[1]), fp(W2),
                                       fp(b2), C.c_long(W2.shape[1]), fp(W3), fp(b3), C.c_long(W3.shape[1]), fp(labels),
                                       C.c_double(tol), C.c_float(scale), out)
        return rc, out[0], out[1], out[2]

    def set_bias_grad_with_weight_grad(self, on):
        """The bias gradient of a fused layer with its weight gradient (the default) or on its own."""
        self.cdll.cth_set_bias_grad_with_weight_grad(int(on))

    def time_mlp(self, x, W1, b1, W2, b2, labels, warm=2, steps=3):
        """One class-index training step timed by the harness: (ms per step, operator launches per step)."""
        x, W1, b1, W2, b2, labels = map(f32, (x, W1, b1, W2, b2, labels))
        out = (C.c_double * 6)()
        L = C.c_long
        rc = self.cdll.cth_time_mlp(fp(x), L(x.shape[0]), L(x.shape[1]), fp(W1), fp(b1), L(W1.shape[1]), fp(W2), fp(b2),
                                    L(W2.shape[1]), fp(labels), C.c_int(warm), C.c_int(steps), out)
        assert rc == steps, rc
        return out[0], int(out[4])

    def mlp_step(self, x, W1, b1, W2, b2, target, target_is_index=False):
        return Reference.mlp_step(self, x, W1, b1, W2, b2, target, C.c_int(int(target_is_index)))

    def expr(self, X, R, T, expect_failure=False):
        """R may be the full [rows, cols] operand or the row vector [cols] (row-broadcast Div).
        expect_failure: the call must report an exception (returns None)."""
        if expect_failure:
            try:
                Reference.expr(self, X, R, T, C.c_int(int(np.ndim(R) == 1)))
            except AssertionError as e:
                assert e.args and e.args[0] == -1, e.args
                return None
            raise AssertionError("the call succeeded")
        return Reference.expr(self, X, R, T, C.c_int(int(np.ndim(R) == 1)))

    # ---- the MNIST demo's path on the device
    reference_tape = True     # mnist_train: the reference's tape properties, or live leaves + column sums
    last_train_ms = 0.0

    def _train_extra(self):
        return (C.c_int(int(self.reference_tape)),)

    def _train_tail(self):
        self._ms = C.c_double(0)
        return (C.byref(self._ms),)

    def mnist_train(self, images, labels, params, batch, steps, lr, reference_tape=True):
        self.reference_tape = reference_tape
        out = Reference.mnist_train(self, images, labels, params, batch, steps, lr)
        self.last_train_ms = self._ms.value
        return out

    def mnist_predict(self, x, params):
        x = f32(x)
        P = [f32(q) for q in params]
        I, H1 = P[0].shape
        H2, Cn = P[4].shape
        probs = np.empty((x.shape[0], Cn), np.float32)
        self.cdll.cth_mnist_predict.restype = C.c_long
        rc = self.cdll.cth_mnist_predict(fp(x), C.c_long(x.shape[0]), C.c_long(I), C.c_long(H1), C.c_long(H2),
                                         C.c_long(Cn), *[fp(q) for q in P], fp(probs))
        assert rc == probs.size, rc
        return probs

    def mnist_demo(self, directory, epochs=5, batch=128, lr=0.01, hidden1=128, hidden2=64, reference_tape=False):
        """reference_tape: False / True, or 2 for live leaves with the step replayed from a recorded graph."""
        losses = np.empty(epochs, np.float32)
        acc = np.empty(2, np.float32)
        sec = C.c_double(0)
        self.cdll.cth_mnist_demo.restype = C.c_long
        rc = self.cdll.cth_mnist_demo(directory.encode(), C.c_int(epochs), C.c_int(batch), C.c_float(lr),
                                      C.c_int(hidden1), C.c_int(hidden2), C.c_int(int(reference_tape)), fp(losses),
                                      fp(acc), C.byref(sec))
        return rc, losses, acc, sec.value


# ----------------------------------------------------------------- tensors that are not fp32
TYPED_EDGE = np.array([0.0, -0.0, 1.5, -1.5, 2.9, -2.9, 3e9, -3e9, 1e19, -1e19, np.nan, np.inf, -np.inf, 2147483520.0,
                       -2147483648.0, 2147483648.0, 9.2233715e18, 9.223372e18, -9.223372e18, 1e-40, 0.99, -0.99, 16777216.0,
                       1e10, -1e10, 255.0, 1.0], np.float32)


def typed_cases(o):
    """[(name, fp32 input, dtype, steps)] for Oracle.typed / Reference.typed: conversions of edge values,
    every scalar operator on every arithmetic dtype (scalars that truncate, wrap and change sign), zero / ones,
    and the double softmax along both dimensions."""
    cases = []
    wide = np.concatenate([TYPED_EDGE, o.normal((997,), 71, 0, 1000), o.normal((300,), 72, 0, 3e9)]).astype(np.float32)
    for dt in (1, 2, 3, 4):
        cases.append(("cast_%d" % dt, wide, dt, []))
        cases.append(("zero_%d" % dt, wide[:37], dt, [(3, 0.0)]))
        cases.append(("ones_%d" % dt, wide[:37], dt, [(4, 0.0)]))
    vals = o.normal((1031,), 73, 0, 40000)
    scalars = [(0, 2.7), (0, -1e10), (0, 3e9), (1, -3.9), (1, 1e6), (1, 0.3), (1, 123456.0), (2, 2.5), (2, -1.0), (2, -7.9), (2, 1e-3),
               (2, 3e9)]
    for dt in (1, 2, 3):
        for k, (what, sc) in enumerate(scalars):
            if dt != 1 and what == 2 and abs(sc) < 1:
                continue                               # integer division by 0: the reference's process stops
            cases.append(("scalar_%d_%d" % (dt, k), vals, dt, [(what, sc)]))
        cases.append(("chain_%d" % dt, vals, dt, [(1, 3.0), (0, -17.5), (2, 4.0), (1, 65537.0), (1, 65537.0), (0, 1.0)]))
    for shape, seed in (((37, 19), 74), ((5, 301), 75), ((64,), 76), ((1, 1), 77), ((130, 3), 78)):
        z = o.normal(shape, seed, 0, 3)
        for dim in ((0,) if len(shape) == 1 else (0, 1)):
            cases.append(("softmax_%s_%d" % ("x".join(map(str, shape)), dim), z, 1, [(1, 1.0000001), (0, 0.1), (5, float(dim))]))
    return cases

"""Per-kernel timings of the launch layer through the C ABI on one MI355X.

    python -m ctorch_amd.kernel_bench [--json] [--skip-matmul] [--only-matmul] [--only-expr] [--only-declared] [--only-mlp]

Every operator is launched on operands resident in HBM (torch only provides the memory and the
stream), timed with events over back-to-back launches after a warm-up, and reported as time,
achieved rate and fraction of the published peak (8 TB/s HBM, 157.3 TFLOP/s fp32 matrix), with the
algorithmic bytes per element each operator must move.  Operands rotate through four buffer sets so
that the 256 MiB memory-side cache cannot serve the traffic (a few rows say "one buffer set": the
same launch repeated over the same buffers, for comparison).  Run it under
`rocprofv3 --kernel-trace --stats` to get the same kernels' durations from the profiler.
"""
import argparse
import ctypes as C
import json
import sys
import time

HBM_PEAK = 8.0e12
MFMA_F32_PEAK = 157.3e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--json", action="store_true", help="one JSON object instead of a table")
    ap.add_argument("--skip-matmul", action="store_true")
    ap.add_argument("--only-expr", action="store_true", help="only the fused-expression programs (for counter runs)")
    ap.add_argument("--only-declared", action="store_true",
                    help="only the operators the reference declares without defining: abs .. leaky_relu, reductions along an axis, log_softmax")
    ap.add_argument("--only-matmul", action="store_true", help="only the fp32 MatMul rows")
    ap.add_argument("--only-mlp", action="store_true",
                    help="only the launches of one 784-256-10 training step at batch 256 and 8192 (the small-product kernels)")
    args = ap.parse_args()

    import torch
    from ctorch_amd import capi

    lib = capi.load()
    torch.cuda.init()
    torch.zeros(1, device="cuda:0")
    capi.check(lib.ctamd_init(0))
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: C.c_void_p(t.data_ptr())
    call = lambda name, *a: capi.check(getattr(lib, name)(*a))
    results = []

    # (the chip's clock keeps moving for about 25 ms after a change of load - up after idling, down and part of
    # the way back under heavy vector work: a run of fused config-5 launches reads 190, 174, 162, 155, 155, ... us
    # over successive 10 ms - so every row first keeps its launches coming for `settle` seconds)
    def timeit(fn, reps, warm=3, settle=0.03):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < settle:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

    def report(name, seconds, nbytes=None, flops=None):
        e = {"kernel": name, "us": round(seconds * 1e6, 1)}
        if nbytes is not None:
            e.update({"GB/s": round(nbytes / seconds / 1e9, 1), "frac_of_hbm_peak": round(nbytes / seconds / HBM_PEAK, 4)})
        if flops is not None:
            e.update({"TFLOP/s": round(flops / seconds / 1e12, 2), "frac_of_mfma_peak": round(flops / seconds / MFMA_F32_PEAK, 4)})
        results.append(e)
        if not args.json:
            rate = ("%8.1f GB/s %5.1f%% of 8 TB/s" % (e["GB/s"], 100 * e["frac_of_hbm_peak"]) if nbytes is not None else
                    "%8.2f TFLOP/s %5.1f%% of 157.3" % (e["TFLOP/s"], 100 * e["frac_of_mfma_peak"]))
            print("%-44s %9.1f us  %s" % (name, e["us"], rate), flush=True)

    # ---- fp32 MatMul, square, the three operand layouts
    # (the chip takes some tens of milliseconds of matrix work to reach its clocks: [2048]^3 measured right
    # after start reads 10% slower than the same launch a little later, so every row first launches for
    # 40 ms untimed)
    def warm_up(fn, seconds=0.04):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()

    def matmul_rows():
        for M in (1024, 2048, 4096, 8192):
            a, b = torch.randn(M, M, device="cuda"), torch.randn(M, M, device="cuda")
            c = torch.empty(M, M, device="cuda")
            for name, (x, y) in (("A.B", (a, b)), ("A.B^T", (a, b.t())), ("A^T.B", (a.t(), b))):
                fn = lambda x=x, y=y: call("ctamd_matmul_f32", P(x), x.stride(0), x.stride(1), P(y), y.stride(0), y.stride(1),
                                           P(c), M, M, M, S)
                warm_up(fn)
                report("matmul %s %d^3" % (name, M), timeit(fn, 20 if M < 8192 else 4, warm=2), flops=2.0 * M ** 3)
            del a, b, c
        # not square: a long K over one 64 x 64 tile per CU, and a K that ends inside a k tile
        for (m, n, k) in ((1024, 1024, 4096), (4096, 4096, 4088)):
            a, b, c = torch.randn(m, k, device="cuda"), torch.randn(k, n, device="cuda"), torch.empty(m, n, device="cuda")
            fn = lambda: call("ctamd_matmul_f32", P(a), k, 1, P(b), n, 1, P(c), m, n, k, S)
            warm_up(fn)
            report("matmul A.B [%d x %d, K = %d]" % (m, n, k), timeit(fn, 20, warm=2), flops=2.0 * m * n * k)
            del a, b, c

    # ---- the launches of one training step of the 784-256-10 perceptron, each on its own: the fused
    # layers forward, the class-index cross entropy with its gradient, the product with the ReLU mask,
    # the weight-gradient products and the bias-gradient column sums.  (Operands of a few MiB: they
    # stay cached from launch to launch, as they do inside a step.)
    def mlp_rows(batch):
        I, H, Cn = 784, 256, 10
        x = torch.rand(batch, I, device="cuda")
        W1, b1 = torch.randn(I, H, device="cuda") * 0.03, torch.zeros(H, device="cuda")
        W2, b2 = torch.randn(H, Cn, device="cuda") * 0.06, torch.zeros(Cn, device="cuda")
        h, z = torch.empty(batch, H, device="cuda"), torch.empty(batch, Cn, device="cuda")
        dz, dh = torch.randn(batch, Cn, device="cuda"), torch.empty(batch, H, device="cuda")
        gW1, gW2 = torch.empty(I, H, device="cuda"), torch.empty(H, Cn, device="cuda")
        gb1, gb2 = torch.empty(H, device="cuda"), torch.empty(Cn, device="cuda")
        labels = torch.randint(0, Cn, (batch,), device="cuda").float()
        loss, status = torch.empty(1, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
        mm = lambda a, b, c, m, n, k: call("ctamd_matmul_f32", P(a), a.stride(0), a.stride(1), P(b), b.stride(0), b.stride(1), P(c), m, n, k, S)
        tag = "MLP step, batch %d: " % batch
        def row(name, fn, flops=None, nbytes=None):
            report(tag + name, timeit(fn, 50, warm=10), nbytes=nbytes, flops=flops)
        row("h = relu(x.W1 + b1) [%d x 784].[784 x 256]" % batch,
            lambda: call("ctamd_matmul_bias_f32", P(x), I, 1, P(W1), H, 1, P(b1), 1, P(h), batch, H, I, S), flops=2.0 * batch * H * I)
        row("z = h.W2 + b2 [%d x 256].[256 x 10]" % batch,
            lambda: call("ctamd_matmul_bias_f32", P(h), H, 1, P(W2), Cn, 1, P(b2), 0, P(z), batch, Cn, H, S), flops=2.0 * batch * Cn * H)
        row("cross entropy (class index), loss + gradient [%d x 10]" % batch,
            lambda: call("ctamd_cross_entropy_index_fused_f32", P(z), P(labels), P(loss), P(status), P(dz), batch, Cn, S), nbytes=8.0 * batch * Cn)
        row("dh = (dz.W2^T) * [h > 0] [%d x 10].[10 x 256]" % batch,
            lambda: call("ctamd_matmul_relu_mask_f32", P(dz), Cn, 1, P(W2), 1, Cn, P(h), P(dh), batch, H, Cn, S), flops=2.0 * batch * H * Cn)
        row("gW2 = h^T.dz [256 x %d].[%d x 10]" % (batch, batch), lambda: mm(h.t(), dz, gW2, H, Cn, batch), flops=2.0 * batch * H * Cn)
        row("gb2 = column sums of dz [%d x 10]" % batch, lambda: call("ctamd_colsum_f32", P(dz), P(gb2), batch, Cn, S), nbytes=4.0 * batch * Cn)
        row("gW1 = x^T.dh [784 x %d].[%d x 256]" % (batch, batch), lambda: mm(x.t(), dh, gW1, I, H, batch), flops=2.0 * batch * H * I)
        row("gb1 = column sums of dh [%d x 256]" % batch, lambda: call("ctamd_colsum_f32", P(dh), P(gb1), batch, H, S), nbytes=4.0 * batch * H)
        # what the tape calls for a layer whose bias wants its gradient: both in one call (one launch while batch <= 512)
        mmcs = lambda a, b, c, sums, m, n, k: call("ctamd_matmul_colsum_f32", P(a), a.stride(0), a.stride(1), P(b), b.stride(0), b.stride(1),
                                                   P(c), P(sums), m, n, k, S)
        # the last layer, its cross entropy and the three gradients that leave them, in one pass over h
        pair = torch.zeros(2, device="cuda")
        row("z, loss, dz, dh, gW2, gb2 in one pass over h (the classifier head)",
            lambda: call("ctamd_linear_ce_head_f32", P(h), P(W2), P(b2), P(labels), P(pair), P(status), P(z), P(dz), P(dh), 1, P(gW2), P(gb2),
                         batch, H, Cn, S), flops=6.0 * batch * H * Cn)
        row("gW2 and gb2 in one call", lambda: mmcs(h.t(), dz, gW2, gb2, H, Cn, batch), flops=2.0 * batch * H * Cn)
        row("gW1 and gb1 in one call", lambda: mmcs(x.t(), dh, gW1, gb1, I, H, batch), flops=2.0 * batch * H * I)
    if args.only_matmul:
        matmul_rows()
        if args.json:
            print(json.dumps({"device": torch.cuda.get_device_name(0), "results": results}))
        return 0
    if args.only_mlp:
        for batch in (256, 8192):
            mlp_rows(batch)
        if args.json:
            print(json.dumps({"device": torch.cuda.get_device_name(0), "results": results}))
        return 0

    # ---- elementwise, scalar, fill, reductions: 2^26 elements (256 MiB per tensor), four buffer sets
    n, sets = 1 << 26, 4
    A = [torch.randn(n, device="cuda") for _ in range(sets)]
    B = [torch.randn(n, device="cuda").abs_() + 0.5 for _ in range(sets)]
    R = [torch.empty(n, device="cuda") for _ in range(sets)]
    out = torch.empty(1, device="cuda")
    turn = [0]

    def rotating(fn):
        def f():
            k = turn[0] % sets
            turn[0] += 1
            fn(k)
        return f

    def ew(name, fn, bytes_per_elem):
        report("%s, n=2^26 (%d B/elem)" % (name, bytes_per_elem), timeit(rotating(fn), 20), bytes_per_elem * n)

    plain = not args.only_expr and not args.only_declared
    for op in ("add", "sub", "mul", "div") if plain else ():
        ew(op, lambda k, op=op: call("ctamd_%s_f32" % op, P(A[k]), P(B[k]), P(R[k]), n, S), 12)
    for op in ("neg", "relu", "sin", "cos", "tanh", "sigmoid") if plain else ():
        ew(op, lambda k, op=op: call("ctamd_%s_f32" % op, P(A[k]), P(R[k]), n, S), 8)
    for op in ("relu", "sigmoid", "tanh", "sin", "cos") if plain else ():
        ew(op + " backward", lambda k, op=op: call("ctamd_%s_backward_f32" % op, P(A[k]), P(B[k]), P(R[k]), n, S), 12)
    if plain:
        ew("tensor + scalar", lambda k: call("ctamd_add_scalar_f32", P(A[k]), C.c_float(5.0), P(R[k]), n, S), 8)
        ew("fill", lambda k: call("ctamd_fill_f32", P(R[k]), C.c_float(5.0), n, S), 4)
        ew("accumulate", lambda k: call("ctamd_accumulate_f32", P(R[k]), P(A[k]), n, S), 12)
        ew("sgd step", lambda k: call("ctamd_sgd_step_f32", P(R[k]), P(A[k]), C.c_float(0.01), n, S), 12)
        ew("row-broadcast div [16384 x 4096]", lambda k: call("ctamd_div_rowbcast_f32", P(A[k]), P(B[0]), P(R[k]), 16384, 4096, S), 8)
        ew("sum", lambda k: call("ctamd_sum_f32", P(A[k]), P(out), n, S), 4)
        ew("dot", lambda k: call("ctamd_dot_f32", P(A[k]), P(B[k]), P(out), n, S), 8)
        ew("mse", lambda k: call("ctamd_mse_f32", P(A[k]), P(B[k]), P(out), n, S), 8)
        ew("mae", lambda k: call("ctamd_mae_f32", P(A[k]), P(B[k]), P(out), n, S), 8)
    # the operators the reference declares without defining: unary maps and their gradients ...
    if not args.only_expr:
        for op in ("abs", "exp", "log", "sqrt", "square", "tan"):
            src = B if op in ("log", "sqrt") else A
            ew(op, lambda k, op=op, src=src: call("ctamd_%s_f32" % op, P(src[k]), P(R[k]), n, S), 8)
        ew("leaky_relu", lambda k: call("ctamd_leaky_relu_f32", P(A[k]), C.c_float(0.01), P(R[k]), n, S), 8)
        ew("tensor - scalar", lambda k: call("ctamd_sub_scalar_f32", P(A[k]), C.c_float(5.0), P(R[k]), n, S), 8)
        for op in ("abs", "sqrt", "square", "tan"):
            ew(op + " backward", lambda k, op=op: call("ctamd_%s_backward_f32" % op, P(B[k]), P(A[k]), P(R[k]), n, S), 12)
        ew("leaky_relu backward", lambda k: call("ctamd_leaky_relu_backward_f32", P(A[k]), P(B[k]), C.c_float(0.01), P(R[k]), n, S), 12)
        # ... reductions along an axis: a whole tensor, the rows and the columns of [16384 x 4096]
        small = torch.empty(16384, device="cuda")
        small_i = torch.empty(16384, dtype=torch.int32, device="cuda")
        small_m = torch.empty(16384, device="cuda")
        for kind, code in (("sum", 0), ("mean", 1), ("max", 2), ("min", 3), ("var", 4), ("std", 5)):
            for what, (o, l, i) in (("all", (1, n, 1)), ("rows of [16384 x 4096]", (16384, 4096, 1)), ("columns of [16384 x 4096]", (1, 16384, 4096))):
                if kind in ("mean", "min", "std") and what != "all":
                    continue
                ew("%s, %s" % (kind, what), lambda k, code=code, o=o, l=l, i=i: call("ctamd_reduce_dim_f32", code, P(A[k]), P(small), P(small_i),
                                                                                       P(small_m), o, l, i, 1, S), 4)
        for kind, code, per in (("sum", 0, 4), ("max", 2, 4), ("var", 4, 8)):
            for what, (o, l, i) in (("rows of [16384 x 4096]", (16384, 4096, 1)), ("columns of [16384 x 4096]", (1, 16384, 4096))):
                ew("%s backward, %s" % (kind, what), lambda k, code=code, o=o, l=l, i=i: call(
                    "ctamd_reduce_dim_backward_f32", code, P(A[k]), P(small), P(small_i), P(small_m), P(small), P(R[k]), o, l, i, 1, S), per)
        ew("log_softmax columns [16384 x 4096]", lambda k: call("ctamd_log_softmax_cols_f32", P(A[k]), P(R[k]), 16384, 4096, S), 8)
        ew("log_softmax rows [16384 x 4096]", lambda k: call("ctamd_log_softmax_rows_f32", P(A[k]), P(R[k]), 16384, 4096, S), 8)
        ew("log_softmax backward rows [16384 x 4096]", lambda k: call("ctamd_log_softmax_backward_rows_f32", P(A[k]), P(B[k]), P(R[k]), 16384, 4096, S), 12)
    if args.only_declared:
        del A, B, R
        torch.cuda.empty_cache()
        rows, cols = 8192, 32000
        X = torch.randn(rows, cols, device="cuda") * 2
        Y = torch.empty_like(X)
        report("log_softmax rows [8192 x 32000] (8 B/elem)", timeit(lambda: call("ctamd_log_softmax_rows_f32", P(X), P(Y), rows, cols, S), 10), 8 * rows * cols)
        report("log_softmax backward rows [8192 x 32000] (12 B/elem)",
               timeit(lambda: call("ctamd_log_softmax_backward_rows_f32", P(Y), P(X), P(Y), rows, cols, S), 10), 12 * rows * cols)
        if args.json:
            print(json.dumps({"device": torch.cuda.get_device_name(0), "results": results}))
        return 0
    # fused expressions: a cheap chain (bound by the memory stream) ...
    class Insn(C.Structure):
        _fields_ = [("op", C.c_uint8), ("dst", C.c_uint8), ("a", C.c_uint8), ("b", C.c_uint8), ("imm", C.c_float)]

    def program(*insns):
        return (Insn * len(insns))(*[Insn(*q) for q in insns]), len(insns)

    def run_expr(prog, ins, outs, rows, cols):
        pin = (C.c_void_p * len(ins))(*[t.data_ptr() for t in ins])
        pout = (C.c_void_p * len(outs))(*[t.data_ptr() for t in outs])
        call("ctamd_expr_run_f32", prog[0], prog[1], pin, len(ins), pout, len(outs), None, rows, cols, S)

    LOADF, LOADR, ADD, SUB, MUL, DIV, NEG, RELU, SIGM, TANH, SIN, COS, ADDS, STORE = 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 18
    chain = program((LOADF, 0, 0, 0, 0.0), (LOADF, 1, 1, 0, 0.0), (MUL, 0, 0, 1, 0.0), (ADDS, 0, 0, 0, 5.0), (RELU, 0, 0, 0, 0.0),
                    (STORE, 0, 0, 0, 0.0))
    bare = program((LOADF, 0, 0, 0, 0.0), (STORE, 0, 0, 0, 0.0))
    ew("fused load + store only", lambda k: run_expr(bare, [A[k]], [R[k]], 16384, 4096), 8)
    ew("fused relu(a * b + 5)", lambda k: run_expr(chain, [A[k], B[k]], [R[k]], 16384, 4096), 12)
    # the same launches over ONE buffer set (how a benchmark loop of the reference calls an operator):
    # nothing here fits the 256 MiB memory-side cache whole, but hinted streams leave it alone
    same = lambda name, fn, per: report("%s, n=2^26, one buffer set (%d B/elem)" % (name, per), timeit(lambda: fn(0), 20), per * n)
    same("add", lambda k: call("ctamd_add_f32", P(A[k]), P(B[k]), P(R[k]), n, S), 12)
    same("fused load + store only", lambda k: run_expr(bare, [A[k]], [R[k]], 16384, 4096), 8)
    same("fused relu(a * b + 5)", lambda k: run_expr(chain, [A[k], B[k]], [R[k]], 16384, 4096), 12)
    # ... and the config-5 expression sigmoid(X / r) - tanh(X) * sin(X) + cos(-X) (bound by its five transcendentals)
    c5 = program((LOADF, 0, 0, 0, 0.0), (LOADR, 1, 1, 0, 0.0), (DIV, 2, 0, 1, 0.0), (SIGM, 2, 2, 0, 0.0), (TANH, 3, 0, 0, 0.0),
                 (SIN, 4, 0, 0, 0.0), (MUL, 3, 3, 4, 0.0), (SUB, 2, 2, 3, 0.0), (NEG, 3, 0, 0, 0.0), (COS, 3, 3, 0, 0.0),
                 (ADD, 2, 2, 3, 0.0), (STORE, 0, 2, 0, 0.0))
    ew("fused sigmoid(X/r) - tanh(X)*sin(X) + cos(-X) [16384 x 4096]", lambda k: run_expr(c5, [A[k], B[0]], [R[k]], 16384, 4096), 8)
    # the rows above ran as kernels compiled for their programs (from the second launch on); the same
    # programs through the interpreter, for comparison
    jit = lib.ctamd_expr_jit()
    call("ctamd_set_expr_jit", 0)
    ew("interpreted relu(a * b + 5)", lambda k: run_expr(chain, [A[k], B[k]], [R[k]], 16384, 4096), 12)
    ew("interpreted sigmoid(X/r) - tanh(X)*sin(X) + cos(-X) [16384 x 4096]", lambda k: run_expr(c5, [A[k], B[0]], [R[k]], 16384, 4096), 8)
    call("ctamd_set_expr_jit", jit)
    if args.only_expr:
        if args.json:
            print(json.dumps({"device": torch.cuda.get_device_name(0), "results": results}))
        return 0
    # comparisons (bool out: 9 and 5 B/elem), pixel bytes to floats (5 B/elem), column softmax
    bout = torch.empty(n, dtype=torch.uint8, device="cuda")
    ew("a > b (bool tensor)", lambda k: call("ctamd_compare_f32", 0, P(A[k]), P(B[k]), P(bout), n, S), 9)
    ew("a > 0.25 (bool tensor)", lambda k: call("ctamd_compare_scalar_f32", 0, P(A[k]), C.c_float(0.25), P(bout), n, S), 5)
    ew("pixel bytes / 255", lambda k: call("ctamd_u8_to_unit_f32", P(bout), P(R[k]), n, S), 5)
    ew("softmax columns [16384 x 4096]", lambda k: call("ctamd_softmax_cols_f32", P(A[k]), P(R[k]), 16384, 4096, S), 8)
    ew("softmax backward columns [16384 x 4096]", lambda k: call("ctamd_softmax_backward_cols_f32", P(A[k]), P(B[k]), P(R[k]), 16384, 4096, S), 12)
    cs = torch.empty(4096, device="cuda")
    ew("column sum [16384 x 4096]", lambda k: call("ctamd_colsum_f32", P(A[k]), P(cs), 16384, 4096, S), 4)
    # tensors that are not fp32: conversion, scalar operators, accumulation (2^26 elements), double softmax
    D64 = [torch.empty(n, dtype=torch.float64, device="cuda").normal_() for _ in range(2)]
    I32 = [torch.randint(-1000, 1000, (n,), dtype=torch.int32, device="cuda") for _ in range(2)]
    ew("fp32 -> double", lambda k: call("ctamd_cast_from_f32", P(A[k]), P(D64[0]), 1, n, S), 12)
    ew("fp32 -> int32", lambda k: call("ctamd_cast_from_f32", P(A[k]), P(I32[0]), 2, n, S), 8)
    ew("double * 2.5f", lambda k: call("ctamd_scalar_op_typed", P(D64[k % 2]), P(D64[1 - k % 2]), 1, 1, C.c_float(2.5), n, S), 16)
    ew("int32 / 3.0f", lambda k: call("ctamd_scalar_op_typed", P(I32[k % 2]), P(I32[1 - k % 2]), 2, 2, C.c_float(3.0), n, S), 8)
    ew("double += double", lambda k: call("ctamd_accumulate_typed", P(D64[0]), P(D64[1]), 1, n, S), 24)
    ew("ones (double)", lambda k: call("ctamd_fill_typed", P(D64[0]), 1, C.c_double(1.0), n, S), 8)
    D64[0].normal_()
    ew("softmax rows, double [8192 x 8192]", lambda k: call("ctamd_softmax_f64", P(D64[0]), P(D64[1]), 8192, 8192, 1, S), 16)
    ew("softmax columns, double [8192 x 8192]", lambda k: call("ctamd_softmax_f64", P(D64[0]), P(D64[1]), 8192, 8192, 0, S), 16)
    del D64, I32
    del A, B, R
    torch.cuda.empty_cache()

    # ---- row softmax / cross entropy at [8192 x 32000]
    rows, cols = 8192, 32000
    m = rows * cols
    X = torch.randn(rows, cols, device="cuda") * 2
    Y = torch.empty_like(X)
    idx = torch.randint(0, cols, (rows,), device="cuda").float()
    g1 = torch.ones(1, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    stats = torch.empty(rows, 2, device="cuda")

    def row(name, fn, bytes_per_elem):
        report("%s [8192 x 32000] (%d B/elem)" % (name, bytes_per_elem), timeit(fn, 10), bytes_per_elem * m)

    row("softmax rows", lambda: call("ctamd_softmax_rows_f32", P(X), P(Y), rows, cols, S), 8)
    row("cross entropy (class index) forward", lambda: call("ctamd_cross_entropy_index_stats_f32", P(X), P(idx), P(out),
                                                            P(status), P(stats), rows, cols, S), 4)
    row("cross entropy (class index) backward", lambda: call("ctamd_cross_entropy_backward_index_f32", P(X), P(idx), P(g1),
                                                             P(Y), rows, cols, S), 8)
    row("cross entropy backward from forward statistics", lambda: call("ctamd_cross_entropy_backward_index_stats_f32", P(X),
                                                                       P(idx), P(stats), P(g1), P(Y), rows, cols, S), 8)
    row("cross entropy loss + gradient in one pass", lambda: call("ctamd_cross_entropy_index_fused_f32", P(X), P(idx), P(out),
                                                                  P(status), P(Y), rows, cols, S), 8)
    row("softmax backward rows", lambda: call("ctamd_softmax_backward_rows_f32", P(Y), P(X), P(Y), rows, cols, S), 12)
    del X, Y
    torch.cuda.empty_cache()
    # rows beyond what a block keeps in registers (more than 32768 columns): two sweeps per row
    rows, cols = 4096, 65536
    X = torch.randn(rows, cols, device="cuda") * 2
    Y = torch.empty_like(X)
    G2 = torch.randn(rows, cols, device="cuda")
    report("softmax rows [4096 x 65536] (8 B/elem)", timeit(lambda: call("ctamd_softmax_rows_f32", P(X), P(Y), rows, cols, S), 10), 8 * rows * cols)
    report("softmax backward rows [4096 x 65536] (12 B/elem)",
           timeit(lambda: call("ctamd_softmax_backward_rows_f32", P(Y), P(G2), P(X), rows, cols, S), 10), 12 * rows * cols)
    del X, Y, G2
    torch.cuda.empty_cache()

    if not args.skip_matmul:
        matmul_rows()
    if args.json:
        print(json.dumps({"device": torch.cuda.get_device_name(0), "results": results}))
    return 0


if __name__ == "__main__":
    sys.exit(main())

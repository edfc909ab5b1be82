"""Whole training steps of configurations 3 and 5 through the C++ front-end, a few repetitions each.

    python -m ctorch_amd.step_trace

Meant to be run under `rocprofv3 --kernel-trace`: the trace then shows which kernels one step
launches, in order, with their start times and durations (the dependent-launch gaps included).
Prints the front-end's own figure per step (host clock around a step that ends with reading the
loss) and its count of operator launches.  The steps are the ones bench.py reports: the
784-256-10 perceptron at batch 256 and 8192 with fused layers and the one-pass classifier head (class
indices uploaded from the host: the step reads no flag back), and the broadcast expression of configuration 5 as one fused
expression, inputs from the configurations' seeds.
"""
import ctypes as C
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_LIB = os.path.join(ROOT, "ctorch_amd", "host", "tests", "harness", "libctorch_amd_harness.so")


# untimed steps before the timed ones: some 40 ms of the same work, because the chip's clock keeps moving for
# about 25 ms after a change of load (up after idling, down and part of the way back under heavy vector work)
WARM_MLP, WARM_EXPR = 400, 150


def main():
    import numpy as np
    from ctorch_amd import rng
    if not os.path.exists(HOST_LIB):
        raise RuntimeError("%s is missing: run `make -C ctorch_amd/host`" % HOST_LIB)
    host = C.CDLL(HOST_LIB)
    host.cth_quiet()
    FP, L, I, D6 = C.POINTER(C.c_float), C.c_long, C.c_int, C.c_double * 6
    fp = lambda a: a.ctypes.data_as(FP)
    f32 = lambda a: np.ascontiguousarray(a, dtype=np.float32)
    W1, b1 = rng.uniform((784, 256), 311, -1 / 28.0, 1 / 28.0), rng.uniform(256, 312, -1 / 28.0, 1 / 28.0)
    W2, b2 = rng.uniform((256, 10), 313, -1 / 16.0, 1 / 16.0), rng.uniform(10, 314, -1 / 16.0, 1 / 16.0)
    host.cth_set_fused_layers(1)
    host.cth_set_fused_head(1)
    for batch in (256, 8192):
        x = f32(rng.ints((batch, 784), 301, 256) / np.float32(255.0))
        lab = rng.ints(batch, 302, 10)
        out = D6()
        rc = host.cth_time_mlp(fp(x), L(batch), L(784), fp(W1), fp(b1), L(256), fp(W2), fp(b2), L(10), fp(lab), I(WARM_MLP), I(20), out)
        assert rc >= 0
        print("MLP 784-256-10 step, batch %d, fused layers, one-pass head: %.1f us per step, %d operator launches" % (batch, out[0] * 1e3, round(out[4])), flush=True)
    host.cth_set_fused_layers(0)
    host.cth_set_fused_head(0)
    n = 4096
    X, rv, T = rng.uniform((n, n), 501, -2, 2), rng.uniform(n, 502, 0.5, 2), rng.normal((n, n), 503)
    host.cth_set_fused_expr(1)
    out = D6()
    rc = host.cth_time_expr(fp(X), fp(rv), fp(T), L(n), L(n), I(WARM_EXPR), I(20), out)
    assert rc >= 0
    host.cth_set_fused_expr(0)
    print("configuration 5 step [4096 x 4096], fused expression: %.1f us per step, %d operator launches" % (out[0] * 1e3, round(out[4])), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

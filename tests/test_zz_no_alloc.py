"""The entry point that allocates nothing: ctamd_dot_static_f32 keeps its per-block partial sums in
an array of the library's device image instead of the scratch buffer ctamd_init() allocates.  It
runs the kernels of ctamd_dot_f32 on the same grid, so the two must agree bit for bit; two calls in
a row (the second on a smaller input) share the array and must not see each other's partials."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _dot(G, name, a, b):
    import torch
    out = torch.full((1,), float("nan"), device=G.DEV)
    G.call(name, G.ptr(a), G.ptr(b), G.ptr(out), a.numel(), G.stream())
    return G.host(out).copy()


def _free_device_bytes(lib):
    """hipMemGetInfo of the HIP runtime the library itself is bound to (its symbols are reachable
    through the library's handle): what any allocation by the call, torch's or hipMalloc's, would lower."""
    fn = lib.hipMemGetInfo
    fn.argtypes, fn.restype = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)], C.c_int
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert fn(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_dot_equals_dot_on_two_calls_in_a_row():
    import gpu_support as G
    import torch
    from support import Oracle
    o = Oracle()
    lib = G.lib()
    sizes = [(1 << 22) + 3, 4099]            # 1025 blocks with a ragged tail, then a 2-block input
    for k, n in enumerate(sizes):
        a_h, b_h = o.uniform((n,), 211 + 10 * k, -1, 1), o.uniform((n,), 212 + 10 * k, -1, 1)
        a, b = G.dev(a_h), G.dev(b_h)
        out = torch.full((1,), float("nan"), device=G.DEV)
        torch.cuda.synchronize()
        before, before_torch = _free_device_bytes(lib), torch.cuda.memory_reserved()
        G.call("ctamd_dot_static_f32", G.ptr(a), G.ptr(b), G.ptr(out), a.numel(), G.stream())
        torch.cuda.synchronize()
        # the call took no device memory: neither from the driver nor from torch's pool
        assert _free_device_bytes(lib) == before and torch.cuda.memory_reserved() == before_torch
        got = G.host(out).copy()
        want = _dot(G, "ctamd_dot_f32", a, b)
        assert got.view(np.uint32)[0] == want.view(np.uint32)[0], (n, got, want)
        # and both within the reduction bar of an fp64 dot product
        exact = float(np.dot(a_h.astype(np.float64), b_h.astype(np.float64)))
        scale = float(np.sum(np.abs(a_h.astype(np.float64) * b_h.astype(np.float64))))
        assert abs(float(got[0]) - exact) <= 1e-5 * scale
        # the oracle's sequential fp32 dot product is inside the same bar
        assert abs(float(o.dot(a_h, b_h)) - float(got[0])) <= 2e-5 * scale


def test_static_dot_edges_and_limit():
    import gpu_support as G
    import torch
    l = G.lib()
    a = G.dev(np.arange(1, 8, dtype=np.float32))
    b = G.dev(np.full(7, 0.5, np.float32))
    assert _dot(G, "ctamd_dot_static_f32", a, b)[0] == np.float32(14.0)         # unaligned-length tail path
    assert _dot(G, "ctamd_dot_static_f32", a[1:], b[1:])[0] == np.float32(13.5)  # operands off a 16-byte boundary
    out = torch.full((1,), 5.0, device=G.DEV)
    assert l.ctamd_dot_static_f32(None, None, G.ptr(out), 0, G.stream()) == 0    # empty: the sum of nothing
    assert G.host(out)[0] == 0.0
    too_many = C.c_size_t((1 << 31))
    assert l.ctamd_dot_static_f32(G.ptr(a), G.ptr(b), G.ptr(out), too_many, G.stream()) == -5
    assert b"exceed the supported maximum" in l.ctamd_last_error()
    assert l.ctamd_dot_static_f32(None, G.ptr(b), G.ptr(out), 7, G.stream()) == -1

"""The library's one device scratch (partials of reductions, losses, column softmax, parts of split
matrix products) serves one stream at a time: a second stream is refused while the first has such
work pending, accepted once the first is idle, and the null stream and blocking streams - which
order themselves with each other - alternate freely."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
import gpu_support as G  # noqa: E402

pytestmark = pytest.mark.gpu


def test_a_second_stream_is_refused_the_scratch_while_the_first_is_busy(oracle):
    print("case scratch claim", flush=True)
    L = G.lib()
    n = 1 << 26
    a = torch.ones(n, device=G.DEV)
    b = torch.full((n,), 0.5, device=G.DEV)
    small = G.dev(oracle.uniform((4096,), 71, -1, 1))
    out1 = torch.zeros((), device=G.DEV)
    out2 = torch.zeros((), device=G.DEV)
    torch.cuda.synchronize()
    s1, s2 = C.c_void_p(), C.c_void_p()
    assert L.ctamd_stream_create(C.byref(s1)) == 0 and L.ctamd_stream_create(C.byref(s2)) == 0
    try:
        for _ in range(40):                                   # a few milliseconds of reductions pending on s1
            assert L.ctamd_dot_f32(G.ptr(a), G.ptr(b), G.ptr(out1), n, s1) == 0
        rc = L.ctamd_sum_f32(G.ptr(small), G.ptr(out2), small.numel(), s2)
        msg = L.ctamd_last_error().decode()
        assert L.ctamd_sync(s1) == 0
        assert rc != 0 and "scratch" in msg, (rc, msg)
        # the first stream is idle now: the second may take over, and the null stream may follow it
        assert L.ctamd_sum_f32(G.ptr(small), G.ptr(out2), small.numel(), s2) == 0
        assert L.ctamd_sync(s2) == 0
        want = np.float32(np.sum(G.host(small), dtype=np.float64))   # the kernel adds in double precision
        assert np.float32(out2.item()) == want
        assert L.ctamd_sum_f32(G.ptr(small), G.ptr(out2), small.numel(), None) == 0
        assert L.ctamd_sum_f32(G.ptr(small), G.ptr(out1), small.numel(), s2) == 0   # blocking stream after the null stream: ordered
        assert L.ctamd_sync(None) == 0 and L.ctamd_sync(s2) == 0
        assert np.float32(out1.item()) == want and np.float32(out2.item()) == want
        assert float(n) * 0.5 == 33554432.0
    finally:
        L.ctamd_sync(s1)
        L.ctamd_sync(s2)
        L.ctamd_stream_destroy(s1)
        L.ctamd_stream_destroy(s2)

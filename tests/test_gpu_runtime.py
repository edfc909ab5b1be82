"""The library's one device scratch (partials of reductions, losses, column softmax, parts of split
matrix products) serves every stream of a device: a stream other than the previous user is made to
wait, on the device, for the previous user's scratch-using work (an event the library records after
that work), so results stay right when streams that do not order themselves interleave such calls."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
import gpu_support as G  # noqa: E402

pytestmark = pytest.mark.gpu


def test_streams_that_share_the_scratch_are_put_in_order(oracle):
    print("case scratch ordering", flush=True)
    L = G.lib()
    n = 1 << 26
    a = torch.ones(n, device=G.DEV)
    b = torch.full((n,), 0.5, device=G.DEV)
    small = G.dev(oracle.uniform((4096,), 71, -1, 1))
    want_small = np.float32(np.sum(G.host(small), dtype=np.float64))   # the kernel adds in double precision
    out1 = torch.zeros(48, device=G.DEV)
    out2 = torch.zeros(48, device=G.DEV)
    torch.cuda.synchronize()
    s1, s2 = C.c_void_p(), C.c_void_p()
    assert L.ctamd_stream_create(C.byref(s1)) == 0 and L.ctamd_stream_create(C.byref(s2)) == 0
    nb = torch.cuda.Stream()                                   # a non-blocking stream the library does not own
    s3 = C.c_void_p(nb.cuda_stream)
    one = lambda t, k: C.c_void_p(t.data_ptr() + 4 * k)
    try:
        # a long reduction on one stream, a short one on another right behind it, without any host wait:
        # unordered, the second would overwrite the partials the first is still folding
        for k in range(40):
            assert L.ctamd_dot_f32(G.ptr(a), G.ptr(b), one(out1, k), n, s1) == 0
            assert L.ctamd_sum_f32(G.ptr(small), one(out2, k), small.numel(), s2 if k % 2 else s3) == 0, L.ctamd_last_error()
        assert L.ctamd_sum_f32(G.ptr(small), one(out2, 40), small.numel(), None) == 0        # the null stream joins in
        assert L.ctamd_dot_f32(G.ptr(a), G.ptr(b), one(out1, 40), n, s3) == 0
        assert L.ctamd_sum_f32(G.ptr(small), one(out2, 41), small.numel(), s1) == 0
        for s in (s1, s2, s3, None):
            assert L.ctamd_sync(s) == 0
        assert (G.host(out1)[:41] == np.float32(n * 0.5)).all(), G.host(out1)
        assert (G.host(out2)[:42] == want_small).all(), G.host(out2)
    finally:
        for s in (s1, s2, s3, None):
            L.ctamd_sync(s)
        L.ctamd_stream_destroy(s1)
        L.ctamd_stream_destroy(s2)


def test_a_destroyed_foreign_stream_is_never_touched_again(oracle):
    """The previous user of the scratch may be a stream its owner has destroyed since: the next claim
    waits on the library's own event, not on that handle."""
    print("case scratch stale stream", flush=True)
    L = G.lib()
    x = G.dev(oracle.uniform((1 << 20,), 72, -1, 1))
    want = np.float32(np.sum(G.host(x), dtype=np.float64))
    out = torch.zeros(4, device=G.DEV)
    torch.cuda.synchronize()
    one = lambda k: C.c_void_p(out.data_ptr() + 4 * k)
    raw = C.c_void_p()
    assert L.ctamd_stream_create(C.byref(raw)) == 0
    assert L.ctamd_sum_f32(G.ptr(x), one(0), x.numel(), raw) == 0
    assert L.ctamd_sync(raw) == 0
    destroy = L.hipStreamDestroy                                # the HIP runtime the library itself is bound to
    destroy.argtypes, destroy.restype = [C.c_void_p], C.c_int
    assert destroy(raw) == 0                                    # destroyed behind the library's back
    s2 = C.c_void_p()
    assert L.ctamd_stream_create(C.byref(s2)) == 0
    try:
        assert L.ctamd_sum_f32(G.ptr(x), one(1), x.numel(), s2) == 0, L.ctamd_last_error()
        assert L.ctamd_sum_f32(G.ptr(x), one(2), x.numel(), None) == 0
        assert L.ctamd_sync(s2) == 0 and L.ctamd_sync(None) == 0
        assert (G.host(out)[:3] == want).all()
    finally:
        L.ctamd_stream_destroy(s2)


def test_small_reads_land_behind_the_queued_work(oracle):
    """ctamd_read_small: a few bytes read after the work queued on a stream, through the page-locked buffer
    the library keeps per host thread - the value of the kernel launched just before, from several host
    threads, and the refusals."""
    print("case small reads", flush=True)
    import threading
    L = G.lib()
    a = G.dev(oracle.uniform((1 << 20,), 73, -1, 1))
    b = G.dev(oracle.uniform((1 << 20,), 74, -1, 1))
    out = torch.zeros(4, device=G.DEV)
    want = np.float32(np.dot(G.host(a).astype(np.float64), G.host(b).astype(np.float64)))
    got = (C.c_float * 4)()
    for _ in range(5):
        out.zero_()
        G.call("ctamd_dot_f32", G.ptr(a), G.ptr(b), G.ptr(out), 1 << 20, G.stream())
        assert L.ctamd_read_small(got, G.ptr(out), 16, G.stream()) == 0
        assert abs(got[0] - want) <= 1e-6 * abs(want) + 1e-6 and got[1] == 0.0
    raw = torch.arange(64, dtype=torch.float32, device=G.DEV)
    wide = (C.c_float * 64)()
    assert L.ctamd_read_small(wide, G.ptr(raw), 256, G.stream()) == 0 and list(wide) == [float(i) for i in range(64)]
    assert L.ctamd_read_small(wide, G.ptr(raw), 0, G.stream()) == 0
    assert L.ctamd_read_small(wide, G.ptr(torch.zeros(128, device=G.DEV)), 260, G.stream()) == -5
    assert L.ctamd_read_small(None, G.ptr(raw), 4, G.stream()) == -1 and L.ctamd_read_small(wide, None, 4, G.stream()) == -1
    torch.cuda.synchronize()
    # every host thread has a landing buffer of its own
    results = {}

    def worker(i):
        mine = (C.c_float * 1)()
        ok = all(L.ctamd_read_small(mine, C.c_void_p(raw.data_ptr() + 4 * i), 4, G.stream()) == 0 and mine[0] == float(i) for _ in range(50))
        results[i] = ok

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(1, 5)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert results == {1: True, 2: True, 3: True, 4: True}

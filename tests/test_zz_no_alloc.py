"""apk_argmax_rows_noalloc (the entry that allocates nothing: its scratch is a static device array of the library)
against apk_argmax_rows, through the C ABI: two calls in a row, the second with a smaller input; then beyond the
array's 2048 rows (declined) and inside a recording."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_noalloc_argmax_matches_the_allocating_entry():
    import torch

    import allpaka_amd.lib as lib
    import oracle as ora

    ora.build()
    L = lib.load()
    h = C.c_void_p()
    lib.check(L.apk_init(0, C.byref(h)))
    try:
        g = np.random.default_rng(20)

        def run(rows, n, plant_ties):
            x = g.standard_normal((rows, n)).astype(np.float32)
            if plant_ties:  # equal maxima: the last one wins
                for r in range(rows):
                    m = np.float32(x[r].max() + 1.0)
                    x[r, g.integers(0, n, size=3)] = m
            x[0, : min(4, n)] = np.array([-0.0, 0.0, np.nan, -np.inf][: min(4, n)], np.float32)
            dx = torch.from_numpy(x).cuda()
            a = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
            b = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
            lib.check(L.apk_argmax_rows(h, dx.data_ptr(), rows, n, a.data_ptr()))
            lib.check(L.apk_argmax_rows_noalloc(h, dx.data_ptr(), rows, n, b.data_ptr()))
            lib.check(L.apk_sync(h))
            want = np.array([ora.argmax_last(x[r]) for r in range(rows)], np.uint32)
            assert np.array_equal(a.cpu().numpy().view(np.uint32), want)
            assert np.array_equal(b.cpu().numpy().view(np.uint32), want), (rows, n)

        run(64, 151936, True)   # the benchmark's shape: 19 parts per row
        run(5, 1000, False)     # right after it, a smaller input on the same scratch lines
        run(2048, 4096, True)   # the array's last row
        run(1, 151937, False)   # a ragged row (element-wise path)
        # beyond the static array: declined, nothing launched
        big = torch.zeros((2049, 8), device="cuda")
        out = torch.zeros(2049, dtype=torch.int32, device="cuda")
        assert L.apk_argmax_rows_noalloc(h, big.data_ptr(), 2049, 8, out.data_ptr()) == lib.DECLINE_SHAPE
        assert b"2048" in L.apk_last_error()
        # inside a recording (where the allocating entry may have to decline), replayed twice
        x = g.standard_normal((300, 5000)).astype(np.float32)
        dx = torch.from_numpy(x).cuda()
        o = torch.zeros(300, dtype=torch.int32, device="cuda")
        gr = C.c_void_p()
        lib.check(L.apk_capture_begin(h))
        lib.check(L.apk_argmax_rows_noalloc(h, dx.data_ptr(), 300, 5000, o.data_ptr()))
        lib.check(L.apk_capture_end(h, C.byref(gr)))
        for _ in range(2):
            o.fill_(-1)
            torch.cuda.synchronize()
            lib.check(L.apk_graph_launch(h, gr))
            lib.check(L.apk_sync(h))
            assert np.array_equal(o.cpu().numpy().view(np.uint32), np.array([ora.argmax_last(x[r]) for r in range(300)], np.uint32))
        lib.check(L.apk_graph_destroy(h, gr))
    finally:
        L.apk_shutdown(h)

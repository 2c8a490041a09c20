"""Calls from several host threads: one context serialises them on its mutex (the reference's
process-wide `static GPU: OnceLock<Option<Mutex<..>>>`, gpu/cuda/runtime/device.rs:267), and
separate contexts are independent.  ctypes releases the GIL around every call, so the threads
really do meet inside the library."""
import ctypes as C
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _worker(L, h, bufs, iters, errors, idx):
    try:
        x, d, hh, g, gate, up = bufs
        n = g.numel()
        for _ in range(iters):
            rc = L.apk_add_rmsnorm_rows(h, x.data_ptr(), d.data_ptr(), hh.data_ptr(), g.data_ptr(), n, x.numel() // n, 1e-6, 0)
            rc |= L.apk_swiglu(h, gate.data_ptr(), up.data_ptr(), gate.numel(), 0)
            if rc:
                errors.append((idx, rc))
                return
        if L.apk_sync(h):
            errors.append((idx, "sync"))
    except Exception as e:  # pragma: no cover
        errors.append((idx, repr(e)))


def _expected(x, d, g, gate, up, iters):
    """the same chain on one thread with torch (float64 statistics like the device's f32 path)"""
    x = x.clone()
    gate = gate.clone()
    for _ in range(iters):
        x = x + d
        gate = (gate / (1 + torch.exp(-gate))) * up
    ms = (x.double() ** 2).mean(dim=1, keepdim=True)
    h = ((x.double() / torch.sqrt(ms + 1e-6)).float()) * g
    return x, h, gate


@pytest.mark.parametrize("shared_context", [True, False])
def test_four_threads(shared_context):
    import allpaka_amd.lib as apklib

    L = apklib.load()
    n_threads, iters = 4, 60
    ctxs = []
    for _ in range(1 if shared_context else n_threads):
        h = C.c_void_p()
        apklib.check(L.apk_init(0, C.byref(h)))
        ctxs.append(h)
    gen = torch.Generator(device="cuda").manual_seed(7)
    bufs, want = [], []
    for t in range(n_threads):
        rows, n = 3 + t, 1024
        x = torch.randn((rows, n), generator=gen, device="cuda")
        d = torch.randn((rows, n), generator=gen, device="cuda") * 0.01
        g = 1 + 0.05 * torch.randn(n, generator=gen, device="cuda")
        gate = torch.randn(5000 + t, generator=gen, device="cuda") * 0.5
        up = torch.full_like(gate, 1.01)
        want.append(_expected(x, d, g, gate, up, iters))
        bufs.append((x, d, torch.empty_like(x), g, gate, up))
    torch.cuda.synchronize()
    errors = []
    threads = [threading.Thread(target=_worker, args=(L, ctxs[0 if shared_context else t], bufs[t], iters, errors, t))
               for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=60)
    assert not any(th.is_alive() for th in threads), "a thread is stuck inside the library"
    assert not errors, errors
    for h in ctxs:
        apklib.check(L.apk_sync(h))
    for t in range(n_threads):
        x, d, hh, g, gate, up = bufs[t]
        wx, wh, wg = want[t]
        assert torch.equal(x, wx)  # 60 exact f32 additions in the same order
        assert torch.allclose(hh, wh, rtol=1e-5, atol=1e-6)
        assert torch.allclose(gate, wg, rtol=2e-4, atol=1e-6)  # 60 chained SwiGLUs: rounding compounds
    calls = C.c_uint64()
    L.apk_stats(ctxs[0], C.byref(calls), None, None, None)
    assert calls.value >= (n_threads if shared_context else 1) * iters * 2
    for h in ctxs:
        apklib.check(L.apk_shutdown(h))

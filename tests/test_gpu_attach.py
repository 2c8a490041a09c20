"""The ownership boundary through the C ABI: weights named by host address inside an attached mapping
(gpu::attach / detach, gpu/stub.rs:37-41; resolve_w, gpu/cuda/runtime/select.rs:80-84; owner counting and
sub-ranges, gpu/cuda/runtime/device.rs:588-621).  The idiom of the reference's own parity test: the same bytes
opened twice, once inside the attached region (device path) and once as a heap copy (foreign memory, declined:
crates/allpaka-backend/tests/gpu_parity.rs:139-208)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _addr(a):
    return a.ctypes.data


def test_attach_resolve_run_detach():
    import torch

    import allpaka_amd.lib as lib
    import oracle as ora
    from allpaka_amd import synth

    ora.build()
    L = lib.load()
    h = C.c_void_p()
    lib.check(L.apk_init(0, C.byref(h)))
    NOT_ATTACHED, SHAPE, CAPTURE = lib.DECLINE_NOT_ATTACHED, lib.DECLINE_SHAPE, lib.DECLINE_CAPTURE
    try:
        # a "model file" on the host: a Q4_K embedding table [512 x 5120], then f32 norm weights [5120], 64-byte aligned
        g = synth.rng(2, 77)
        vocab, H, eps = 512, 5120, 1e-6
        table = synth.q4_k_table(g, vocab, H).reshape(-1)
        gamma = synth.normal_f32(g, H, 1.0, 0.05)
        off_gamma = (table.nbytes + 63) // 64 * 64
        mapping = np.zeros(off_gamma + gamma.nbytes + 100, np.uint8)
        mapping[: table.nbytes] = table
        mapping[off_gamma : off_gamma + gamma.nbytes] = gamma.view(np.uint8)
        base, total = _addr(mapping), mapping.nbytes
        owners = C.c_size_t()

        def n_owners(p, n):
            lib.check(L.apk_attached_owners(h, p, n, C.byref(owners)))
            return owners.value

        dev = C.c_void_p()
        assert L.apk_resolve(h, base, 16, C.byref(dev)) == NOT_ATTACHED and dev.value is None  # nothing attached yet
        assert L.apk_detach(h, base) == NOT_ATTACHED
        lib.check(L.apk_attach(h, base, total))
        assert n_owners(base, total) == 1
        lib.check(L.apk_attach(h, base, total))  # the same mapping again: one more owner, no second copy
        assert n_owners(base, total) == 2
        lib.check(L.apk_attach(h, base + 4096, 1000))  # a range inside it: fine, not counted
        assert n_owners(base, total) == 2 and n_owners(base + 4096, 1000) == 0
        assert L.apk_attach(h, base + 4096, total) == SHAPE  # runs off the end of the attached mapping
        assert L.apk_attach(h, base - 64, 128) == SHAPE      # straddles its start
        assert b"overlaps" in L.apk_last_error()

        # interior addresses -> device addresses; the ops run on them
        d_table, d_gamma = C.c_void_p(), C.c_void_p()
        lib.check(L.apk_resolve(h, base, table.nbytes, C.byref(d_table)))
        lib.check(L.apk_resolve(h, base + off_gamma, gamma.nbytes, C.byref(d_gamma)))
        assert d_gamma.value - d_table.value == off_gamma
        ids = np.array([0, vocab - 1, 3, 3, 117, 256], np.uint32)
        t = len(ids)
        d_ids = torch.from_numpy(ids.view(np.int32)).cuda()
        rows = torch.empty((t, H), device="cuda")
        lib.check(L.apk_embed_rows(h, lib.FMT_Q4K, d_table, vocab, H, d_ids.data_ptr(), t, rows.data_ptr(), lib.F32))
        hs = torch.empty((t, H), device="cuda")
        x = torch.zeros((t, H), device="cuda")
        lib.check(L.apk_add_rmsnorm_rows(h, x.data_ptr(), rows.data_ptr(), hs.data_ptr(), d_gamma, H, t, eps, lib.F32))
        lib.check(L.apk_sync(h))
        want_rows = ora.embed_rows(table, ora.FMT["Q4K"], vocab, H, ids)
        assert np.array_equal(rows.cpu().numpy(), want_rows)  # bit-exact from the attached copy
        wx, wh = np.zeros((t, H), np.float32), np.zeros((t, H), np.float32)
        ora.add_rmsnorm_rows(wx, want_rows, wh, gamma, eps)
        assert np.array_equal(x.cpu().numpy(), wx)
        assert np.allclose(hs.cpu().numpy(), wh, rtol=1e-5, atol=1e-7)

        # foreign memory: the same bytes on the heap, a range that runs off the end, a range before the start
        heap_copy = mapping.copy()
        assert L.apk_resolve(h, _addr(heap_copy), 16, C.byref(dev)) == NOT_ATTACHED and dev.value is None
        assert L.apk_resolve(h, base + total - 8, 16, C.byref(dev)) == NOT_ATTACHED
        assert L.apk_resolve(h, base - 8, 16, C.byref(dev)) == NOT_ATTACHED
        lib.check(L.apk_resolve(h, base + total, 0, C.byref(dev)))  # the empty range at the very end is inside

        # owners: two attaches need two detaches; a wrong length is another key
        assert L.apk_detach_range(h, base, total - 1) == NOT_ATTACHED
        lib.check(L.apk_detach_range(h, base, total))
        assert n_owners(base, total) == 1
        lib.check(L.apk_resolve(h, base, 16, C.byref(dev)))  # still resident
        # a recorded graph bakes in device addresses; attach and detach cannot run inside a recording
        gr = C.c_void_p()
        lib.check(L.apk_capture_begin(h))
        assert L.apk_attach(h, base, total) == CAPTURE and L.apk_detach(h, base) == CAPTURE  # not inside a recording
        lib.check(L.apk_embed_rows(h, lib.FMT_Q4K, d_table, vocab, H, d_ids.data_ptr(), t, rows.data_ptr(), lib.F32))
        lib.check(L.apk_capture_end(h, C.byref(gr)))
        rows.zero_()
        torch.cuda.synchronize()
        lib.check(L.apk_graph_launch(h, gr))
        lib.check(L.apk_sync(h))
        assert np.array_equal(rows.cpu().numpy(), want_rows)  # the mapping is still there
        # a graph recorded before the mapping was attached again below is untouched by that mapping's detach
        early = C.c_void_p()
        hs.zero_()
        x.zero_()
        lib.check(L.apk_capture_begin(h))
        lib.check(L.apk_swiglu(h, hs.data_ptr(), x.data_ptr(), hs.numel(), lib.F32))
        lib.check(L.apk_capture_end(h, C.byref(early)))
        lib.check(L.apk_detach(h, base))  # the last owner: the device copy goes, with the graphs alive
        assert n_owners(base, total) == 0
        assert L.apk_resolve(h, base, 16, C.byref(dev)) == NOT_ATTACHED and dev.value is None
        assert L.apk_detach(h, base) == NOT_ATTACHED
        assert L.apk_detach(h, _addr(heap_copy)) == NOT_ATTACHED  # never attached
        # both graphs were recorded while the mapping was attached: they hold its freed addresses (or may) and are
        # never replayed again -- declined, nothing launched (the reference drops its graphs here, device.rs:604-621)
        rows.fill_(-1.0)
        torch.cuda.synchronize()
        assert L.apk_graph_launch(h, gr) == NOT_ATTACHED and b"record it again" in L.apk_last_error()
        assert L.apk_graph_launch(h, early) == NOT_ATTACHED
        lib.check(L.apk_sync(h))
        assert float(rows.min()) == -1.0 and float(rows.max()) == -1.0
        # a new mapping at the same host address gets a fresh copy (the reason detach must free: gpu/cuda/mod.rs:51-54):
        # changed bytes are what runs, and the stale graph stays stale
        mapping[: table.nbytes] = synth.q4_k_table(g, vocab, H).reshape(-1)
        lib.check(L.apk_attach(h, base, total))
        lib.check(L.apk_resolve(h, base, table.nbytes, C.byref(d_table)))
        lib.check(L.apk_embed_rows(h, lib.FMT_Q4K, d_table, vocab, H, d_ids.data_ptr(), t, rows.data_ptr(), lib.F32))
        lib.check(L.apk_sync(h))
        new_rows = ora.embed_rows(mapping[: table.nbytes], ora.FMT["Q4K"], vocab, H, ids)
        assert np.array_equal(rows.cpu().numpy(), new_rows) and not np.array_equal(new_rows, want_rows)
        assert L.apk_graph_launch(h, gr) == NOT_ATTACHED
        # a graph recorded now replays; one recorded before an unrelated, later mapping came and went does too
        fresh = C.c_void_p()
        lib.check(L.apk_capture_begin(h))
        lib.check(L.apk_embed_rows(h, lib.FMT_Q4K, d_table, vocab, H, d_ids.data_ptr(), t, rows.data_ptr(), lib.F32))
        lib.check(L.apk_capture_end(h, C.byref(fresh)))
        other = np.zeros(4096, np.uint8)
        lib.check(L.apk_attach(h, _addr(other), other.nbytes))
        lib.check(L.apk_detach(h, _addr(other)))  # attached after `fresh` was recorded: cannot be inside it
        rows.zero_()
        torch.cuda.synchronize()
        lib.check(L.apk_graph_launch(h, fresh))
        lib.check(L.apk_sync(h))
        assert np.array_equal(rows.cpu().numpy(), new_rows)
        for gx in (gr, early, fresh):
            lib.check(L.apk_graph_destroy(h, gx))
        lib.check(L.apk_detach(h, base))
    finally:
        L.apk_shutdown(h)


def test_host_mirror_names_weights_by_host_address():
    """The same through the host-side mirror: Backend.attach / resolve / detach and QuantMat.from_mapping."""
    import torch

    import allpaka_amd as apk
    import oracle as ora
    from allpaka_amd import synth

    ora.build()
    be = apk.Backend(0)
    try:
        g = synth.rng(0, 78)
        vocab, H = 300, 1024
        mapping = np.zeros(vocab * 1088 + 4096, np.uint8)
        table = synth.q8_0_table(g, vocab, H).reshape(-1)
        mapping[64 : 64 + table.nbytes] = table
        view = mapping[64 : 64 + table.nbytes]
        with pytest.raises(apk.Declined):  # not attached yet: foreign memory
            apk.QuantMat.from_mapping(be, view, apk.GgmlType.Q8_0, vocab, H)
        assert be.attach(mapping) and be.attach(mapping) and be.owners(mapping) == 2
        qm = apk.QuantMat.from_mapping(be, view, apk.GgmlType.Q8_0, vocab, H)
        assert be.resolve(view) == be.resolve(mapping) + 64 and be.resolve(view.copy()) is None
        ids = np.array([299, 0, 41], np.uint32)
        out = torch.empty((3, H), device="cuda")
        qm.rows_into(torch.from_numpy(ids.view(np.int32)).cuda(), out)
        assert np.array_equal(out.cpu().numpy(), ora.embed_rows(table, ora.FMT["Q8_0"], vocab, H, ids))
        assert np.array_equal(qm.row(299).cpu().numpy(), ora.embed_rows(table, ora.FMT["Q8_0"], vocab, H, ids[:1])[0])
        with pytest.raises(ValueError):
            apk.QuantMat.from_mapping(be, view[:-1], apk.GgmlType.Q8_0, vocab, H)
        assert be.detach(mapping) and be.detach(mapping)
        assert not be.detach(mapping)  # silent, as the reference
        assert be.owners(mapping) == 0 and be.resolve(view) is None
        # the QuantMat borrowed its bytes and holds no owner: with the mapping gone every call declines, nothing launches
        d0 = be.stats()[1]
        out.fill_(7.0)
        for call in (lambda: qm.row(0), lambda: qm.rows_into(torch.from_numpy(ids.view(np.int32)).cuda(), out),
                     lambda: qm.dequant_rows(0, 2)):
            with pytest.raises(apk.Declined):
                call()
        assert be.stats()[1] == d0 and float(out.min()) == 7.0
        # attached again (new bytes at the same address): the same QuantMat reads the new copy
        table2 = synth.q8_0_table(g, vocab, H).reshape(-1)
        mapping[64 : 64 + table.nbytes] = table2
        assert be.attach(mapping)
        qm.rows_into(torch.from_numpy(ids.view(np.int32)).cuda(), out)
        assert np.array_equal(out.cpu().numpy(), ora.embed_rows(table2, ora.FMT["Q8_0"], vocab, H, ids))
        assert be.detach(mapping)
    finally:
        be.close()
